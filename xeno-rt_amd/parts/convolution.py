"""Short causal convolutions over time, one filter per channel, and the interpolation of a token with the one before it.

Both look a few tokens back along the sequence, so a sequence keeps its last inputs as state: [taps - 1, channels]
float32 for every sequence, zeros when it starts. The arithmetic is float32; the result has the compute dtype.
"""
from __future__ import annotations

from typing import Dict, Sequence, Tuple

import torch

from .base import CacheNeeds, Part, Runtime, StateSpec, WeightSpec


class ShortConvolution(Part):
    """y[t] = sum_j w[:, j] * u[t - taps + 1 + j] on every channel, zeros before the sequence's start; with
    plus_input the result is u + y. `names` are the filters' tensors ([channels_i, taps] each), side by side along
    the channels in the order given (so one pass serves the q, k and v of an attention). `bias_names`: a tensor [channels_i]
    beside every filter, added to the sum; `activation` ("silu") is applied last. The inputs may be float32 beside a
    compute dtype of bfloat16 (a product's sums): the state then keeps them unrounded, and the result is rounded once."""
    capturable = True

    def __init__(self, names: Sequence[str], channels: Sequence[int], taps: int, state_name: str, plus_input: bool = False,
                 bias_names: Sequence[str] = (), activation=None):
        if taps < 1:
            raise ValueError(f"a convolution over time needs at least one tap, found {taps}")
        self.names, self.channel_counts = list(names), [int(c) for c in channels]
        self.channels = sum(self.channel_counts)
        self.taps = int(taps)
        self.state_name = state_name
        self.plus_input = plus_input
        self.bias_names, self.activation = list(bias_names), activation
        if self.bias_names and len(self.bias_names) != len(self.names):
            raise ValueError("a convolution's biases come one for every filter")
        self.weight = self.bias = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {name: WeightSpec((count, self.taps), kind="vector") for name, count in zip(self.names, self.channel_counts)}
        specs.update({name: WeightSpec((count,), init="zeros", kind="vector") for name, count in zip(self.bias_names, self.channel_counts)})
        return specs

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.taps - 1, self.channels))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = torch.cat([runtime.vector(tensors[name]) for name in self.names]).contiguous()
        if self.bias_names:
            self.bias = torch.cat([runtime.vector(tensors[name]) for name in self.bias_names]).to(self.weight.dtype).contiguous()

    def forward(self, u: torch.Tensor, batch, cache) -> torch.Tensor:
        out = self.runtime.empty((u.shape[0], self.channels))
        extra = {} if self.bias is None and self.activation is None else {"bias": self.bias, "activation": self.activation}
        self.runtime.ops.short_conv(u, self.weight, cache.states[self.state_name], batch, out,
                                    mode="plus_input" if self.plus_input else "plain", **extra)
        return out


    def forward_normed(self, x: torch.Tensor, norm, batch, cache) -> torch.Tensor:
        """This convolution of norm(x). Where every sequence brings one token and the norm is a plain RMSNorm over whole
        rows, one kernel does both (to the same bits as the two would)."""
        rt = self.runtime
        scale = norm.row_scale()
        fused = getattr(rt.ops, "rmsnorm_conv_step", None)
        if (fused is None or scale is None or len(self.names) != 1 or self.bias is not None or self.activation is not None or int(batch.max_count) != 1
                or int(batch.n_tokens) != int(batch.n_sequences) or x.shape[1] != self.channels or self.taps > 8):
            return self.forward(norm.forward(x), batch, cache)
        out = rt.empty((x.shape[0], self.channels))
        fused(x, scale[0], scale[1], self.weight, cache.states[self.state_name], batch, out, plus_input=self.plus_input)
        return out


class TokenShift(Part):
    """For each of several readers its own mix of a token and the one before it: u + (u[t - 1] - u) * mu, with
    mu [channels] per reader and zeros before the sequence's start. Returns [readers, tokens, channels], or with
    `single` (one reader) [tokens, channels]: so it can stand as a sublayer's input transform."""
    capturable = True

    def __init__(self, names: Sequence[str], channels: int, state_name: str, single: bool = False):
        self.names, self.channels, self.state_name = list(names), int(channels), state_name
        if single and len(self.names) != 1:
            raise ValueError("a token shift that returns a matrix has one reader")
        self.single = bool(single)
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {name: WeightSpec((self.channels,), kind="vector") for name in self.names}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((1, self.channels))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = torch.stack([runtime.vector(tensors[name]) for name in self.names]).contiguous()

    def forward(self, u: torch.Tensor, batch, cache) -> torch.Tensor:
        out = self.runtime.empty((len(self.names), u.shape[0], self.channels), u.dtype)
        self.runtime.ops.short_conv(u, self.weight, cache.states[self.state_name], batch, out, mode="towards_last")
        return out[0] if self.single else out

    def forward_normed(self, x: torch.Tensor, norm, batch, cache) -> torch.Tensor:
        """The shift of norm(x). Where there is one reader and the norm is a layer norm over whole rows, one kernel does
        both and keeps everything float32 up to the one rounding of its result (the state then holds the normed row
        itself, not what the compute dtype made of it; an engine takes this path in every step or in none)."""
        rt = self.runtime
        fused = getattr(rt.ops, "layernorm_shift", None)
        centred = getattr(norm, "centred", None)
        if fused is None or centred is None or not self.single or x.shape[1] != self.channels:
            return self.forward(norm.forward(x), batch, cache)
        weight, bias, eps = centred()
        out = rt.empty((x.shape[0], self.channels))
        state = cache.states[self.state_name]
        fused(x, weight, bias, eps, self.weight[0], state.view(state.shape[0], self.channels), batch, out)
        return out
