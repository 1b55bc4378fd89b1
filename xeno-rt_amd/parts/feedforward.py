"""Dense gated feed-forward: x + W_down (act(W_gate y) * (W_up y)), no biases.

The reference's SwiGLU block (crates/xrt-models/src/llama.rs:582-601) with
silu(z) = z / (1 + exp(-z)) (crates/xrt-kernels/src/cpu/silu.rs:1-3, 22-24).
Gate and up are bound as one matrix [2I][H] so that one product reads the
normed activations once, as the reference fuses the two dispatches
(llama.rs:584-594).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import FeedForward, Runtime, WeightSpec, register_part


class GatedMLP(FeedForward):
    capturable = True
    passes_norms = True

    ACTIVATIONS = ("silu",)

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu",
                 gate: str = "gate_proj.weight", up: str = "up_proj.weight", down: str = "down_proj.weight"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation must be one of {self.ACTIVATIONS}, found {activation!r}")
        self.prefix = prefix
        self.hidden = hidden
        self.intermediate = intermediate
        self.activation = activation
        self.gate_name, self.up_name, self.down_name = prefix + gate, prefix + up, prefix + down
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden, self.intermediate
        return {
            self.gate_name: WeightSpec((i, h)),
            self.up_name: WeightSpec((i, h)),
            self.down_name: WeightSpec((h, i)),
        }

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.w_gate_up = runtime.weight([tensors[self.gate_name], tensors[self.up_name]], "gated", gated_n=self.intermediate)
        self.w_down = runtime.weight(tensors[self.down_name])

    def forward_into(self, h, batch, out: torch.Tensor) -> None:
        """The feed-forward's output into `out` (float32 [tokens, hidden]) instead of onto the residual stream: for a
        block that puts a norm between the two."""
        rt = self.runtime
        act = rt.empty((h.shape[0], self.intermediate))
        rt.ops.linear_glu(h, self.w_gate_up, act, activation=self.activation)
        rt.ops.linear(act, self.w_down, out)

    def forward(self, h, batch, residual: torch.Tensor, then=None):
        rt = self.runtime
        tokens = h.shape[0]
        act = rt.empty((tokens, self.intermediate))
        rt.ops.linear_glu(h, self.w_gate_up, act, activation=self.activation)
        return rt.ops.linear(act, self.w_down, residual, accumulate=True,
                             then_norm=None if then is None else then.row_scale())


class DenseMLP(FeedForward):
    """x + W_down act(W_up y), no gate and no biases. act: "silu", "tanh", or "xielu", which has two learnt numbers
    (p, q) in the tensor `act`: z > 0: softplus(p) z^2 + z / 2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2.
    The activation reads the product's float32 sums and rounds once, to the compute dtype."""
    capturable = True

    ACTIVATIONS = ("silu", "tanh", "xielu")

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "xielu",
                 up: str = "up", down: str = "down", act: Optional[str] = "act"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation must be one of {self.ACTIVATIONS}, found {activation!r}")
        self.hidden, self.intermediate, self.activation = hidden, intermediate, activation
        self.up_name, self.down_name = prefix + up, prefix + down
        self.act_name = prefix + act if activation == "xielu" else None
        self.w_up = self.w_down = self.act_params = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {self.up_name: WeightSpec((self.intermediate, self.hidden)),
                 self.down_name: WeightSpec((self.hidden, self.intermediate))}
        if self.act_name is not None:
            specs[self.act_name] = WeightSpec((2,), kind="vector")
        return specs

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.w_up = runtime.weight(tensors[self.up_name])
        self.w_down = runtime.weight(tensors[self.down_name])
        if self.act_name is not None:
            self.act_params = runtime.vector(tensors[self.act_name])

    def forward(self, h, batch, residual: torch.Tensor) -> None:
        rt = self.runtime
        sums = rt.empty((h.shape[0], self.intermediate), torch.float32)
        rt.ops.linear(h, self.w_up, sums)
        act = rt.empty((h.shape[0], self.intermediate))
        rt.ops.activation(sums, act, self.activation, self.act_params)
        rt.ops.linear(act, self.w_down, residual, accumulate=True)


class ClampedGLU(FeedForward):
    """W_down (g sigmoid(alpha g) (u + 1)) with g = min(W_gate y, limit) and u = clamp(W_up y, -limit, limit); no biases.
    Gate and up are one product with float32 sums; the clamps and the activation read those and round once."""
    capturable = True

    def __init__(self, prefix: str, hidden: int, intermediate: int, limit: float, alpha: float = 1.702,
                 gate: str = "gate", up: str = "up", down: str = "down"):
        if limit <= 0:
            raise ValueError(f"the clamp's limit must be positive, found {limit}")
        self.hidden, self.intermediate, self.limit, self.alpha = hidden, intermediate, float(limit), float(alpha)
        self.gate_name, self.up_name, self.down_name = prefix + gate, prefix + up, prefix + down
        self.w_gate_up = self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden, self.intermediate
        return {self.gate_name: WeightSpec((i, h)), self.up_name: WeightSpec((i, h)), self.down_name: WeightSpec((h, i))}

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.w_gate_up = runtime.weight([tensors[self.gate_name], tensors[self.up_name]])
        self.w_down = runtime.weight(tensors[self.down_name])

    def _activated(self, h):
        rt = self.runtime
        sums = rt.empty((h.shape[0], 2 * self.intermediate), torch.float32)
        rt.ops.linear(h, self.w_gate_up, sums)
        act = rt.empty((h.shape[0], self.intermediate))
        rt.ops.glu_clamped(sums, act, self.limit, self.alpha)
        return act

    def forward_into(self, h, batch, out: torch.Tensor) -> None:
        self.runtime.ops.linear(self._activated(h), self.w_down, out)

    def forward(self, h, batch, residual: torch.Tensor) -> None:
        self.runtime.ops.linear(self._activated(h), self.w_down, residual, accumulate=True)


class ExpertsMLP(FeedForward):
    """A mixture of small gated feed-forwards (`e<n>.gate|up|down`, silu, no biases) of which every token uses `top`.
    The router (`router` [experts, hidden]) gives logits in float32; scores are their sigmoids. Experts stand in
    `groups` equal groups of neighbours, a group's score is the sum of its two largest scores, only experts of the `keep`
    best groups can be chosen (groups None: all can); the `top` largest scores are chosen and divided by their sum
    (+ 1e-20) as weights; the output is the weighted sum of the chosen experts' outputs.

    Every expert's gate and up rows lie in one matrix and their down columns in another. A step of few tokens multiplies
    every token with every expert (the step reads all weights once either way), weights each expert's stretch of the
    activations by the router's weight (zero for experts not chosen) and lets the down product add them up. A step of many
    tokens sorts its picks by expert, and every expert multiplies the rows that chose it (`ops.experts_sorted`). Either way
    a token's result never depends on what else the step holds.

    Options: `scores="softmax"` takes the softmax of the logits over all experts as scores; `group_top` is the number of a
    group's largest scores whose sum is the group's score (1: its largest score); `scale` multiplies the chosen experts'
    weights; `clamp=(limit, alpha)` makes the experts clamped ones, W_down (g sigmoid(alpha g) (u + 1)) with
    g = min(W_gate h, limit) and u = clamp(W_up h, -limit, limit): their gate and up rows then lie expert after expert in one
    matrix whose product keeps float32 sums, which the clamps and the activation read and round once."""
    capturable = True
    GROUP_TOP = 2
    WEIGHT_FLOOR = 1e-20

    def __init__(self, prefix: str, hidden: int, intermediate: int, experts: int, top: int, groups=None, keep=None,
                 router: str = "router", expert: str = "e{}.", gate: str = "gate", up: str = "up", down: str = "down",
                 scores: str = "sigmoid", group_top: Optional[int] = None, scale: float = 1.0, clamp=None):
        if experts <= 0 or not 0 < top <= experts:
            raise ValueError(f"{top} of {experts} experts")
        if scores not in ("sigmoid", "softmax"):
            raise ValueError(f"the router's scores are 'sigmoid' or 'softmax', found {scores!r}")
        self.scores, self.scale = scores, float(scale)
        self.group_top = self.GROUP_TOP if group_top is None else int(group_top)
        self.clamp = None if clamp is None else (float(clamp[0]), float(clamp[1]))
        if self.group_top <= 0 or (self.clamp is not None and self.clamp[0] <= 0):
            raise ValueError("a group's score sums one score at least, and a clamp's limit is positive")
        self.hidden, self.intermediate, self.experts, self.top = hidden, intermediate, int(experts), int(top)
        self.groups, self.keep = (1, 1) if groups is None else (int(groups), int(keep))
        if self.experts % self.groups != 0 or not 0 < self.keep <= self.groups or self.top > self.keep * (self.experts // self.groups):
            raise ValueError(f"{experts} experts in {self.groups} groups, {self.keep} kept, {top} chosen")
        self.router_name = prefix + router
        self.expert_names = [tuple(prefix + expert.format(n) + name for name in (gate, up, down)) for n in range(self.experts)]
        self.w_router = self.w_gate_up = self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden, self.intermediate
        specs = {self.router_name: WeightSpec((self.experts, h))}
        for gate, up, down in self.expert_names:
            specs.update({gate: WeightSpec((i, h)), up: WeightSpec((i, h)), down: WeightSpec((h, i))})
        return specs

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.w_router = runtime.matrix(tensors[self.router_name])
        total = self.experts * self.intermediate
        if self.clamp is not None:
            # every expert's [gate rows | up rows] one below the other: the float32 sums of a token and an expert are one stretch,
            # and an expert's rows are a matrix of their own for the product of sorted picks
            self.w_gate_up = runtime.weight([tensors[name] for names in self.expert_names for name in names[:2]])
        else:
            # [all gates | all ups] x hidden, and hidden x [every expert's stretch of the activations]; packed for a gated epilogue the
            # former lies expert after expert, which is what the product of sorted picks reads
            self.w_gate_up = runtime.weight([tensors[names[0]] for names in self.expert_names] + [tensors[names[1]] for names in self.expert_names],
                                            "gated", gated_n=total, needed=self.intermediate % 64 == 0 and self.top < self.experts)
        down = torch.empty((self.hidden, total), dtype=runtime.dtype, device=runtime.device)
        for n, names in enumerate(self.expert_names):
            down[:, n * self.intermediate:(n + 1) * self.intermediate].copy_(tensors[names[2]])
        self.w_down = runtime.weight(down)

    def _weights(self, h, chosen=None):
        rt = self.runtime
        logits = rt.empty((h.shape[0], self.experts), torch.float32)
        rt.ops.linear(h, self.w_router, logits)
        weights = rt.empty((h.shape[0], self.experts), torch.float32)
        rt.ops.route_experts(logits, weights, self.top, self.groups, self.keep, self.group_top, self.WEIGHT_FLOOR, chosen=chosen,
                             scores=self.scores, scale=self.scale)
        return weights

    def forward_into(self, h, batch, out: torch.Tensor) -> None:
        rt = self.runtime
        # A step of many tokens of which each uses few of the experts: the picks sorted by expert, every expert multiplies the
        # tokens that chose it. (Where the kernels have no such product, or it would not pay, every token meets every expert.)
        takes = getattr(rt.ops, "experts_sorted_takes", None)
        stacked = {} if self.clamp is None else {"stacked": True}
        if takes is not None and takes(h, self.w_gate_up, self.w_down, self.experts, self.intermediate, self.top, **stacked):
            chosen = rt.empty((h.shape[0], self.top), torch.int32)
            weights = self._weights(h, chosen)
            rt.ops.experts_sorted(h, self.w_gate_up, self.w_down, weights, chosen, self.intermediate, out,
                                  **({"activation": "silu"} if self.clamp is None else {"clamp": self.clamp}))
            return
        weights = self._weights(h)
        act = rt.empty((h.shape[0], self.experts * self.intermediate))
        if self.clamp is not None:
            sums = rt.empty((h.shape[0], 2 * self.experts * self.intermediate), torch.float32)
            rt.ops.linear(h, self.w_gate_up, sums)
            # (the router's weights ride along: a row of the sums is a (token, expert) pair)
            rt.ops.glu_clamped(sums.view(-1, 2 * self.intermediate), act.view(-1, self.intermediate), *self.clamp, row_weights=weights)
        else:
            rt.ops.linear_glu(h, self.w_gate_up, act, activation="silu")
            rt.ops.scale_blocks(act, weights, self.intermediate)
        rt.ops.linear(act, self.w_down, out)

    def forward(self, h, batch, residual: torch.Tensor) -> None:
        out = self.runtime.empty(residual.shape, torch.float32)
        self.forward_into(h, batch, out)
        self.runtime.ops.add(residual, out)


register_part("feed_forward", "gated_mlp", GatedMLP)
register_part("feed_forward", "clamped_glu", ClampedGLU)
register_part("feed_forward", "experts_mlp", ExpertsMLP)
register_part("feed_forward", "dense_mlp", DenseMLP)
