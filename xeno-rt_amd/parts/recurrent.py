"""Mixers whose memory is a matrix per head: S <- diag(decay) S + k v^T, read with the query.

Five of them, which differ in where the decay comes from and in what surrounds the recurrence:
  Retention             a fixed decay per head; k scaled by dim^-1/2; the heads' outputs divided by their root mean
                        square, gated by silu of a projection
  GatedLinearAttention  a decay per key channel and token, sigmoid(z)^(1/tau) with z from a low-rank projection with
                        bias; q scaled by dim^-1/2; the heads' outputs RMS-normed with a weight [vdim], gated
  TimeMixWKV            every projection reads its own mix of the token and the one before it; decay
                        exp(-exp(w0 + W2 tanh(W1 mix))) per key channel and token; the current token is read with a
                        bonus u before it enters the state; outputs divided by their root mean square, times a weight
                        over all heads, gated
  StateSpaceDuality     one projection makes gate, values, keys, queries and a step size per head; values, keys and queries
                        pass a short causal convolution with bias and silu; the head's channels all decay by
                        exp(-exp(A_log) step), values enter the state times the step, a skip D per head reads the value
                        itself; queries and keys may be shared by groups of heads; the row of all heads is gated, then
                        RMS-normed in equal parts
  LightningAttention    a fixed decay per head; q, k and v are silu of their projections and nothing is scaled; the row of
                        all heads is RMS-normed as one, with a weight, then gated by the sigmoid of a projection
And one whose memory is a vector per channel (`SelectiveStateSpace`): step sizes per channel from a low-rank projection,
decays exp(step A) per channel and entry, what is fed and read (B, C) shared by all channels of a token
(`ops.selective_scan`).
The state [heads, dim, vdim] is float32 and so are decays, norms and gates' activations; projections run in the compute dtype.
All run through one kernel (`ops.linear_recurrence`), which walks a sequence's tokens in order from the state that
the steps before left, so a request gives the same result however it is cut into steps.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .base import CacheNeeds, Mixer, Runtime, StateSpec, WeightSpec, register_part
from .convolution import ShortConvolution, TokenShift


class _RecurrentMixer(Mixer):
    capturable = True

    def _project_into(self, out_or_residual, o, accumulate: bool):
        return self.runtime.ops.linear(o, self.w_o, out_or_residual, accumulate=accumulate)

    def forward(self, h, batch, cache, residual: torch.Tensor) -> None:
        """Adds the mixer's output to the float32 residual stream."""
        self._project_into(residual, self.mixed(h, batch, cache), True)

    def forward_into(self, h, batch, cache, out: torch.Tensor) -> None:
        """Writes the mixer's output to `out` (float32) instead: for a mixer that is one of several side by side."""
        self._project_into(out, self.mixed(h, batch, cache), False)


class Retention(_RecurrentMixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, decay: Sequence[float], eps: float,
                 state_name: str = "retention"):
        if len(decay) != heads:
            raise ValueError(f"retention: {len(decay)} decays for {heads} heads")
        self.prefix, self.hidden, self.heads, self.dim, self.vdim = prefix, hidden, heads, dim, vdim
        self.decay_values, self.eps, self.state_name = [float(d) for d in decay], float(eps), state_name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd, vd = self.prefix, self.hidden, self.heads * self.dim, self.heads * self.vdim
        return {p + "q": WeightSpec((kd, w)), p + "k": WeightSpec((kd, w)), p + "v": WeightSpec((vd, w)),
                p + "g": WeightSpec((vd, w)), p + "o": WeightSpec((w, vd))}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.vdim))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.w_in = runtime.weight([tensors[p + name] for name in "qkvg"])
        self.w_o = runtime.weight(tensors[p + "o"])
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=runtime.device)

    def mixed(self, h, batch, cache):
        rt = self.runtime
        kd, vd = self.heads * self.dim, self.heads * self.vdim
        qkvg = rt.empty((h.shape[0], 2 * kd + 2 * vd))
        rt.ops.linear(h, self.w_in, qkvg)
        o = rt.empty((h.shape[0], vd))
        rt.ops.linear_recurrence(qkvg[:, :kd], qkvg[:, kd:2 * kd], qkvg[:, 2 * kd:2 * kd + vd], cache.states[self.state_name], batch, o,
                                 self.heads, self.dim, self.vdim, self.decay, "per_head", k_scale=self.dim ** -0.5,
                                 norm_eps=self.eps, gate=qkvg[:, 2 * kd + vd:], gate_activation="silu")
        return o


class LightningAttention(_RecurrentMixer):
    """S <- decay_h S + k v^T, o = S^T q per head with q = silu(W_q h), k = silu(W_k h), v = silu(W_v h); the heads' outputs side
    by side are RMS-normed together with a weight [heads * vdim], multiplied by sigmoid(W_g h), and projected."""

    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, decay: Sequence[float], eps: float,
                 state_name: str = "lightning"):
        if len(decay) != heads:
            raise ValueError(f"lightning attention: {len(decay)} decays for {heads} heads")
        self.prefix, self.hidden, self.heads, self.dim, self.vdim = prefix, hidden, heads, dim, vdim
        self.decay_values, self.eps, self.state_name = [float(d) for d in decay], float(eps), state_name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd, vd = self.prefix, self.hidden, self.heads * self.dim, self.heads * self.vdim
        return {p + "q": WeightSpec((kd, w)), p + "k": WeightSpec((kd, w)), p + "v": WeightSpec((vd, w)),
                p + "g": WeightSpec((vd, w)), p + "o": WeightSpec((w, vd)), p + "norm": WeightSpec((vd,), init="ones", kind="vector")}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.vdim))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.w_in = runtime.weight([tensors[p + name] for name in "qkvg"])
        self.w_o = runtime.weight(tensors[p + "o"])
        self.norm_weight = runtime.vector(tensors[p + "norm"])
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(runtime.device)

    def mixed(self, h, batch, cache):
        rt = self.runtime
        kd, vd = self.heads * self.dim, self.heads * self.vdim
        # the activations of q, k, v and the gate are worked out in float32 inside the kernels, from the projection's rows
        qkvg = rt.empty((h.shape[0], 2 * kd + 2 * vd))
        rt.ops.linear(h, self.w_in, qkvg)
        o = rt.empty((h.shape[0], vd))
        rt.ops.linear_recurrence(qkvg[:, :kd], qkvg[:, kd:2 * kd], qkvg[:, 2 * kd:2 * kd + vd], cache.states[self.state_name], batch, o,
                                 self.heads, self.dim, self.vdim, self.decay, "per_head", norm_eps=self.eps,
                                 norm_weight=self.norm_weight, norm_groups=1, gate_after_norm=True, gate=qkvg[:, 2 * kd + vd:],
                                 gate_activation="sigmoid", input_activation="silu")
        return o


class GatedLinearAttention(_RecurrentMixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, tau: float, low_rank: int, eps: float,
                 state_name: str = "gla"):
        self.prefix, self.hidden, self.heads, self.dim, self.vdim = prefix, hidden, heads, dim, vdim
        self.tau, self.low_rank, self.eps, self.state_name = float(tau), int(low_rank), float(eps), state_name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd, vd = self.prefix, self.hidden, self.heads * self.dim, self.heads * self.vdim
        return {p + "q": WeightSpec((kd, w)), p + "k": WeightSpec((kd, w)), p + "v": WeightSpec((vd, w)),
                p + "g": WeightSpec((vd, w)), p + "o": WeightSpec((w, vd)),
                p + "a1": WeightSpec((self.low_rank, w)), p + "a2": WeightSpec((kd, self.low_rank)),
                p + "a2.b": WeightSpec((kd,), kind="vector"),
                p + "norm": WeightSpec((self.vdim,), init="ones", kind="vector")}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.vdim))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.w_in = runtime.weight([tensors[p + name] for name in "qkvg"])
        self.w_a1 = runtime.weight(tensors[p + "a1"])
        self.w_a2 = runtime.weight(tensors[p + "a2"])
        self.a2_bias = runtime.vector(tensors[p + "a2.b"])
        self.norm_weight = runtime.vector(tensors[p + "norm"])
        self.w_o = runtime.weight(tensors[p + "o"])

    def mixed(self, h, batch, cache):
        rt = self.runtime
        tokens, kd, vd = h.shape[0], self.heads * self.dim, self.heads * self.vdim
        qkvg = rt.empty((tokens, 2 * kd + 2 * vd))
        rt.ops.linear(h, self.w_in, qkvg)
        low = rt.empty((tokens, self.low_rank))
        rt.ops.linear(h, self.w_a1, low)
        z = rt.empty((tokens, kd), torch.float32)                        # what the decay is made of stays float32
        rt.ops.linear(low, self.w_a2, z)
        o = rt.empty((tokens, vd))
        rt.ops.linear_recurrence(qkvg[:, :kd], qkvg[:, kd:2 * kd], qkvg[:, 2 * kd:2 * kd + vd], cache.states[self.state_name], batch, o,
                                 self.heads, self.dim, self.vdim, z, "sigmoid_power", decay_bias=self.a2_bias,
                                 decay_power=1.0 / self.tau, q_scale=self.dim ** -0.5, norm_eps=self.eps,
                                 norm_weight=self.norm_weight, gate=qkvg[:, 2 * kd + vd:], gate_activation="silu")
        return o


class TimeMixWKV(_RecurrentMixer):
    READERS = ("r", "k", "v", "g", "w")

    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, low_rank: int, eps: float, state_name: str = "wkv"):
        self.prefix, self.hidden, self.heads, self.dim = prefix, hidden, heads, dim
        self.low_rank, self.eps, self.state_name = int(low_rank), float(eps), state_name
        self.shift = TokenShift([prefix + "mu." + reader for reader in self.READERS], hidden, state_name + ".before")

    @property
    def capturable(self) -> bool:
        return self.shift.capturable

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd = self.prefix, self.hidden, self.heads * self.dim
        specs = {p + name: WeightSpec((kd, w)) for name in "rkvg"}
        specs.update({p + "w1": WeightSpec((self.low_rank, w)), p + "w2": WeightSpec((kd, self.low_rank)),
                      p + "w0": WeightSpec((kd,), kind="vector"),
                      p + "u": WeightSpec((self.heads, self.dim), kind="vector"),
                      p + "norm": WeightSpec((kd,), init="ones", kind="vector"), p + "o": WeightSpec((w, kd))})
        specs.update(self.shift.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.dim))),)).merged(self.shift.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.shift.bind(tensors, runtime)
        self.w_r, self.w_k, self.w_v, self.w_g = (runtime.weight(tensors[p + name]) for name in "rkvg")
        self.w_1 = runtime.weight(tensors[p + "w1"])
        self.w_2 = runtime.weight(tensors[p + "w2"])
        self.w0 = runtime.vector(tensors[p + "w0"])
        self.bonus = runtime.vector(tensors[p + "u"])
        self.norm_weight = runtime.vector(tensors[p + "norm"])
        self.w_o = runtime.weight(tensors[p + "o"])

    def mixed(self, h, batch, cache):
        rt = self.runtime
        tokens, kd = h.shape[0], self.heads * self.dim
        mixes = self.shift.forward(h, batch, cache)                      # [5, tokens, hidden]: r, k, v, g, w
        rkvg = [rt.empty((tokens, kd)) for _ in range(4)]
        for mix, weight, out in zip(mixes, (self.w_r, self.w_k, self.w_v, self.w_g), rkvg):
            rt.ops.linear(mix, weight, out)
        low = rt.empty((tokens, self.low_rank), torch.float32)
        rt.ops.linear(mixes[4], self.w_1, low)
        squashed = rt.empty((tokens, self.low_rank))
        rt.ops.activation(low, squashed, "tanh")
        z = rt.empty((tokens, kd), torch.float32)
        rt.ops.linear(squashed, self.w_2, z)
        o = rt.empty((tokens, kd))
        rt.ops.linear_recurrence(rkvg[0], rkvg[1], rkvg[2], cache.states[self.state_name], batch, o, self.heads, self.dim, self.dim,
                                 z, "exp_neg_exp", decay_bias=self.w0, bonus=self.bonus, norm_eps=self.eps,
                                 norm_weight=self.norm_weight, gate=rkvg[3], gate_activation="silu")
        return o


class StateSpaceDuality(_RecurrentMixer):
    """W_in h = [z: inner | x: inner | B: groups * n | C: groups * n | dt: heads], inner = heads * vdim. x, B, C pass a causal
    convolution per channel (`conv` [channels, taps], bias `conv.b`) and silu. step = softplus(dt + dt_bias); per head, with
    the B and C of its group, S <- exp(-exp(A_log) step) S + step B x^T (S is n x vdim), y = S^T C + D x. Then y * silu(z),
    RMS norm in `norm_groups` equal parts of the row times `norm` [inner], and W_o. The projection's sums stay float32 for
    the gate and the step sizes; the convolution keeps its inputs in float32 and rounds its result once."""

    def __init__(self, prefix: str, hidden: int, heads: int, vdim: int, state: int, groups: int, norm_groups: int, taps: int,
                 eps: float, state_name: str = "ssd"):
        if heads % groups != 0 or (heads * vdim) % norm_groups != 0:
            raise ValueError(f"{heads} heads of {vdim} in {groups} groups and {norm_groups} parts of the norm: neither divides")
        self.prefix, self.hidden, self.heads, self.vdim, self.n, self.groups = prefix, hidden, heads, vdim, int(state), groups
        self.norm_groups, self.eps, self.state_name = int(norm_groups), float(eps), state_name
        self.inner = heads * vdim
        self.conv_width = self.inner + 2 * groups * self.n
        self.convolution = ShortConvolution([prefix + "conv"], [self.conv_width], taps, state_name + ".conv",
                                            bias_names=[prefix + "conv.b"], activation="silu")

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w = self.prefix, self.hidden
        specs = {p + "in": WeightSpec((2 * self.inner + 2 * self.groups * self.n + self.heads, w)),
                 p + "dt_bias": WeightSpec((self.heads,), init="zeros", kind="vector"),
                 p + "A_log": WeightSpec((self.heads,), init="zeros", kind="vector"),
                 p + "D": WeightSpec((self.heads,), init="ones", kind="vector"),
                 p + "norm": WeightSpec((self.inner,), init="ones", kind="vector"), p + "o": WeightSpec((w, self.inner))}
        specs.update(self.convolution.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.n, self.vdim))),)).merged(self.convolution.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.convolution.bind(tensors, runtime)
        self.w_in = runtime.weight(tensors[p + "in"])
        self.w_o = runtime.weight(tensors[p + "o"])
        self.step_bias, self.rate, self.skip = (runtime.vector(tensors[p + name]) for name in ("dt_bias", "A_log", "D"))
        self.norm_weight = runtime.vector(tensors[p + "norm"])

    def mixed(self, h, batch, cache):
        rt = self.runtime
        tokens, inner, gn = h.shape[0], self.inner, self.groups * self.n
        proj = rt.empty((tokens, 2 * inner + 2 * gn + self.heads), torch.float32)
        rt.ops.linear(h, self.w_in, proj)
        xbc = self.convolution.forward(proj[:, inner:2 * inner + 2 * gn], batch, cache)          # compute dtype
        o = rt.empty((tokens, inner))
        rt.ops.linear_recurrence(xbc[:, inner + gn:], xbc[:, inner:inner + gn], xbc[:, :inner], cache.states[self.state_name], batch, o,
                                 self.heads, self.n, self.vdim, proj[:, 2 * inner + 2 * gn:], "step", decay_bias=self.step_bias,
                                 decay_rate=self.rate, qk_heads=self.groups, skip=self.skip, norm_eps=self.eps,
                                 norm_weight=self.norm_weight, norm_groups=self.norm_groups, gate=proj[:, :inner],
                                 gate_activation="silu")
        return o


class SelectiveStateSpace(_RecurrentMixer):
    """W_in h = [x: inner | z: inner]; x passes a causal convolution per channel (`conv`, bias `conv.b`) and silu. W_x x =
    [dt: rank | B: n | C: n]; step = softplus(W_dt dt + `dt.b`) per channel; A = -exp(A_log) [inner, n]. Per channel c:
    S[c] <- exp(step_c A[c]) S[c] + step_c x_c B, y_c = S[c] . C + D_c x_c; then y * silu(z), and W_o. Steps, B, C and the gate
    stay float32 from their products' sums on; the low-rank dt is rounded to the compute dtype for the product that follows."""

    def __init__(self, prefix: str, hidden: int, inner: int, state: int, rank: int, taps: int, state_name: str = "scan"):
        self.prefix, self.hidden, self.inner, self.n, self.rank, self.state_name = prefix, hidden, int(inner), int(state), int(rank), state_name
        self.convolution = ShortConvolution([prefix + "conv"], [self.inner], taps, state_name + ".conv",
                                            bias_names=[prefix + "conv.b"], activation="silu")

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w = self.prefix, self.hidden
        specs = {p + "in": WeightSpec((2 * self.inner, w)), p + "x": WeightSpec((self.rank + 2 * self.n, self.inner)),
                 p + "dt": WeightSpec((self.inner, self.rank)), p + "dt.b": WeightSpec((self.inner,), init="zeros", kind="vector"),
                 p + "A_log": WeightSpec((self.inner, self.n), init="zeros", kind="vector"),
                 p + "D": WeightSpec((self.inner,), init="ones", kind="vector"), p + "o": WeightSpec((w, self.inner))}
        specs.update(self.convolution.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.inner, self.n))),)).merged(self.convolution.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.convolution.bind(tensors, runtime)
        self.w_in = runtime.weight(tensors[p + "in"])
        low = tensors[p + "x"]
        self.w_low, self.w_bc = runtime.weight(low[:self.rank]), runtime.weight(low[self.rank:])
        self.w_step = runtime.weight(tensors[p + "dt"])
        self.w_o = runtime.weight(tensors[p + "o"])
        self.step_bias, self.skip = (runtime.vector(tensors[p + name]).to(torch.float32) for name in ("dt.b", "D"))
        self.a_log = runtime.vector(tensors[p + "A_log"]).to(torch.float32)

    def mixed(self, h, batch, cache):
        rt = self.runtime
        tokens, inner, n = h.shape[0], self.inner, self.n
        proj = rt.empty((tokens, 2 * inner), torch.float32)
        rt.ops.linear(h, self.w_in, proj)
        x = self.convolution.forward(proj[:, :inner], batch, cache)                                # compute dtype
        low = rt.empty((tokens, self.rank))
        rt.ops.linear(x, self.w_low, low)
        bc = rt.empty((tokens, 2 * n), torch.float32)
        rt.ops.linear(x, self.w_bc, bc)
        step = rt.empty((tokens, inner), torch.float32)
        rt.ops.linear(low, self.w_step, step)
        o = rt.empty((tokens, inner))
        rt.ops.selective_scan(x, step, bc[:, :n], bc[:, n:], cache.states[self.state_name], batch, o, self.a_log,
                              step_bias=self.step_bias, skip=self.skip, gate=proj[:, inner:])
        return o


register_part("mixer", "retention", Retention)
register_part("mixer", "lightning_attention", LightningAttention)
register_part("mixer", "state_space_duality", StateSpaceDuality)
register_part("mixer", "selective_state_space", SelectiveStateSpace)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "time_mix_wkv", TimeMixWKV)
