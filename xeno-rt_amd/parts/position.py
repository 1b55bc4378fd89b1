"""Position encodings applied to queries and keys before the keys are cached.

Rotary: pairs (i, i + rope_dim/2) of every head are rotated by the angle
pos * scale / theta_i with theta_i = base^(2i/rope_dim); formulas of the
reference's crates/xrt-kernels/src/cpu/rope.rs:10-16 (table), :59-68 (angle),
:71-89 (rotation). Table, angle, sine and cosine are float32.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import HalfSplitRotation, PositionEncoding, Runtime, register_part


class Rotary(PositionEncoding):
    capturable = True

    def __init__(self, rope_dim: int, base: float, scale: float = 1.0, table_positions: int = 0):
        """table_positions: positions (from 0 on) whose cosines and sines are worked out once, when the part is bound,
        for kernels that can read them (a decode step's attention, where it also finishes q and k); 0: none."""
        if rope_dim <= 0 or rope_dim % 2 != 0:
            raise ValueError(f"rotary width must be positive and even, found {rope_dim}")
        self.rope_dim = rope_dim
        self.base = float(base)
        self.scale = float(scale)
        self.table_positions = int(table_positions)
        self.theta = None
        self.table = None

    def bind(self, tensors, runtime: Runtime) -> None:
        if self.theta is not None and getattr(self, "runtime", None) is runtime:
            return                                  # one encoding may serve many mixers: bound once
        super().bind(tensors, runtime)
        pair = torch.arange(self.rope_dim // 2, dtype=torch.float32)
        # float32 power, like the reference's powf (rope.rs:13)
        theta = torch.tensor(self.base, dtype=torch.float32) ** ((2.0 * pair) / float(self.rope_dim))
        self.theta = theta.to(runtime.device)
        make_table = getattr(runtime.ops, "rope_table", None)
        if self.table_positions > 0 and make_table is not None and self.theta.device.type == "cuda":
            self.table = make_table(self.theta, self.rope_dim, self.scale, self.table_positions)

    def rotation(self) -> HalfSplitRotation:
        return HalfSplitRotation(self.rope_dim, self.scale, self.theta, self.table)

    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        self.runtime.ops.qkv_prepare(
            qkv, n_heads, n_kv_heads, head_dim, batch.positions, batch.slots,
            rope_theta=self.theta, rope_dim=self.rope_dim, rope_scale=self.scale)


class NoPosition(PositionEncoding):
    """Leaves queries and keys as they are."""
    capturable = True


    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        return None


class DistanceSlopes(PositionEncoding):
    """Positions enter the scores only: a key at distance d behind the query loses slope_h * d, with
    slope_h = 2^(-span (h + 1) / n_heads) for head h. Queries and keys stay as they are."""
    capturable = True

    def __init__(self, n_heads: int, span: float = 8.0):
        self.n_heads, self.span = int(n_heads), float(span)
        self.slopes = None

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        exponents = torch.arange(1, self.n_heads + 1, dtype=torch.float64) * (-self.span / self.n_heads)
        self.slopes = torch.pow(torch.tensor(2.0, dtype=torch.float64), exponents).to(torch.float32).to(runtime.device)

    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        return None

    def score_slopes(self):
        return self.slopes


class PairRotation(PositionEncoding):
    """Pairs of dims of every head of q and k turn by the angle position * f_n, the first rope_dim dims of a head in
    pairs of neighbours (2n, 2n + 1) or of halves (n, n + rope_dim / 2); the rest pass. f_n = base^(-2n / rope_dim), or
    with `scaling` = {factor, original, fast, slow} stretched for contexts beyond the `original` length: with
    c(t) = rope_dim ln(original / (2 pi t)) / (2 ln base) the pair at which a wave makes t turns over that length,
    lo = max(floor(c(fast)), 0), hi = min(ceil(c(slow)), rope_dim - 1), r_n = clamp((n - lo) / max(hi - lo, 0.001), 0, 1),
    the frequency is f_n / factor * r_n + f_n (1 - r_n) (slow waves are stretched by the factor, fast ones stay, those
    between are blended), and cosines and sines are multiplied by 0.1 ln(factor) + 1. The table of frequencies is made
    on the host in float64 and kept in float32; angles, cosines and sines are the kernel's, in float32."""
    capturable = True
    RAMP_FLOOR = 0.001
    MAGNITUDE_SLOPE = 0.1

    def __init__(self, rope_dim: int, base: float, neighbours: bool = True, scaling: Optional[dict] = None):
        """A second rule of stretching, by wavelength, is asked for with scaling = {factor, low, high, original}: with the
        wavelength l = 2 pi / f a frequency stays where l < original / high, becomes f / factor where l > original / low, and
        between the two, with s = (original / l - low) / (high - low), (1 - s) f / factor + s f; cosines and sines stay as
        they are."""
        if rope_dim <= 0 or rope_dim % 2 != 0:
            raise ValueError(f"rotary width must be positive and even, found {rope_dim}")
        self.rope_dim, self.base, self.neighbours = int(rope_dim), float(base), bool(neighbours)
        self.by_wavelength = bool(scaling) and "low" in scaling
        keys = ("factor", "original", "low", "high") if self.by_wavelength else ("factor", "original", "fast", "slow")
        self.scaling = None if not scaling else {key: float(scaling[key]) for key in keys}
        self.frequencies = None
        self.magnitude = 1.0 if self.scaling is None or self.by_wavelength else self.MAGNITUDE_SLOPE * math.log(self.scaling["factor"]) + 1.0

    def frequency_table(self):
        """The pairs' frequencies, as Python floats."""
        plain = [self.base ** (-2.0 * n / self.rope_dim) for n in range(self.rope_dim // 2)]
        if self.scaling is None:
            return plain
        c = self.scaling
        if self.by_wavelength:
            out = []
            for f in plain:
                wavelength = 2.0 * math.pi / f
                if wavelength > c["original"] / c["low"]:
                    f = f / c["factor"]
                elif wavelength >= c["original"] / c["high"]:
                    share = (c["original"] / wavelength - c["low"]) / (c["high"] - c["low"])
                    f = (1.0 - share) * f / c["factor"] + share * f
                out.append(f)
            return out

        def pair_of(turns: float) -> float:
            return self.rope_dim * math.log(c["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

        lo = max(math.floor(pair_of(c["fast"])), 0)
        hi = min(math.ceil(pair_of(c["slow"])), self.rope_dim - 1)
        out = []
        for n, f in enumerate(plain):
            ramp = min(max((n - lo) / max(hi - lo, self.RAMP_FLOOR), 0.0), 1.0)
            out.append(f / c["factor"] * ramp + f * (1.0 - ramp))
        return out

    def bind(self, tensors, runtime: Runtime) -> None:
        if self.frequencies is not None and getattr(self, "runtime", None) is runtime:
            return
        super().bind(tensors, runtime)
        self.frequencies = torch.tensor(self.frequency_table(), dtype=torch.float64).to(torch.float32).to(runtime.device)

    def pair_rotation(self):
        """(frequencies float32 [rope_dim / 2] on the device, rope_dim, neighbours, magnitude): for the kernel that completes
        q and k after their projection."""
        return self.frequencies, self.rope_dim, self.neighbours, self.magnitude

    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        raise NotImplementedError("a rotation of pairs with a table of frequencies is done by the kernel that completes q and k")


class DistanceBuckets(PositionEncoding):
    """Positions enter the scores only: a learnt number per head and bucket of distance is added to the scaled score.
    The table `name` is [rows, n_heads]; a key n tokens behind the query reads row n for n < rows / 2 (halves rounded
    down), else row min(rows - 1, rows / 2 + floor(ln(n / (rows / 2)) / ln(far / (rows / 2)) * (rows - rows / 2))): steps
    that grow with the distance and reach the last row at `far`. Bound, it is a dense table [n_heads, span] by distance,
    whose last column holds for every distance beyond."""
    capturable = True

    def __init__(self, name: str, n_heads: int, rows: int, far: float):
        if rows < 2 or far <= rows // 2:
            raise ValueError(f"a table of {rows} buckets that ends at distance {far}: two rows at least, and an end beyond half of them")
        self.name, self.n_heads, self.rows, self.far = name, int(n_heads), int(rows), float(far)
        self.table = None

    def weight_specs(self):
        from .base import WeightSpec
        return {self.name: WeightSpec((self.rows, self.n_heads), kind="vector")}

    def bucket(self, n: int) -> int:
        half = self.rows // 2
        if n < half:
            return n
        return min(self.rows - 1, half + int(math.floor(math.log(n / half) / math.log(self.far / half) * (self.rows - half))))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        span = 1
        while self.bucket(span - 1) < self.rows - 1:
            span += 1
        rows = torch.tensor([self.bucket(n) for n in range(span)], dtype=torch.long)
        learnt = tensors[self.name].to(torch.float32).to("cpu")
        self.table = learnt[rows].t().contiguous().to(runtime.device)          # [n_heads, span]

    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        return None

    def score_bias_table(self):
        return self.table


register_part("position", "pair_rotation", PairRotation)
register_part("position", "distance_buckets", DistanceBuckets)
register_part("position", "distance_slopes", DistanceSlopes)
register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
