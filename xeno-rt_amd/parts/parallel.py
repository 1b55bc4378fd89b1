"""Two mixers side by side that read the same input: their outputs are RMS-normed over the model width, each with a
gain of its own, and half their sum goes onto the residual stream. Each half writes its output (float32) through
`forward_into(h, batch, cache, out)`; what either keeps per sequence lies in the same cache entry under its own names.

`WeightedPair` is the plain form: left_scale * left + right_scale * right, no norms and no gains. It hands its two
outputs and their scales to whoever sums them (`forward_terms`), so that a block which adds several sublayers' outputs
to the residual stream does so in one pass."""
from __future__ import annotations

from typing import Dict

import torch

from .base import CacheNeeds, Mixer, Runtime, WeightSpec, register_part


class ParallelMixer(Mixer):
    def __init__(self, left: Mixer, right: Mixer, hidden: int, left_gain: str, right_gain: str, eps: float, scale: float = 0.5):
        self.left, self.right, self.hidden = left, right, hidden
        self.gain_names, self.eps, self.scale = (left_gain, right_gain), float(eps), float(scale)

    @property
    def capturable(self) -> bool:
        return self.left.capturable and self.right.capturable

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {name: WeightSpec((self.hidden,), init="ones", kind="vector") for name in self.gain_names}
        specs.update(self.left.weight_specs())
        specs.update(self.right.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        return self.left.cache_needs().merged(self.right.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.left.bind(tensors, runtime)
        self.right.bind(tensors, runtime)
        self.gains = [runtime.vector(tensors[name]) for name in self.gain_names]

    def forward(self, h, batch, cache, residual: torch.Tensor) -> None:
        rt = self.runtime
        outs = [rt.empty(residual.shape, torch.float32) for _ in range(2)]
        self.left.forward_into(h, batch, cache, outs[0])
        self.right.forward_into(h, batch, cache, outs[1])
        rt.ops.add_normed(residual, list(zip(outs, self.gains)), self.eps, self.scale)


register_part("mixer", "parallel", ParallelMixer)


class WeightedPair(Mixer):
    def __init__(self, left: Mixer, right: Mixer, left_scale: float = 1.0, right_scale: float = 1.0):
        self.left, self.right = left, right
        self.scales = (float(left_scale), float(right_scale))

    @property
    def capturable(self) -> bool:
        return self.left.capturable and self.right.capturable

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = dict(self.left.weight_specs())
        specs.update(self.right.weight_specs())
        return specs

    def ignored_names(self):
        return [name for part in (self.left, self.right) for name in getattr(part, "ignored_names", lambda: [])()]

    def cache_needs(self) -> CacheNeeds:
        return self.left.cache_needs().merged(self.right.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.left.bind(tensors, runtime)
        self.right.bind(tensors, runtime)

    def forward_terms(self, h, batch, cache, like: torch.Tensor):
        """[(output float32 shaped like `like`, scale)] of the two halves; their scaled sum is the mixer's output."""
        rt = self.runtime
        outs = [rt.empty(like.shape, torch.float32) for _ in range(2)]
        self.left.forward_into(h, batch, cache, outs[0])
        self.right.forward_into(h, batch, cache, outs[1])
        return list(zip(outs, self.scales))

    def forward(self, h, batch, cache, residual: torch.Tensor) -> None:
        self.runtime.ops.add_weighted(residual, [(y, None, scale) for y, scale in self.forward_terms(h, batch, cache, residual)])


register_part("mixer", "weighted_pair", WeightedPair)
