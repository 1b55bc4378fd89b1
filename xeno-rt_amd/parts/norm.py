"""RMSNorm: y = (x / sqrt(mean(x^2) + eps)) * w, computed in float32.

Formula: crates/xrt-kernels/src/cpu/rmsnorm.rs:26-43 of the reference; the
weight is used as stored (not 1 + w).

LayerNorm: y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the squared deviations; not in the reference's model.

A norm may also stand behind a sublayer, on the sublayer's way onto the residual stream: `add_to(residual, y, scale)` is
residual += scale * norm(y), all of it float32.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Norm, Runtime, WeightSpec, register_part


class RMSNorm(Norm):
    capturable = True

    def __init__(self, prefix: str, dim: int, eps: float, name: Optional[str] = None):
        """The gain is the tensor `prefix + "weight"`, or `name` if given."""
        self.prefix = prefix
        self.name = prefix + "weight" if name is None else name
        self.dim = dim
        self.eps = float(eps)
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.dim,), init="ones", kind="vector")}

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = runtime.vector(tensors[self.name])

    def row_scale(self):
        return self.weight, self.eps

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        count = x.shape[0] if rows is None else rows.shape[0]
        out = self.runtime.empty((count, self.dim))
        self.runtime.ops.rmsnorm(x, self.weight, self.eps, out, rows=rows)
        return out

    def add_to(self, residual: torch.Tensor, y: torch.Tensor, scale: float = 1.0) -> None:
        """residual += scale * norm(y); y float32 like the residual."""
        self.runtime.ops.add_normed(residual, [(y, self.weight)], self.eps, scale)


class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * w + b over whole rows. `name` is the weight's tensor, `bias_name` the bias's."""
    capturable = True

    def __init__(self, name: str, bias_name: str, dim: int, eps: float):
        self.name, self.bias_name, self.dim, self.eps = name, bias_name, int(dim), float(eps)
        self.weight = self.bias = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.dim,), init="ones", kind="vector"),
                self.bias_name: WeightSpec((self.dim,), init="zeros", kind="vector")}

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = runtime.vector(tensors[self.name])
        self.bias = runtime.vector(tensors[self.bias_name]).to(self.weight.dtype)

    def centred(self):
        """(weight, bias, eps): what a kernel that does this norm on its way needs."""
        return self.weight, self.bias, self.eps

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        count = x.shape[0] if rows is None else rows.shape[0]
        out = self.runtime.empty((count, self.dim))
        self.runtime.ops.layernorm(x, self.weight, self.bias, self.eps, out, rows=rows)
        return out

    def add_to(self, residual: torch.Tensor, y: torch.Tensor, scale: float = 1.0, pre_bias: Optional[torch.Tensor] = None,
               then: Optional["LayerNorm"] = None) -> Optional[torch.Tensor]:
        """residual += scale * norm(y + pre_bias). With `then`, another layer norm, its result on the updated residual is
        returned as well (compute dtype), made in the same pass."""
        out = None if then is None else self.runtime.empty(residual.shape)
        if pre_bias is not None:
            pre_bias = pre_bias.to(self.weight.dtype)
        self.runtime.ops.add_layernormed(residual, y, self.weight, self.bias, self.eps, scale, pre_bias=pre_bias,
                                         then=None if then is None else then.centred(), then_out=out)
        return out


class ScalarRMSNorm(RMSNorm):
    """RMSNorm whose gain is one number for all coordinates: y = x / sqrt(mean(x^2) + eps) * g. `name` is the tensor
    that holds g (shape []); it is spread over the row when bound, and the norm then runs as any other."""

    def __init__(self, name: str, dim: int, eps: float):
        super().__init__(name, dim, eps)
        self.name = name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((), init="ones", kind="vector")}

    def bind(self, tensors, runtime: Runtime) -> None:
        Norm.bind(self, tensors, runtime)
        self.weight = runtime.vector(tensors[self.name]).reshape(1).expand(self.dim).contiguous()


class OffsetRMSNorm(RMSNorm):
    """RMSNorm whose tensor w holds the gain minus one: y = x / sqrt(mean(x^2) + eps) * (1 + w). `name` is the tensor that holds
    w; 1 + w is worked out in float32 when the part is bound, and the norm then runs as any other."""

    def __init__(self, name: str, dim: int, eps: float):
        super().__init__(name, dim, eps)
        self.name = name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.dim,), init="zeros", kind="vector")}

    def bind(self, tensors, runtime: Runtime) -> None:
        Norm.bind(self, tensors, runtime)
        self.weight = (tensors[self.name].to(torch.float32) + 1.0).to(runtime.device).contiguous()


register_part("norm", "offset_rmsnorm", OffsetRMSNorm)
register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
register_part("norm", "scalar_rmsnorm", ScalarRMSNorm)
