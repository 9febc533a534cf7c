"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, with eps on the mean square and
sum and rsqrt in float (reference: engine/kernels/rmsnorm.cu:16-41).  With ``offset`` the stored weight is
counted from it: y = x * rsqrt(...) * (offset + w) -- a weight stored around zero has offset 1.  With ``groups`` the row
is cut into that many equal runs of neighbouring channels, every run is brought to unit mean square by itself, and one weight spans the row."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part


class RMSNorm(Part):
    category = "norm"
    graph_safe = True

    def __init__(self, size: int, eps: float, offset: float = 0.0, groups: int = 1):
        self.size, self.eps, self.offset, self.groups = int(size), float(eps), float(offset), int(groups)
        if self.groups <= 0 or self.size % self.groups:
            raise ConfigError(f"rmsnorm: {self.size} channels do not fall into {self.groups} equal groups")
        self.weight = self._multiplier = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.size,), kind="vector", init="ones" if self.offset == 0.0 else "normal")}

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"]
        if self.offset != 0.0:          # the sum in float32, whatever the weight is stored in
            self.weight = (self.weight.to(torch.float32) + self.offset).contiguous()
        self._multiplier = None
        self.out_dtype = rt.act_dtype

    def add_to(self, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        """x += norm(y), in place on the float32 residual stream: the norm after a sublayer."""
        if self.groups != 1:
            raise ConfigError("rmsnorm: a norm in groups is not added to the stream by a kernel of its own")
        if self._multiplier is None:
            self._multiplier = self.weight.to(torch.float32).contiguous()
        return ops.rmsnorm_add(x, y, self._multiplier, self.eps)

    def fusable(self):
        """What a product needs to absorb this norm: (scale vector, eps); None for a norm in groups, which no product absorbs."""
        return (self.weight, self.eps) if self.groups == 1 else None

    def forward(self, x: torch.Tensor, ctx=None, rows=None, n_rows=None) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, self.out_dtype, rows=rows, n_rows=n_rows, groups=self.groups)

    def after_update(self, x: torch.Tensor, y: torch.Tensor, scale=None, bias=None, keep: bool = True) -> torch.Tensor:
        """x = (x if keep else 0) + scale * y + bias on the float32 stream, and this norm of the new x, in one kernel."""
        return ops.stream_update(x, y, scale, bias, keep, norm_weight=self.weight, eps=self.eps, groups=self.groups,
                                 out_dtype=self.out_dtype)


class DynamicTanh(Part):
    """y = (tanh(alpha x) * w + b) * out_scale, element by element: a norm that computes no mean and no variance.
    ``alpha`` is one number stored beside the weight.  Arithmetic is float32.  The input may be the residual stream
    in several copies, [T, n, H]: the norm is then taken of their sum."""
    category = "norm"
    graph_safe = True

    def __init__(self, size: int, out_scale: float = 1.0):
        self.size, self.out_scale = int(size), float(out_scale)
        self.weight = self.bias = self.alpha = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.size,), kind="vector", init="ones"), "b": WeightSpec((self.size,), kind="vector"),
                "alpha": WeightSpec((), kind="vector", init="ones")}

    def bind(self, tensors, rt) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).reshape(-1).contiguous()      # noqa: E731
        self.weight, self.bias, self.alpha = f32("weight"), f32("b"), f32("alpha")
        self.out_dtype = rt.act_dtype

    def pointwise(self):
        """What a kernel that has the norm's input in registers needs to apply it: (alpha [1], w, b, out_scale)."""
        return self.alpha, self.weight, self.bias, self.out_scale

    def forward(self, x: torch.Tensor, ctx=None, rows=None, n_rows=None) -> torch.Tensor:
        return ops.streams_read(x if x.dim() == 3 else x.unsqueeze(1), None, self.pointwise(), self.out_dtype, rows=rows, n_rows=n_rows)


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "dynamic_tanh", DynamicTanh)
