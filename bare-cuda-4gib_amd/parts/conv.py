"""A short causal convolution over time on each channel, continued across a request's steps."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.specs import States
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part


class CausalConv(Part):
    """out[t, c] = bias[c] + sum_j w[c, j] * v[t - taps + 1 + j, c] over a request's rows v, zeros before its first
    token; the last column of w is the current token's.  The request's last taps - 1 rows are its state (``tail``, in
    the activations' dtype), so a prompt may be cut anywhere.  ``forward(v, ctx, view, add_input)`` returns the
    convolution, with ``add_input`` v + the convolution."""
    category = "conv"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, channels: int, taps: int, bias: bool = False):
        if channels <= 0 or taps < 1:
            raise ConfigError(f"causal convolution: {channels} channels and {taps} taps")
        self.channels, self.taps, self.bias = int(channels), int(taps), bool(bias)
        self.w = self.b = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        out = {"weight": WeightSpec((self.channels, self.taps), kind="vector")}
        if self.bias:
            out["bias"] = WeightSpec((self.channels,), kind="vector")
        return out

    def bind(self, tensors, rt) -> None:
        self.w = tensors["weight"].to(torch.float32).t().contiguous()      # by taps: neighbouring channels side by side
        self.b = tensors["bias"].to(torch.float32).contiguous() if self.bias else None

    def cache_spec(self):
        return States((("tail", (self.taps - 1, self.channels), None),))

    def forward(self, v: torch.Tensor, ctx, view, add_input: bool = False, in_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.causal_conv(v, self.w, view.tail if self.taps > 1 else None, ctx, in_bias=in_bias, out_bias=self.b,
                               add_input=add_input)


class TokenShift(Part):
    """out[t] = h[t] + (h[t - 1] - h[t]) * m, element by element, along a request's rows; h[-1] = 0.  The h on the right
    are the rows as they came in.  A request's last row is its state (``tail``, in the activations' dtype), so a prompt
    may be cut anywhere.  It is the causal convolution with the taps (m, -m) plus its input.  ``after(norm, x, ...)`` is
    the shift of norm(x): behind an RMS norm both are one kernel (the same state, the same roundings)."""
    category = "conv"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, channels: int):
        if channels <= 0:
            raise ConfigError(f"token shift: {channels} channels")
        self.channels = int(channels)
        self.w = self.m = self._norm = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.channels,), kind="vector")}

    def bind(self, tensors, rt) -> None:
        m = tensors["weight"].to(torch.float32)
        self.w = torch.stack([m, -m], dim=0).contiguous()      # by taps: the row before, the row itself
        self.m = m.contiguous()
        self.out_dtype = rt.act_dtype

    def cache_spec(self):
        return States((("tail", (1, self.channels), None),))

    def forward(self, h: torch.Tensor, ctx, view) -> torch.Tensor:
        return ops.causal_conv(h, self.w, view.tail, ctx, add_input=True)

    def after(self, norm, x: torch.Tensor, ctx, view) -> torch.Tensor:
        """The shift of norm(x) for the float32 stream x [T, H]."""
        fusable = getattr(norm, "fusable", None)
        if fusable is None or fusable() is None or x.dim() != 2 or x.dtype != torch.float32:
            return self.forward(norm.forward(x, ctx), ctx, view)
        if self._norm is None or self._norm[0] is not norm:
            g, eps = fusable()
            self._norm = (norm, g.to(torch.float32).contiguous(), float(eps))
        return ops.rmsnorm_shift(x, self._norm[1], self._norm[2], self.m, view.tail, ctx, self.out_dtype)


register_part("conv", "causal", CausalConv)
register_part("conv", "token_shift", TokenShift)
