"""What a stack that runs some of its layers several times does to the residual stream before a pass."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear


class StreamReentry(Part):
    """Before pass t of a run of layers (the first pass too): x = W [x; x0] + s_t, with x0 the embedding's output for the
    same tokens, W ``in`` [hidden, 2 hidden] (the stream's half first) and s ``step`` [passes, hidden].  The stream is
    replaced, not added to; the sum with s_t is float32, and the kernel that writes the new stream also norms it for the
    pass's first layer where that layer's norm can follow an update."""
    category = "reentry"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, hidden_size: int, passes: int):
        self.hidden_size, self.passes = int(hidden_size), int(passes)
        if self.passes < 1:
            raise ConfigError(f"stream reentry: {self.passes} passes")
        self.w_in = self.steps = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h = self.hidden_size
        return {"in": WeightSpec((h, 2 * h)), "step": WeightSpec((self.passes, h), kind="vector")}

    def bind(self, tensors, rt) -> None:
        self.w_in = ops.StreamedWeight(tensors["in"])
        self.steps = tensors["step"].to(torch.float32).contiguous()
        self.act_dtype = rt.act_dtype

    def forward(self, x: torch.Tensor, ctx, embedding, turn: int, next_norm=None):
        """Replaces the float32 stream x [T, hidden] in place; returns ``next_norm`` of the new stream if that norm could be
        computed on the way, else None."""
        if not 0 <= turn < self.passes:
            raise ConfigError(f"stream reentry: pass {turn} of {self.passes}")
        both = embedding.beside(x, ctx, self.act_dtype)
        y = linear(both, self.w_in, out_dtype=torch.float32)
        if next_norm is not None and hasattr(next_norm, "after_update"):
            return next_norm.after_update(x, y, bias=self.steps[turn], keep=False)
        ops.stream_update(x, y, bias=self.steps[turn], keep=False)
        return None


register_part("reentry", "stream_reentry", StreamReentry)
