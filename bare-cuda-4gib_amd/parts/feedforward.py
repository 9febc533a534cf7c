"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear, linear_swiglu


class SwiGLU(Part):
    """x += (silu(h Wg^T) * (h Wu^T)) Wd^T with silu(g) = g / (1 + exp(-g)), no
    biases (reference: engine/src/model.cpp:579-603, engine/kernels/swiglu.cu:17-25)."""
    category = "feedforward"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    accepts_lazy_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.w_gu = self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": WeightSpec((i, h)), "up_proj.weight": WeightSpec((i, h)),
                "down_proj.weight": WeightSpec((h, i))}

    def bind(self, tensors, rt) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        dt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        i, h = self.intermediate_size, self.hidden_size
        # One product for gate and up.  For the matrix-core kernels (bfloat16, I a multiple of 8) the
        # rows go in blocks of 16 -- eight gate rows, then the eight up rows of the same outputs -- so
        # that one workgroup of the weight-streaming kernel holds both halves of its outputs;
        # otherwise gate's rows, then up's.
        self.interleaved = dt == torch.bfloat16 and i % 8 == 0
        if self.interleaved:
            self.w_gu = torch.stack([g.view(i // 8, 8, h), u.view(i // 8, 8, h)], dim=1).reshape(2 * i, h).contiguous()
        else:
            self.w_gu = torch.cat([g.to(dt), u.to(dt)], dim=0).contiguous()
        self.w_gu = ops.StreamedWeight(self.w_gu)
        self.w_down = ops.StreamedWeight(tensors["down_proj.weight"])
        self.act_dtype = rt.act_dtype

    def wants_prepared_norm(self, n_rows: int) -> bool:
        """Whether the gate-up product, at this many rows, is better served by a norm that the product before
        prepared than by fusing the norm or running it: the weight's own plan says (ops.LinearPlan.wants_prepared)."""
        return self.interleaved and self.w_gu.plan.wants_prepared(n_rows, swiglu=True)

    def forward(self, h, ctx, residual) -> None:
        act = linear_swiglu(h, self.w_gu, self.interleaved)
        linear(act, self.w_down, accumulate_into=residual, ctx=ctx)


class DenseXIELU(Part):
    """x += Wd act(Wu h), no biases, with act(z) = softplus(p) z^2 + z/2 for z > 0 and
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 otherwise; p and q are the two numbers of the tensor ``act``."""
    category = "feedforward"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    accepts_lazy_norm = True
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.w_up = self.w_down = self.pq = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {"up": WeightSpec((i, h)), "down": WeightSpec((h, i)), "act": WeightSpec((2,), kind="vector")}

    def bind(self, tensors, rt) -> None:
        self.w_up = ops.StreamedWeight(tensors["up"])
        self.w_down = ops.StreamedWeight(tensors["down"])
        self.pq = tensors["act"].to(torch.float32).contiguous()
        self.act_dtype = rt.act_dtype

    def forward(self, h, ctx, residual) -> None:
        z = linear(h, self.w_up, out_dtype=self.act_dtype)
        linear(ops.xielu(z, self.pq, out=z), self.w_down, accumulate_into=residual, ctx=ctx)


class ClampedGLU(Part):
    """x += Wd (g sigmoid(slope g) (u + 1)) with g = min(Wg h, limit) and u = clamp(Wu h, -limit, limit), no biases."""
    category = "feedforward"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, slope: float = 1.702):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.limit, self.slope = float(limit), float(slope)
        self.w_gu = self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {"gate": WeightSpec((i, h)), "up": WeightSpec((i, h)), "down": WeightSpec((h, i))}

    def bind(self, tensors, rt) -> None:
        # one product for gate and up: the gates' rows, then the ups'
        self.w_gu = ops.StreamedWeight(torch.cat([tensors["gate"], tensors["up"]], dim=0).contiguous())
        self.w_down = ops.StreamedWeight(tensors["down"])
        self.act_dtype = rt.act_dtype

    def step_work(self, batch, rows: int, elem: int):
        flops, nbytes = super().step_work(batch, rows, elem)
        return flops + 8.0 * rows * self.intermediate_size, nbytes

    def forward(self, h, ctx, residual) -> None:
        gu = linear(h, self.w_gu, out_dtype=self.act_dtype)
        linear(ops.clamped_glu(gu, self.limit, self.slope), self.w_down, accumulate_into=residual, ctx=ctx)


class DenseGELU(Part):
    """x += Wd gelu(Wu h), no biases, with the exact gelu z Phi(z)."""
    category = "feedforward"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    accepts_lazy_norm = True
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.w_up = self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {"up": WeightSpec((i, h)), "down": WeightSpec((h, i))}

    def bind(self, tensors, rt) -> None:
        self.w_up = ops.StreamedWeight(tensors["up"])
        self.w_down = ops.StreamedWeight(tensors["down"])
        self.act_dtype = rt.act_dtype

    def step_work(self, batch, rows: int, elem: int):
        flops, nbytes = super().step_work(batch, rows, elem)
        return flops + 10.0 * rows * self.intermediate_size, nbytes

    def forward(self, h, ctx, residual) -> None:
        z = linear(h, self.w_up, out_dtype=self.act_dtype)
        linear(ops.gelu(z, out=z), self.w_down, accumulate_into=residual, ctx=ctx)


class RoutedExperts(Part):
    """A mixture of clamped gated units: x += sum over the chosen experts e of s_e * expert_e(h), plus, if there is one, a
    shared expert for every row times sigmoid(Wsg h).

    The router: z = Wr h in float32, s = softmax(z) over all experts; the choice goes by s + ``correction``; the experts
    lie in ``groups`` equal groups of neighbours, a group counts by its largest choice, and only experts of the ``keep``
    best groups can be chosen; the ``top`` largest choices win.  The weights are the chosen experts' s, as they are.
    An expert: Wd (g sigmoid(slope g) (u + 1)) with g = min(Wg h, limit), u = clamp(Wu h, -limit, limit), no biases.

    All experts' gate and up matrices are one product and all their down matrices another: between the two, a row's
    units of the experts it did not choose are multiplied by zero and those of the chosen by their weights, so that the
    second product adds up the weighted sum (the router's and the shared gate's logits are one small float32 product).
    Tensors: ``router`` [experts, hidden], ``correction`` [experts], ``e<i>.{gate,up,down}``, ``shared.{gate,up,down}``,
    ``shared.sg`` [1, hidden].

    ``router`` "sigmoid": s = sigmoid(z), every expert by itself.  ``normalize``: the weights are the chosen experts' s divided
    by their sum (+ 1e-20).  ``route_scale`` multiplies the weights.  ``unit`` "gelu": an expert is Wd gelu(Wu h) with the exact
    gelu -- no gate matrix, no limit (``e<i>.{up,down}``, ``shared.{up,down}``).  ``shared_gate`` False: the shared expert is
    added as it is (no ``shared.sg``)."""
    category = "feedforward"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    accepts_lazy_norm = True
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, experts: int, top: int, intermediate_size: int, limit: float = 0.0, groups: int = 1,
                 keep: int = 1, correction: bool = True, shared_size: int = 0, shared_limit: float = 0.0, slope: float = 1.702,
                 router: str = "softmax", normalize: bool = False, route_scale: float = 1.0, unit: str = "clamped_glu",
                 shared_gate: bool = True):
        if router not in ("softmax", "sigmoid") or unit not in ("clamped_glu", "gelu"):
            raise ConfigError(f"routed experts: router {router!r} ('softmax' or 'sigmoid'), unit {unit!r} ('clamped_glu' or 'gelu')")
        self.squash, self.normalize, self.route_scale = router == "sigmoid", bool(normalize), float(route_scale)
        self.gated, self.shared_gate = unit == "clamped_glu", bool(shared_gate) and unit == "clamped_glu"
        self.hidden_size, self.experts, self.top, self.ff = int(hidden_size), int(experts), int(top), int(intermediate_size)
        self.limit, self.groups, self.keep, self.correction = float(limit), int(groups), int(keep), bool(correction)
        self.shared_ff, self.shared_limit, self.slope = int(shared_size), float(shared_limit), float(slope)
        if not (0 < self.experts <= ops.MOE_MAX_EXPERTS) or not (0 < self.top <= self.experts) or self.ff <= 0:
            raise ConfigError(f"routed experts: {self.top} of {self.experts} experts (at most {ops.MOE_MAX_EXPERTS}) of size {self.ff}")
        if self.groups <= 0 or self.experts % self.groups or not (0 < self.keep <= self.groups):
            raise ConfigError(f"routed experts: {self.experts} experts in {self.groups} groups of which {self.keep} are kept")
        if self.top > self.keep * (self.experts // self.groups):
            raise ConfigError(f"routed experts: {self.top} experts cannot be chosen from {self.keep} groups of "
                              f"{self.experts // self.groups}")

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, f = self.hidden_size, self.ff
        out = {"router": WeightSpec((self.experts, h))}
        if self.correction:
            out["correction"] = WeightSpec((self.experts,), kind="vector")
        for name, size in [(f"e{e}", f) for e in range(self.experts)] + ([("shared", self.shared_ff)] if self.shared_ff else []):
            out.update({f"{name}.up": WeightSpec((size, h)), f"{name}.down": WeightSpec((h, size))})
            if self.gated:
                out[f"{name}.gate"] = WeightSpec((size, h))
        if self.shared_ff and self.shared_gate:
            out["shared.sg"] = WeightSpec((1, h))
        return out

    def bind(self, tensors, rt) -> None:
        names = [f"e{e}" for e in range(self.experts)] + (["shared"] if self.shared_ff else [])
        # per expert its gates' rows, then its ups'; the down matrices side by side along their inputs
        # (plain units have no gates: every expert's ups' rows)
        inner = ("gate", "up") if self.gated else ("up",)
        self.w_gu = ops.StreamedWeight(torch.cat([tensors[f"{n}.{part}"] for n in names for part in inner], dim=0).contiguous())
        self.w_down = ops.StreamedWeight(torch.cat([tensors[f"{n}.down"] for n in names], dim=1).contiguous())
        gated_shared = self.shared_ff and self.shared_gate
        self.w_route = ops.StreamedWeight(torch.cat([tensors["router"]] + ([tensors["shared.sg"]] if gated_shared else []),
                                                    dim=0).contiguous())
        self.correction_w = tensors["correction"].to(torch.float32).contiguous() if self.correction else None
        self.act_dtype = rt.act_dtype

    def step_work(self, batch, rows: int, elem: int):
        """What the design asks for: the router, ``top`` experts a row and the shared one; every weight read once."""
        h = self.hidden_size
        units = self.top * self.ff + self.shared_ff
        mats = 3 if self.gated else 2
        flops = 2.0 * rows * h * (self.experts + (1 if self.shared_ff else 0)) + rows * units * (2.0 * mats * h + 8.0)
        nbytes = (self.experts * (mats * self.ff * h + h) + (mats * self.shared_ff * h + h if self.shared_ff else 0)) * elem
        return flops, float(nbytes)

    def working_bytes_per_row(self, elem: int) -> float:
        return 3.0 * (self.experts * self.ff + self.shared_ff) * elem + 8.0 * (self.experts + 1)

    def forward(self, h, ctx, residual) -> None:
        if hasattr(h, "tensor") and callable(h.tensor):      # (three products read the norm: it is computed once)
            h = h.tensor()
        E = self.experts
        z = linear(h, self.w_route, out_dtype=torch.float32)
        weights = ops.moe_route(z, E, self.top, self.groups, self.keep, self.correction_w, squash=self.squash,
                                normalize=self.normalize, factor=self.route_scale)
        gu = linear(h, self.w_gu, out_dtype=self.act_dtype)
        if not self.gated:
            linear(ops.routed_gelu(gu, weights, E, self.ff, self.shared_ff, out=gu), self.w_down, accumulate_into=residual, ctx=ctx)
            return
        y = ops.routed_glu(gu, weights, E, self.ff, self.limit, shared_ff=self.shared_ff, shared_limit=self.shared_limit,
                           shared_logit=z[:, E:E + 1] if self.shared_ff else None, slope=self.slope)
        linear(y, self.w_down, accumulate_into=residual, ctx=ctx)


register_part("feedforward", "swiglu", SwiGLU)
register_part("feedforward", "dense_gelu", DenseGELU)
register_part("feedforward", "routed_experts", RoutedExperts)
register_part("feedforward", "clamped_glu", ClampedGLU)
register_part("feedforward", "dense_xielu", DenseXIELU)
