"""Windowed softmax attention with a sink in the denominator, and what may stand around it: a short convolution over
time behind the projections, rotation and a unit norm of queries and keys, a penalty on distance, heads that mix their
weights, a gate per head."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.specs import Bundle, PagedHeads, States
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, build_part, register_part
from .linear import linear


class SinkAttention(Part):
    """q = Wq h (heads x dim), k = Wk h (kv_heads x dim), v = Wv h (kv_heads x vdim), no biases; query head a reads
    key/value head a // (heads / kv_heads).  In this order, each optional:

    conv_taps   a causal convolution over time on every channel of q, k and v (``q.conv``, ``k.conv``, ``v.conv``:
                [channels, taps], the last tap the current token's); the last taps - 1 projected rows are the request's state
    position    a rotary part: q and k turned by position
    unit_norm   q and k divided by sqrt(mean(head^2) + eps) per head, after the rotation, no weight
    distance    the score loses r1_a ln(1 + r2_a (p - j))  (``r1``, ``r2``: a number a head)
    sink        exp(sink_a) joins head a's denominator: no key, no value, not scaled, counted once
    talking     the heads' finished weights are mixed, w'_a = sum_g talk[a, g] w_g, before they meet the values of a's own
                key/value head (the sink has no weight of its own and is not mixed)
    head_gate   head a's output is multiplied by sigmoid(Wg h)_a (``g``: [heads, hidden])

    score = (q . k) * scale over the keys j with 0 <= p - j < window (window 0: all).  Scores, weights and sums are float32;
    keys and values are cached as they enter the scores (rotated, normed).

    Further parameters, each alone or with the others (not with mixed weights or a head gate):

    bias        ``q.b``, ``k.b``, ``v.b`` are added to the projections
    values      "keys": there is no Wv -- a value head is its key head straight out of the product (what the keys go through afterwards does not touch it), vdim = dim
    row_norm    q and k are normed across all their heads together (one mean square a token), each with a weight as wide as the row
                (``q.norm`` [heads * dim], ``k.norm`` [kv_heads * dim]), before the rotation
    value_unit_norm  every value head divided by sqrt(mean(head^2) + eps), no weight; cached so
    block       instead of the window: a row sees the keys j <= p of its own block of ``block`` positions, counted from the
                sequence's first token (wherever a prompt was cut)
    cap         the scaled score becomes cap tanh(score / cap)
    sink        "unit": the sink is the number 1 in every head's denominator, exp(0), and no tensor
    weights     "sigmoid": no softmax and no sink -- a visible key weighs sigmoid(score + ``pb``[a]) by itself"""
    category = "mixer"
    graph_safe = True     # launches kernels only: may run inside a captured graph
    adds_one_product = True   # the output is one last product through linear(): a block may hand it ops.Fresh

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float = 0.0,
                 window: int = 0, conv_taps: int = 0, position=None, unit_norm: bool = False, sink: bool = True,
                 distance: bool = False, talking: bool = False, head_gate: bool = False, bias: bool = False,
                 values: str = "projected", row_norm: bool = False, value_unit_norm: bool = False, block: int = 0,
                 cap: float = 0.0, weights: str = "softmax"):
        if values not in ("projected", "keys") or weights not in ("softmax", "sigmoid") or sink not in (True, False, "unit", "learned"):
            raise ConfigError(f"sink attention: values {values!r} ('projected' or 'keys'), weights {weights!r} ('softmax' or "
                              f"'sigmoid'), sink {sink!r} (true, false or 'unit')")
        if block < 0 or cap < 0 or (block > 0 and window > 0):
            raise ConfigError(f"sink attention: block {block} and cap {cap} must not be negative, and a block mask stands "
                              f"instead of a window ({window})")
        if values == "keys" and (dim != vdim or conv_taps):
            raise ConfigError(f"sink attention: values taken from the key product have the keys' size ({dim}, not {vdim}) "
                              "and no convolution behind the projections")
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads:
            raise ConfigError(f"sink attention: {heads} heads cannot share {kv_heads} key/value heads")
        if window < 0 or conv_taps < 0:
            raise ConfigError(f"sink attention: window {window} and convolution taps {conv_taps} must not be negative")
        if not (0 < dim <= ops.HEADS_MAX_DIM and 0 < vdim <= ops.HEADS_MAX_DIM):
            raise ConfigError(f"sink attention: dim {dim} and vdim {vdim} must lie in 1..{ops.HEADS_MAX_DIM}")
        self.hidden_size, self.heads, self.kv_heads = int(hidden_size), int(heads), int(kv_heads)
        self.dim, self.vdim, self.scale, self.eps, self.window = int(dim), int(vdim), float(scale), float(eps), int(window)
        self.conv_taps = int(conv_taps) if conv_taps and int(conv_taps) > 0 else 0
        self.unit_norm, self.distance = bool(unit_norm), bool(distance)
        self.squash = weights == "sigmoid"
        self.unit_sink = sink == "unit" and not self.squash
        self.sink = bool(sink) and not self.unit_sink and not self.squash        # (a learned sink: a tensor)
        self.talking, self.head_gate = bool(talking), bool(head_gate)
        self.bias, self.own_values, self.row_norm = bool(bias), values == "projected", bool(row_norm)
        self.value_unit_norm, self.block, self.cap = bool(value_unit_norm), int(block), float(cap)
        self.position = build_part("position", position) if position is not None else None
        if self.position is not None and not hasattr(self.position, "table"):
            raise ConfigError("sink attention: the position part must give a table of cosines and sines")
        if self.position is not None and getattr(self.position, "dim", 0) > self.dim:
            raise ConfigError(f"sink attention: {self.position.dim} rotated elements of a head of {self.dim}")
        # heads that mix their weights or carry a gate of their own go through the kernel that walks a row's heads together
        self.together = self.talking or self.head_gate
        if self.together and not ops.attention_talk_takes(self.heads, self.dim, self.vdim):
            raise ConfigError(f"sink attention: {self.heads} heads of {self.dim} whose weights are mixed are beyond the kernel "
                              f"(at most {ops.TALK_MAX_HEADS} heads, heads x dim rounded up within {ops.TALK_MAX_QUERIES})")
        if self.together and (self.bias or not self.own_values or self.row_norm or self.value_unit_norm or self.block
                              or self.cap or self.squash or self.unit_sink):
            raise ConfigError("sink attention: heads that mix their weights or carry a gate take none of bias, values 'keys', "
                              "row_norm, value_unit_norm, block, cap, a unit sink or sigmoid weights")
        self.channels = (self.heads + self.kv_heads) * self.dim + (self.kv_heads * self.vdim if self.own_values else 0)

    def children(self):
        return [self.position] if self.position is not None else []

    def cache_spec(self):
        kv = PagedHeads(self.kv_heads, self.dim, self.kv_heads, self.vdim, self.window, 0, self.block)
        if not self.conv_taps or self.conv_taps == 1:
            return kv
        return Bundle((("kv", kv), ("conv", States((("tail", (self.conv_taps - 1, self.channels), None),)))))

    def weight_specs(self) -> Dict[str, WeightSpec]:
        H, G, d, e, h = self.heads, self.kv_heads, self.dim, self.vdim, self.hidden_size
        vec = lambda *shape: WeightSpec(tuple(shape), kind="vector")      # noqa: E731
        out = {"q": WeightSpec((H * d, h)), "k": WeightSpec((G * d, h)), "o": WeightSpec((h, H * e))}
        if self.own_values:
            out["v"] = WeightSpec((G * e, h))
        if self.bias:
            out.update({"q.b": vec(H * d), "k.b": vec(G * d)})
            if self.own_values:
                out["v.b"] = vec(G * e)
        if self.row_norm:
            out.update({"q.norm": vec(H * d), "k.norm": vec(G * d)})
        if self.squash:
            out["pb"] = vec(H)
        if self.conv_taps:
            out.update({"q.conv": vec(H * d, self.conv_taps), "k.conv": vec(G * d, self.conv_taps), "v.conv": vec(G * e, self.conv_taps)})
        if self.sink:
            out["sink"] = vec(H)
        if self.distance:
            out.update({"r1": vec(H), "r2": vec(H)})
        if self.talking:
            out["talk"] = vec(H, H)
        if self.head_gate:
            out["g"] = WeightSpec((H, h))
        return out

    def bind(self, tensors, rt) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()      # noqa: E731
        names = ["q", "k"] + (["v"] if self.own_values else []) + (["g"] if self.head_gate else [])
        self.w_in = ops.StreamedWeight(torch.cat([tensors[n] for n in names], dim=0).contiguous())
        self.w_o = ops.StreamedWeight(tensors["o"])
        self.conv_w = None
        if self.conv_taps:      # by taps, the channels of q, k and v side by side as in the product's rows
            self.conv_w = torch.cat([f32(n + ".conv") for n in ("q", "k", "v")], dim=0).t().contiguous()
        self.sink_w = f32("sink") if self.sink else None
        if self.unit_sink:                   # exp(0) in every head's denominator
            self.sink_w = torch.zeros(self.heads, dtype=torch.float32, device=tensors["q"].device)
        self.point_w = f32("pb") if self.squash else None
        self.q_b, self.k_b = (f32("q.b"), f32("k.b")) if self.bias else (None, None)
        self.v_b = (f32("v.b") if self.own_values else self.k_b) if self.bias else None
        self.q_norm, self.k_norm = (f32("q.norm"), f32("k.norm")) if self.row_norm else (None, None)
        self.far = (f32("r1"), f32("r2")) if self.distance else None
        self.talk_w = f32("talk") if self.talking else None
        self.act_dtype = rt.act_dtype

    def _pairs(self, batch):
        """(query-key pairs, keys read) of a step."""
        pairs = keys = 0
        for s in range(batch.n_seqs):
            cached, new = int(batch.seq_ctx[s]), int(batch.seq_start[s + 1] - batch.seq_start[s])
            if self.block > 0:
                pairs += sum((cached + i) % self.block + 1 for i in range(new))
                keys += min(cached + new, cached % self.block + new)
            elif self.window > 0:
                pairs += sum(min(self.window, cached + i + 1) for i in range(new))
                keys += min(cached + new, self.window + new - 1)
            else:
                pairs += new * cached + new * (new + 1) // 2
                keys += cached + new
        return pairs, keys

    def step_work(self, batch, rows: int, elem: int):
        """The products' work, plus attention's own: per visible key and query head a product of dim and one of vdim (and,
        where the heads mix their weights, one of heads), and every visible key and value read once per request."""
        flops, nbytes = super().step_work(batch, rows, elem)
        pairs, keys = self._pairs(batch)
        mixing = self.heads if self.talking else 0
        return (flops + 2.0 * pairs * self.heads * (self.dim + self.vdim + mixing) + 2.0 * rows * self.channels * self.conv_taps,
                nbytes + keys * self.kv_heads * (self.dim + self.vdim) * elem)

    def working_bytes_per_row(self, elem: int) -> float:
        return super().working_bytes_per_row(elem) + self.channels * elem + self.heads * (4 * self.dim + self.vdim * elem)

    def forward(self, h, ctx, cache, residual, writes: bool = True) -> None:
        H, G, d, e, t = self.heads, self.kv_heads, self.dim, self.vdim, h.shape[0]
        x = linear(h, self.w_in, out_dtype=self.act_dtype)
        nq, nk, nv = H * d, G * d, G * e
        gate = x[:, nq + nk + nv:] if self.head_gate else None
        kv = cache
        qkv = x
        if self.conv_taps:
            tail = cache.conv.tail if self.conv_taps > 1 else None
            kv = cache.kv if self.conv_taps > 1 else cache
            qkv = ops.causal_conv(x[:, :self.channels] if self.head_gate else x, self.conv_w, tail, ctx)
        q, k = qkv[:, :nq], qkv[:, nq:nq + nk]
        v = qkv[:, nq + nk:nq + nk + nv] if self.own_values else k      # (else the key product's columns, untouched)
        table = self.position.table(ctx) if self.position is not None else None
        turn = dict(table=table, neighbours=bool(getattr(self.position, "neighbours", False)), unit_after=self.unit_norm, eps=self.eps,
                    norm_rows=self.row_norm)
        q_heads = torch.empty((t, H, d), dtype=torch.float32, device=x.device)
        # queries dense in float32, keys and values straight into their pages: one launch for the three
        sections = [ops.heads_section(q, H, d, q_heads, bias=self.q_b, norm_weight=self.q_norm, **turn)]
        if writes:
            slots = ctx.slot_maps[kv.group]
            sections.append(ops.heads_section(k, G, d, kv.k, slot_map=slots, page_tokens=kv.page_tokens, bias=self.k_b,
                                              norm_weight=self.k_norm, **turn))
            sections.append(ops.heads_section(v, G, e, kv.v, slot_map=slots, page_tokens=kv.page_tokens, bias=self.v_b,
                                              unit_after=self.value_unit_norm, eps=self.eps))
        ops.heads_prepare_many(sections)
        if self.together:
            o = ops.attention_talk(q_heads, kv.k, kv.v, ctx.block_tables[kv.group], ctx, self.act_dtype, H, G, d, e, self.window,
                                   self.scale, sink=self.sink_w, far=self.far, talk=self.talk_w, gate=gate)
        else:
            o = ops.attention_maps(q_heads.view(t, H, 1, d), kv.k, kv.v, ctx.block_tables[kv.group], ctx, self.act_dtype, H, G, 1,
                                   d, e, self.window, 0, self.scale, sink=self.sink_w, far=self.far, block=self.block, cap=self.cap,
                                   point=self.point_w)
        linear(o, self.w_o, accumulate_into=residual, ctx=ctx)


register_part("mixer", "sink_attention", SinkAttention)
