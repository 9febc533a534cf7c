"""How a layer's parts are arranged around the residual stream."""
from __future__ import annotations

import torch

from typing import Dict

import torch

from ..cache.specs import Bundle
from ..csrc import ops
from ..errors import ConfigError
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .lazy import Normed
from .streams import StreamReader


class LayerScale(Part):
    """One learned number a channel by which a sublayer's output is multiplied, element by element and in float32, before it
    joins the residual stream: x += a * f(N(x))."""
    category = "scale"
    graph_safe = True

    def __init__(self, size: int):
        self.size = int(size)
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.size,), kind="vector", init="ones")}

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"].to(torch.float32).contiguous()

    def add_to(self, x: torch.Tensor, y: torch.Tensor, next_norm=None):
        """x += weight * y on the float32 stream; with a norm that can follow an update in the same kernel
        (``after_update``), also that norm of the new x -- else None."""
        if next_norm is not None and hasattr(next_norm, "after_update"):
            return next_norm.after_update(x, y, scale=self.weight)
        ops.stream_update(x, y, scale=self.weight)
        return None


class PreNormBlock(Part):
    """x += mixer(norm(x)); x += ffn(norm(x))  (reference: engine/src/model.cpp:526-604).
    The residual stream x is float32 and is updated in place.  A layer may have no feed-forward, and the mixer may read
    its input through a part that mixes every row with the row before it (``mixer_shift``, a conv part with a state of
    its own: the layer then keeps that state beside its mixer's cache).  With ``mixer_scale`` / ``ffn_scale`` (scale parts)
    a sublayer's output is gathered in float32 and multiplied by one number a channel before it is added; the kernel
    that adds it also norms the stream for whoever reads it next."""
    category = "block"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, mixer, ffn, mixer_norm, ffn_norm, mixer_shift=None, mixer_scale=None, ffn_scale=None):
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm, self.mixer_shift = mixer, ffn, mixer_norm, ffn_norm, mixer_shift
        self.mixer_scale, self.ffn_scale = mixer_scale, ffn_scale
        for part, scale in ((mixer, mixer_scale), (ffn, ffn_scale)):
            if scale is not None and (part is None or not getattr(part, "adds_one_product", False)):
                raise ConfigError("prenorm block: a scaled sublayer must give its output as one last product (adds_one_product)")

    def children(self):
        parts = (self.mixer_norm, self.mixer_shift, self.mixer, self.mixer_scale, self.ffn_norm, self.ffn, self.ffn_scale)
        return [p for p in parts if p is not None]

    def _scaled(self, scale, run, x, ctx) -> None:
        """A sublayer whose output is scaled: ``run(y)`` leaves it in float32 (y an ops.Fresh), then x += scale * y, and the
        norm of whoever reads the stream next with it."""
        y = ops.Fresh()
        run(y)
        reading = ctx.handoff.reading_next
        norm = reading[0] if reading is not None else None
        made = scale.add_to(x, y.tensor, norm)
        if made is not None:
            ctx.handoff.leave(norm, ops.Finished(made))

    def cache_spec(self):
        """The mixer's cache, and beside it the state of the shift in front of the mixer."""
        if self.mixer_shift is None:
            return self.mixer.cache_spec()
        return Bundle((("mixer", self.mixer.cache_spec()), ("shift", self.mixer_shift.cache_spec())))

    def forward(self, x, ctx, cache, writes: bool = True) -> None:
        # Each part is told which norm reads the stream after it, so that its last product can prepare that
        # norm: the feed-forward's after the mixer, the next entry's first after the feed-forward.
        handoff, n = ctx.handoff, x.shape[0]
        after_mixer = (self.ffn_norm, self._wants_prepared(self.ffn, n)) if self.ffn is not None else (handoff.next_entry or (None, False))
        with handoff.reader(*after_mixer):
            if self.mixer_shift is not None:
                pre = handoff.take(self.mixer_norm)
                if isinstance(pre, ops.Finished):
                    h = self.mixer_shift.forward(pre.tensor, ctx, cache.shift)
                elif hasattr(self.mixer_shift, "after"):       # (norm and shift in one kernel where the two know how)
                    h = self.mixer_shift.after(self.mixer_norm, x, ctx, cache.shift)
                else:
                    h = self.mixer_shift.forward(self.mixer_norm.forward(x, ctx), ctx, cache.shift)
                mixer_cache = cache.mixer
            else:
                h, mixer_cache = self._normed(self.mixer, self.mixer_norm, x, ctx), cache
            if self.mixer_scale is not None:
                self._scaled(self.mixer_scale, lambda y: self.mixer.forward(h, ctx, mixer_cache, y, writes), x, ctx)
            else:
                self.mixer.forward(h, ctx, mixer_cache, x, writes)
        if self.ffn is None:
            return
        with handoff.reader(*(handoff.next_entry or (None, False))):
            h = self._normed(self.ffn, self.ffn_norm, x, ctx)
            if self.ffn_scale is not None:
                self._scaled(self.ffn_scale, lambda y: self.ffn.forward(h, ctx, y), x, ctx)
            else:
                self.ffn.forward(h, ctx, x)

    def first_reader(self, n_rows: int):
        """(the norm this block begins with, whether its reader takes the parts of a prepared norm for a step of
        ``n_rows`` rows): what the entry before may prepare."""
        return self.mixer_norm, self._wants_prepared(self.mixer, n_rows)

    @staticmethod
    def _wants_prepared(part, n_rows: int) -> bool:
        """Whether the part's first product is better served by a prepared norm than by fusing the
        norm or running it (parts that do not say are not: nothing is prepared for them)."""
        wants = getattr(part, "wants_prepared_norm", None)
        return bool(wants(n_rows)) if wants is not None else False

    @staticmethod
    def _normed(part, norm, x, ctx):
        """The part's input: the norm's result, or -- for a part that says it takes one -- the
        norm not yet computed, so that the part's first product can absorb it (or take what the
        product before has prepared for it)."""
        pre = ctx.handoff.take(norm)
        if isinstance(pre, ops.Finished):
            return Normed(x, norm, ctx, done=pre.tensor) if getattr(part, "accepts_lazy_norm", False) else pre.tensor
        if getattr(part, "accepts_lazy_norm", False):
            return Normed(x, norm, ctx, pre=pre)
        return norm.forward(x, ctx)


class SandwichBlock(Part):
    """Every sublayer normed on both sides: x += post(mixer(pre(x))); x += post(ffn(pre(x))).  The mixer may read
    h + conv(h) instead of h = pre(x) (``mixer_conv``: a causal convolution over time whose tail is part of the
    request's state), and a layer may have no feed-forward.  The sublayer's output is gathered in float32 and its
    norm is added to the float32 stream in one kernel."""
    category = "block"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, mixer, mixer_norm, mixer_post_norm, ffn=None, ffn_norm=None, ffn_post_norm=None, mixer_conv=None):
        self.mixer, self.mixer_norm, self.mixer_post_norm = mixer, mixer_norm, mixer_post_norm
        self.ffn, self.ffn_norm, self.ffn_post_norm, self.mixer_conv = ffn, ffn_norm, ffn_post_norm, mixer_conv

    def children(self):
        parts = [self.mixer_norm, self.mixer_conv, self.mixer, self.mixer_post_norm, self.ffn_norm, self.ffn, self.ffn_post_norm]
        return [p for p in parts if p is not None]

    def cache_spec(self):
        """The mixer's cache, and beside it the tail of the convolution in front of the mixer."""
        if self.mixer_conv is None:
            return self.mixer.cache_spec()
        return Bundle((("mixer", self.mixer.cache_spec()), ("conv", self.mixer_conv.cache_spec())))

    def forward(self, x, ctx, cache, writes: bool = True) -> None:
        h = self.mixer_norm.forward(x, ctx)
        mixer_cache = cache
        if self.mixer_conv is not None:
            h = self.mixer_conv.forward(h, ctx, cache.conv, add_input=True)
            mixer_cache = cache.mixer
        y = self._sum_for(self.mixer, x)
        self.mixer.forward(h, ctx, mixer_cache, y, writes)
        self.mixer_post_norm.add_to(x, self._sum_of(y))
        if self.ffn is not None:
            y = self._sum_for(self.ffn, x)
            # (a feed-forward that says so gets the norm not yet computed: its first product absorbs it for few rows)
            lazy = getattr(self.ffn, "accepts_lazy_norm", False)
            self.ffn.forward(Normed(x, self.ffn_norm, ctx) if lazy else self.ffn_norm.forward(x, ctx), ctx, y)
            self.ffn_post_norm.add_to(x, self._sum_of(y))

    @staticmethod
    def _sum_for(part, x):
        """What the part adds its output to: nothing yet (ops.Fresh) for a part that says its output is one last product
        through parts.linear.linear (``adds_one_product``), else a cleared buffer."""
        return ops.Fresh() if getattr(part, "adds_one_product", False) else torch.zeros_like(x)

    @staticmethod
    def _sum_of(y):
        return y.tensor if isinstance(y, ops.Fresh) else y


class HyperBlock(Part):
    """Pre-norm sublayers on a residual stream kept in several copies x [T, n, H]: each sublayer reads one weighted sum
    of the copies through its norm and writes all copies at once (parts.streams.HyperConnection):
    y = mixer(norm1(read1(x))); x = write1(x, y); then the same with the feed-forward, if the layer has one.  The read
    of whoever comes next -- this layer's feed-forward, the next layer's mixer -- is made by the write before it."""
    category = "block"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, mixer, mixer_norm, mixer_conn, ffn=None, ffn_norm=None, ffn_conn=None):
        self.mixer, self.mixer_norm, self.mixer_conn = mixer, mixer_norm, mixer_conn
        self.ffn, self.ffn_norm, self.ffn_conn = ffn, ffn_norm, ffn_conn
        self.mixer_reader = StreamReader(mixer_conn, mixer_norm)
        self.ffn_reader = StreamReader(ffn_conn, ffn_norm) if ffn is not None else None

    def children(self):
        parts = [self.mixer_conn, self.mixer_norm, self.mixer, self.ffn_conn, self.ffn_norm, self.ffn]
        return [p for p in parts if p is not None]

    @staticmethod
    def _sum_for(part, x):
        """What the part adds its output [T, H] to: nothing yet for a part whose output is one last product, else a cleared buffer."""
        if getattr(part, "adds_one_product", False):
            return ops.Fresh()
        return torch.zeros((x.shape[0], x.shape[2]), dtype=torch.float32, device=x.device)

    def first_reader(self, n_rows: int):
        """What the entry before may prepare: this block's first input (a reader that takes no parts of an RMSNorm)."""
        return self.mixer_reader, False

    def forward(self, x, ctx, cache, writes: bool = True) -> None:
        handoff = ctx.handoff
        if x.dim() == 2:              # a plain stream is one copy
            x = x.unsqueeze(1)
        h = handoff.take(self.mixer_reader)
        if h is None:
            h = self.mixer_conn.read(x, self.mixer_norm, ctx)
        following = handoff.next_entry[0] if handoff.next_entry is not None else None
        if not isinstance(following, StreamReader) or following.connection.streams != self.mixer_conn.streams:
            following = None
        y = self._sum_for(self.mixer, x)
        self.mixer.forward(h, ctx, cache, y, writes)
        if self.ffn is None:
            last_conn = self.mixer_conn
        else:
            h = self.mixer_conn.write(x, SandwichBlock._sum_of(y), self.ffn_reader, ctx)
            y = self._sum_for(self.ffn, x)
            self.ffn.forward(h, ctx, y)
            last_conn = self.ffn_conn
        made = last_conn.write(x, SandwichBlock._sum_of(y), following, ctx)
        if following is not None:
            handoff.leave(following, made)


register_part("scale", "layer_scale", LayerScale)
register_part("block", "prenorm", PreNormBlock)
register_part("block", "hyper", HyperBlock)
register_part("block", "sandwich", SandwichBlock)
