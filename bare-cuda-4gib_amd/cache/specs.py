"""What a mixer asks of the cache manager.

A cache spec says what is kept and in which tensors; the manager allocates them and does the
bookkeeping, and knows no spec by name.  Two kinds:

per token   ``per_token = True``.  ``page_tensors(page_tokens)`` names the tensors of ONE page
            (name -> shape, or name -> (shape, dtype name) for a tensor that is not in the cache's
            own dtype); the manager allocates ``[num_pages, *shape]`` of each.  When its tokens may be
            given back the spec says itself: ``first_kept(length)`` is the earliest token that any
            query at position ``length`` or later still reads (0: every token is kept), and pages
            wholly before it go back to their pool; ``group_key()`` names the rule -- specs with equal
            keys share a page pool and one block table per request.  A spec that has neither is read
            by its ``window`` (0 or absent = keep everything; W = a query reads the W tokens up to and
            including its own).  ``always_kept()`` (optional) is the number of leading tokens that stay
            whatever ``first_kept`` says: the pages that hold them are never given back before the request ends.
per request ``per_token = False``.  ``slot_tensors()`` names the tensors of ONE request slot
            (name -> (shape, dtype name)); the manager allocates ``[max_requests, *shape]`` of each and
            zeroes a slot when a request is admitted to it.

several     ``members`` names further specs (:class:`Bundle`): a layer that keeps more than one thing -- its mixer's
            cache and the tail of a convolution in front of it, say.  The manager handles every member as a stream
            of its own and hands out one view whose attributes are the members' views.

A mixer gets a :class:`View` of its stream: the tensors by name (``view.k``, ``view.state``, ...) and,
for a paged stream, ``group`` (the key of its block table and slot map in the step's context),
``page_tokens`` and ``window``.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values per token, in pages.  ``window`` 0 keeps every token;
    otherwise only the last ``window`` tokens are ever read again, and pages
    that a request's window has passed are given back.  Keys lie
    ``[page, kv_head, token, dim]``, values transposed ``[page, kv_head, dim, token]``
    (consecutive tokens of one dimension lie together)."""
    num_kv_heads: int
    head_dim: int
    window: int = 0
    per_token = True

    def page_tensors(self, page_tokens: int) -> Dict[str, Tuple[int, ...]]:
        return {"k": (self.num_kv_heads, page_tokens, self.head_dim),
                "v": (self.num_kv_heads, self.head_dim, page_tokens)}

    def group_key(self):
        return ("window", self.window)

    def first_kept(self, length: int) -> int:
        """The query at position ``length`` reads keys from ``length - window + 1`` on."""
        return max(0, length - self.window + 1) if self.window > 0 else 0


@dataclasses.dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (any shape), zeroed when the request is
    admitted, kept across its steps, dropped when it ends."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
    per_token = False

    def slot_tensors(self) -> Dict[str, Tuple[Tuple[int, ...], str]]:
        return {"state": (tuple(self.shape), self.dtype)}


@dataclasses.dataclass(frozen=True)
class PagedLatent:
    """One row of ``rank + rot`` numbers per token, in pages, shared by all heads: a low-rank latent from which keys
    and values are made, followed by a rotated key part.  Rows lie ``[page, token, rank + rot]``.  ``window`` as for
    :class:`PagedKV`."""
    rank: int
    rot: int
    window: int = 0
    per_token = True

    def page_tensors(self, page_tokens: int) -> Dict[str, Tuple[int, ...]]:
        return {"latent": (page_tokens, self.rank + self.rot)}

    def group_key(self):
        return ("window", self.window)

    def first_kept(self, length: int) -> int:
        return max(0, length - self.window + 1) if self.window > 0 else 0


@dataclasses.dataclass(frozen=True)
class PagedHeads:
    """Keys and values per token, in pages, with head counts and sizes of their own: keys
    ``[page, key_heads, token, key_dim]``, values ``[page, value_heads, token, value_dim]`` (a token's elements side by
    side in both).  ``window`` 0 keeps every token; otherwise a query reads the last ``window`` tokens and, whatever its
    position, the first ``keep_first`` tokens of the sequence: pages between those and the window are given back.
    ``block`` (instead of a window): a query reads the keys of its own block of that many positions, counted from the
    sequence's first token; pages wholly before the current block are given back."""
    key_heads: int
    key_dim: int
    value_heads: int
    value_dim: int
    window: int = 0
    keep_first: int = 0
    block: int = 0
    per_token = True

    def page_tensors(self, page_tokens: int) -> Dict[str, Tuple[int, ...]]:
        return {"k": (self.key_heads, page_tokens, self.key_dim), "v": (self.value_heads, page_tokens, self.value_dim)}

    def group_key(self):
        if self.block > 0:
            return ("block", self.block)
        if self.window <= 0 or self.keep_first <= 0:
            return ("window", max(self.window, 0))
        return ("window", self.window, "first", self.keep_first)

    def first_kept(self, length: int) -> int:
        if self.block > 0:
            return length - length % self.block
        return max(0, length - self.window + 1) if self.window > 0 else 0

    def always_kept(self) -> int:
        """The leading tokens that every later query reads, wherever the window stands."""
        return self.keep_first if self.window > 0 else 0


@dataclasses.dataclass(frozen=True)
class States:
    """Several per-request tensors of fixed size under names of their own: ``tensors`` is a tuple of
    (name, shape, dtype name or None for the cache's own dtype).  Zeroed at admission like :class:`FixedState`."""
    tensors: Tuple[Tuple[str, Tuple[int, ...], Optional[str]], ...]
    per_token = False

    def slot_tensors(self) -> Dict[str, Any]:
        return {name: (tuple(shape), dtype) if dtype is not None else tuple(shape) for name, shape, dtype in self.tensors}


@dataclasses.dataclass(frozen=True)
class Bundle:
    """What a layer keeps when it keeps more than one thing: ``members`` is a tuple of (name, spec), every spec one of
    the kinds above (or None).  The layer's view has an attribute for every name."""
    members: Tuple[Tuple[str, Any], ...]
