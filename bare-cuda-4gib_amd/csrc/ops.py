"""The kernels as functions of torch tensors.

Each wrapper checks on the host that shapes, dtypes, devices and strides are
what the kernel and its grid assume, then launches on torch's current stream.
There is no other implementation behind these functions: without the kernel
library, or on a CPU tensor, they raise.
"""
from __future__ import annotations

import ctypes
import dataclasses
import math
from typing import Dict, Optional, Tuple

import torch

from ..errors import KernelError
from . import library

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _dev(what: str, *tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError(f"{what}: tensors must be on the GPU (got {t.device}); there is no CPU path")
        if not t.is_contiguous():
            raise KernelError(f"{what}: tensors must be contiguous (got strides {t.stride()} for shape {tuple(t.shape)})")


def _i32(what: str, name: str, t: torch.Tensor, n: int) -> None:
    if t.dtype != torch.int32 or t.numel() < n:
        raise KernelError(f"{what}: {name} must be int32 with at least {n} elements, got {t.dtype} x {t.numel()}")


def _stream() -> int:
    """The current stream's handle (asked for at every launch: a step runs a few hundred of them, so
    by the short way, without a Stream object)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _gemm_cost(m: int, n: int, k: int, in_bytes: int, w_bytes: int, out_bytes: float, x_readers: int = 1,
               w_readers: int = 1):
    """(operations, bytes moved at least, bytes asked for in all) of an [m, k] x [n, k]^T product; out_bytes per
    output element.  x_readers / w_readers: how many workgroups read every element of x / of w (the
    weight-streaming kernel: every block of 16 columns reads all the rows; the tiled kernel: every row of
    tiles reads all the weights, every column of tiles all the rows)."""
    ideal = m * k * in_bytes + n * k * w_bytes + m * n * out_bytes
    moved = x_readers * m * k * in_bytes + w_readers * n * k * w_bytes + m * n * out_bytes
    return lambda: (2.0 * m * n * k, ideal, moved)


def _skinny_cost(m: int, n: int, k: int, in_bytes: int, out_bytes: float):
    return _gemm_cost(m, n, k, in_bytes, 2, out_bytes, x_readers=-(-n // 16))


def tiled_tile(m: int, n: int, k: int, a_ptr: int = 0, w_ptr: int = 0, qkv: bool = False) -> Tuple[int, int]:
    """(rows, columns) of the output tile the tiled matrix-core kernel takes for an [m, k] x [n, k]^T product of
    operands at these addresses (0: well aligned); ``qkv``: the product with rotation and cache write after it."""
    rows, cols = ctypes.c_int(0), ctypes.c_int(0)
    library.call("bc4g_gemm_mfma_tile", a_ptr or None, w_ptr or None, m, n, k, int(qkv), ctypes.byref(rows),
                 ctypes.byref(cols), launches=False)
    return rows.value, cols.value


def _tiled_cost(m: int, n: int, k: int, out_bytes: float, qkv: bool = False):
    def cost():                                    # asked for by the profiler only: the tile is looked up then
        rows, cols = tiled_tile(m, n, k, qkv=qkv)
        return _gemm_cost(m, n, k, 2, 2, out_bytes, x_readers=-(-n // cols), w_readers=-(-m // rows))()
    return cost


def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, factor: float = 1.0) -> torch.Tensor:
    """out[t, :] = float(table[ids[t], :]) * factor; ids must already be known to lie in [0, vocab)."""
    _dev("embed_gather", table, ids, out)
    vocab, hidden = table.shape
    n = ids.numel()
    _i32("embed_gather", "ids", ids, n)
    if out is None:
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    elif out.dtype != torch.float32 or tuple(out.shape) != (n, hidden):
        raise KernelError(f"embed_gather: out must be float32 [{n}, {hidden}]")
    cost = lambda: (0.0, n * hidden * (table.element_size() + 4))      # noqa: E731
    if factor == 1.0:
        library.call("bc4g_embed_gather", _ptr(table), _code(table, "embed_gather"), _ptr(ids), _ptr(out), n, hidden, vocab, _stream(),
                     cost=cost)
    else:
        library.call("bc4g_embed_rows", _ptr(table), _code(table, "embed_gather"), _ptr(ids), _ptr(out), n, hidden, vocab, float(factor),
                     0, _stream(), cost=cost)
    return out


def embed_add(table: torch.Tensor, ids: torch.Tensor, x: torch.Tensor, factor: float = 1.0) -> torch.Tensor:
    """x[t, :] += float(table[ids[t], :]) * factor in place on the float32 stream x [T, H]."""
    _dev("embed_add", table, ids, x)
    vocab, hidden = table.shape
    n = ids.numel()
    _i32("embed_add", "ids", ids, n)
    if x.dtype != torch.float32 or tuple(x.shape) != (n, hidden) or not x.is_contiguous():
        raise KernelError(f"embed_add: x must be float32 [{n}, {hidden}], got {x.dtype} {tuple(x.shape)}")
    cost = lambda: (1.0 * n * hidden, n * hidden * (table.element_size() + 8))      # noqa: E731
    if factor == 1.0:
        library.call("bc4g_embed_add", _ptr(table), _code(table, "embed_add"), _ptr(ids), _ptr(x), n, hidden, vocab, _stream(), cost=cost)
    else:
        library.call("bc4g_embed_rows", _ptr(table), _code(table, "embed_add"), _ptr(ids), _ptr(x), n, hidden, vocab, float(factor), 1,
                     _stream(), cost=cost)
    return x


def embed_beside(x: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, out_dtype: torch.dtype, factor: float = 1.0) -> torch.Tensor:
    """[T, 2 H] in ``out_dtype``: row t is the float32 stream's row x[t, :] followed by table[ids[t], :] * factor -- the
    operand of a product over the stream and the embedding of the same token."""
    _dev("embed_beside", x, table, ids)
    vocab, hidden = table.shape
    n = ids.numel()
    _i32("embed_beside", "ids", ids, n)
    if x.dtype != torch.float32 or tuple(x.shape) != (n, hidden):
        raise KernelError(f"embed_beside: x must be float32 [{n}, {hidden}], got {x.dtype} {tuple(x.shape)}")
    out = torch.empty((n, 2 * hidden), dtype=out_dtype, device=x.device)
    library.call("bc4g_embed_beside", _ptr(x), _ptr(table), _code(table, "embed_beside"), _ptr(ids), float(factor), _ptr(out),
                 _code(out, "embed_beside"), n, hidden, vocab, _stream(),
                 cost=lambda: (1.0 * n * hidden, n * hidden * (4 + table.element_size() + 2 * out.element_size())))
    return out


def stream_update(x: torch.Tensor, y: torch.Tensor, scale: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                  keep: bool = True, norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0, groups: int = 1,
                  out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """x = (x if keep else 0) + scale * y + bias in place on the float32 stream x [T, H]; y float32 [T, H]; scale and bias
    float32 [H] (absent: 1 and 0).  With ``norm_weight`` [H] the new x's norm in ``groups`` parts (see rmsnorm) is returned in
    ``out_dtype`` -- what the stream's next reader would compute."""
    _dev("stream_update", x, y, scale, bias, norm_weight)
    if x.dtype != torch.float32 or x.dim() != 2 or y.dtype != torch.float32 or y.shape != x.shape or y.data_ptr() == x.data_ptr():
        raise KernelError(f"stream_update: x and y must be two float32 [T, H] tensors, got {x.dtype} {tuple(x.shape)} and "
                          f"{y.dtype} {tuple(y.shape)}")
    t, hidden = x.shape
    _f32("stream_update", "scale", scale, (hidden,))
    _f32("stream_update", "bias", bias, (hidden,))
    if groups <= 0 or hidden % groups:
        raise KernelError(f"stream_update: {hidden} channels do not fall into {groups} equal groups")
    out = None
    if norm_weight is not None:
        if tuple(norm_weight.shape) != (hidden,):
            raise KernelError(f"stream_update: the norm's weight must be [{hidden}], got {tuple(norm_weight.shape)}")
        out = torch.empty((t, hidden), dtype=out_dtype or torch.float32, device=x.device)
    library.call("bc4g_stream_update", _ptr(x), _ptr(y), _ptr(scale), _ptr(bias), 1 if keep else 0, _ptr(norm_weight),
                 _code(norm_weight, "stream_update") if norm_weight is not None else F32, _ptr(out),
                 _code(out, "stream_update") if out is not None else F32, t, hidden, int(groups), float(eps), _stream(),
                 cost=lambda: (6.0 * t * hidden, t * hidden * (12 + (out.element_size() if out is not None else 0))))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None, n_rows: Optional[int] = None, groups: int = 1) -> torch.Tensor:
    """RMSNorm of rows of the float residual stream x [T, H]; with ``rows`` (int32
    indices, the first n_rows are used) only those rows are normed.  ``groups``: a row is that many equal runs of
    neighbouring channels, each brought to unit mean square by itself; the weight spans the row."""
    _dev("rmsnorm", x, weight, rows)
    if x.dtype != torch.float32 or x.dim() != 2:
        raise KernelError(f"rmsnorm: x must be float32 [T, H], got {x.dtype} {tuple(x.shape)}")
    hidden = x.shape[1]
    if tuple(weight.shape) != (hidden,):
        raise KernelError(f"rmsnorm: weight must be [{hidden}], got {tuple(weight.shape)}")
    if rows is None:
        n = x.shape[0]
    else:
        n = rows.numel() if n_rows is None else n_rows
        _i32("rmsnorm", "rows", rows, n)
    if groups <= 0 or hidden % groups:
        raise KernelError(f"rmsnorm: {hidden} channels do not fall into {groups} equal groups")
    out = torch.empty((n, hidden), dtype=out_dtype, device=x.device)
    cost = lambda: (3.0 * n * hidden, n * hidden * (4 + out.element_size()) + hidden * weight.element_size())      # noqa: E731
    if groups == 1:
        library.call("bc4g_rmsnorm", _ptr(x), _ptr(rows), _ptr(weight), _code(weight, "rmsnorm"), _ptr(out),
                     _code(out, "rmsnorm"), n, hidden, float(eps), _stream(), cost=cost)
    else:
        library.call("bc4g_rmsnorm_groups", _ptr(x), _ptr(rows), _ptr(weight), _code(weight, "rmsnorm"), _ptr(out),
                     _code(out, "rmsnorm"), n, hidden, int(groups), float(eps), _stream(), cost=cost)
    return out


def gemm_generic(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = None,
                 accumulate_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed, in plain float arithmetic.  With
    ``accumulate_into`` (float32 [M, N]) the product is added to it in place."""
    w = _rows(w)
    _dev("gemm", a, w, accumulate_into)
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise KernelError(f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not match")
    m, k = a.shape
    n = w.shape[0]
    if accumulate_into is not None:
        out = accumulate_into
        if out.dtype != torch.float32 or tuple(out.shape) != (m, n):
            raise KernelError(f"gemm: accumulate_into must be float32 [{m}, {n}], got {out.dtype} {tuple(out.shape)}")
    else:
        out = torch.empty((m, n), dtype=out_dtype or a.dtype, device=a.device)
    library.call("bc4g_gemm_generic", _ptr(a), _code(a, "gemm"), _ptr(w), _code(w, "gemm"), _ptr(out),
                 _code(out, "gemm"), 1 if accumulate_into is not None else 0, m, n, k, _stream(),
                 cost=_gemm_cost(m, n, k, a.element_size(), w.element_size(),
                                 8 if accumulate_into is not None else out.element_size()))
    return out


def swiglu(gu: torch.Tensor, interleaved: bool = False) -> torch.Tensor:
    """gu [T, 2I] -> silu(gate) * up, [T, I].  gu holds all gates then all ups, or (interleaved)
    blocks of 16: eight gates and the eight ups of the same outputs."""
    _dev("swiglu", gu)
    if gu.dim() != 2 or gu.shape[1] % 2:
        raise KernelError(f"swiglu: input must be [T, 2I], got {tuple(gu.shape)}")
    t, inter = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((t, inter), dtype=gu.dtype, device=gu.device)
    if interleaved and inter % 8:
        raise KernelError(f"swiglu: the interleaved layout needs I={inter} to be a multiple of 8")
    library.call("bc4g_swiglu", _ptr(gu), _ptr(out), _code(gu, "swiglu"), t, inter, 1 if interleaved else 0, _stream(),
                 cost=lambda: (4.0 * t * inter, 3 * t * inter * gu.element_size()))
    return out


def cache_fragment_order(dtype: torch.dtype, head_dim: int, page_tokens: int) -> bool:
    """Whether a cache of these sizes is kept in fragment order -- inside every page and head the
    elements lie as the matrix-core attention kernel's lanes read them -- rather than plain (keys
    [token][dim], values [dim][token]).  The kernels that write and read the cache apply the same rule."""
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and page_tokens % 16 == 0


def cache_from_plain(k: torch.Tensor, v: torch.Tensor):
    """Caches in the layout the kernels expect for their sizes, from plain ones (keys [pages, heads,
    page_tokens, d], values [pages, heads, d, page_tokens]); the shapes stay."""
    n, h, p, d = k.shape
    if not cache_fragment_order(k.dtype, d, p):
        return k, v
    kf = k.view(n, h, p // 16, 16, d // 8, 8).permute(0, 1, 2, 4, 3, 5).contiguous().view(n, h, p, d)
    vf = v.view(n, h, d // 16, 16, p // 16, 4, 4).permute(0, 1, 4, 2, 5, 3, 6).contiguous().view(n, h, d, p)
    return kf, vf


def cache_to_plain(k: torch.Tensor, v: torch.Tensor):
    """The inverse of cache_from_plain: what the kernels wrote, as keys [.., token, dim] and values [.., dim, token]."""
    n, h, p, d = k.shape
    if not cache_fragment_order(k.dtype, d, p):
        return k, v
    kp = k.view(n, h, p // 16, d // 8, 16, 8).permute(0, 1, 2, 4, 3, 5).reshape(n, h, p, d)
    vp = v.view(n, h, p // 16, d // 16, 4, 16, 4).permute(0, 1, 3, 5, 2, 4, 6).reshape(n, h, d, p)
    return kp, vp


def _check_cache(what: str, k: torch.Tensor, v: torch.Tensor, n_kv_heads: int, head_dim: int, dtype: torch.dtype):
    """k: [pages, kv_heads, page_tokens, head_dim]; v transposed: [pages, kv_heads, head_dim, page_tokens]
    (the order inside a page and head: see cache_fragment_order)."""
    ok = (k.dim() == 4 and v.dim() == 4 and k.shape[1] == n_kv_heads and k.shape[3] == head_dim
          and k.dtype == dtype and v.dtype == dtype
          and tuple(v.shape) == (k.shape[0], n_kv_heads, head_dim, k.shape[2]))
    if not ok:
        raise KernelError(f"{what}: caches must be {dtype}, keys [pages, {n_kv_heads}, page_tokens, {head_dim}] and "
                          f"values [pages, {n_kv_heads}, {head_dim}, page_tokens]; got {k.dtype} {tuple(k.shape)} "
                          f"and {v.dtype} {tuple(v.shape)}")


def rope_kv_write(qkv: torch.Tensor, positions: Optional[torch.Tensor], slot_map: Optional[torch.Tensor],
                  k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], n_heads: int,
                  n_kv_heads: int, head_dim: int, rotary_dim: int, theta: float, write_kv: bool = True,
                  block_pairs: bool = False) -> None:
    """Rotate q (in place) and k, write k and v into their pages.  block_pairs: every head's
    dimensions come reordered in blocks of 16 (see bc4g_rope_kv_write)."""
    _dev("rope_kv_write", qkv, positions, slot_map, k_cache, v_cache)
    t = qkv.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width:
        raise KernelError(f"rope_kv_write: qkv must be [T, {width}], got {tuple(qkv.shape)}")
    if positions is not None:
        _i32("rope_kv_write", "positions", positions, t)
    page_tokens = num_pages = 0
    if write_kv:
        _check_cache("rope_kv_write", k_cache, v_cache, n_kv_heads, head_dim, qkv.dtype)
        _i32("rope_kv_write", "slot_map", slot_map, t)
        num_pages, page_tokens = k_cache.shape[0], k_cache.shape[2]
    library.call("bc4g_rope_kv_write", _ptr(qkv), _code(qkv, "rope_kv_write"), _ptr(positions), _ptr(slot_map),
                 _ptr(k_cache), _ptr(v_cache), t, n_heads, n_kv_heads, head_dim, rotary_dim, float(theta),
                 page_tokens, num_pages, 1 if write_kv else 0, 1 if block_pairs else 0, _stream(),
                 cost=lambda: (3.0 * t * (n_heads + n_kv_heads) * head_dim, 2 * t * width * qkv.element_size()))


def rope_table(positions: torch.Tensor, rotary_dim: int, theta: float) -> torch.Tensor:
    """(cos, sin) of every row's angles, float32 [T, rotary_dim / 2, 2]: computed once a step, read
    by every layer's rope_kv_write_blocks."""
    _dev("rope_table", positions)
    t = positions.shape[0]
    _i32("rope_table", "positions", positions, t)
    table = torch.empty((t, rotary_dim // 2, 2), dtype=torch.float32, device=positions.device)
    library.call("bc4g_rope_table", _ptr(positions), _ptr(table), t, int(rotary_dim), float(theta), _stream(),
                 cost=lambda: (0.0, t * rotary_dim * 4))
    return table


def rope_kv_write_blocks(qkv: torch.Tensor, table: Optional[torch.Tensor], slot_map: Optional[torch.Tensor],
                         k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], n_heads: int,
                         n_kv_heads: int, head_dim: int, write_kv: bool = True) -> None:
    """rope_kv_write for heads in block-pair order, rotating the whole head by a table of angles
    (None: no rotation), 16 elements a thread."""
    _dev("rope_kv_write_blocks", qkv, table, slot_map, k_cache, v_cache)
    t = qkv.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width:
        raise KernelError(f"rope_kv_write_blocks: qkv must be [T, {width}], got {tuple(qkv.shape)}")
    if table is not None and (table.dtype != torch.float32 or tuple(table.shape) != (t, head_dim // 2, 2)
                              or not table.is_contiguous()):
        raise KernelError(f"rope_kv_write_blocks: the table must be float32 [{t}, {head_dim // 2}, 2], "
                          f"got {table.dtype} {tuple(table.shape)}")
    page_tokens = 0
    if write_kv:
        _check_cache("rope_kv_write_blocks", k_cache, v_cache, n_kv_heads, head_dim, qkv.dtype)
        _i32("rope_kv_write_blocks", "slot_map", slot_map, t)
        page_tokens = k_cache.shape[2]
    library.call("bc4g_rope_kv_write_blocks", _ptr(qkv), _code(qkv, "rope_kv_write_blocks"), _ptr(table), _ptr(slot_map),
                 _ptr(k_cache), _ptr(v_cache), t, n_heads, n_kv_heads, head_dim, 0 if table is None else 1,
                 page_tokens, 1 if write_kv else 0, _stream(),
                 cost=lambda: (3.0 * t * (n_heads + n_kv_heads) * head_dim, 2 * t * qkv.shape[1] * qkv.element_size()))


def _check_queries(what: str, q: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
    """Queries come as the rows of the fused q|k|v product or as a buffer of queries alone."""
    widths = ((n_heads + 2 * n_kv_heads) * head_dim, n_heads * head_dim)
    if q.dim() != 2 or q.shape[1] not in widths:
        raise KernelError(f"{what}: queries must be [T, {widths[0]}] or [T, {widths[1]}], got {tuple(q.shape)}")


def attention_generic(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_table: torch.Tensor, row_seq: torch.Tensor, positions: torch.Tensor,
                      n_heads: int, n_kv_heads: int, head_dim: int, window: int = 0,
                      scale: Optional[float] = None, work=None) -> torch.Tensor:
    """Causal attention of every row over its request's cache; returns [T, n_heads*head_dim].
    (``work``: what the profiler is told about the call, see attention_work.)"""
    _dev("attention", qkv, k_cache, v_cache, block_table, row_seq, positions)
    t = qkv.shape[0]
    _check_queries("attention", qkv, n_heads, n_kv_heads, head_dim)
    _check_cache("attention", k_cache, v_cache, n_kv_heads, head_dim, qkv.dtype)
    if block_table.dim() != 2 or block_table.dtype != torch.int32:
        raise KernelError("attention: block_table must be int32 [requests, pages]")
    _i32("attention", "row_seq", row_seq, t)
    _i32("attention", "positions", positions, t)
    out = torch.empty((t, n_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    library.call("bc4g_attention_generic", _ptr(qkv), qkv.shape[1], _ptr(out), _code(qkv, "attention"), _ptr(k_cache),
                 _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(row_seq), _ptr(positions), t,
                 n_heads, n_kv_heads, head_dim, k_cache.shape[2], k_cache.shape[0], int(window),
                 float(scale if scale is not None else 1.0 / math.sqrt(head_dim)), _stream(), cost=work)
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Lowest index of each row's maximum, int32 [rows]."""
    _dev("argmax", logits)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelError("argmax: logits must be float32 [rows, vocab]")
    rows = logits.shape[0]
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    part_v = torch.empty((rows, 64), dtype=torch.float32, device=logits.device)
    part_i = torch.empty((rows, 64), dtype=torch.int32, device=logits.device)
    library.call("bc4g_argmax", _ptr(logits), _ptr(out), _ptr(part_v), _ptr(part_i), rows, logits.shape[1], _stream(),
                 cost=lambda: (0.0, rows * logits.shape[1] * 4))
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """One draw per row from softmax(logits / temperature) by inverse CDF with the given
    uniform u in [0, 1); rows with temperature <= 0 get the argmax."""
    _dev("sample", logits, temperature, u)          # (contiguous rows: a strided view would be read as if it were dense)
    rows = logits.shape[0]
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelError("sample: logits must be float32 [rows, vocab]")
    if temperature.dtype != torch.float32 or temperature.numel() != rows:
        raise KernelError("sample: temperature must be float32 [rows]")
    if u.dtype != torch.float64 or u.numel() != rows:
        raise KernelError("sample: u must be float64 [rows]")
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    library.call("bc4g_sample", _ptr(logits), _ptr(temperature), _ptr(u), _ptr(out), rows, logits.shape[1], _stream(),
                 cost=lambda: (3.0 * rows * logits.shape[1], rows * logits.shape[1] * 4))
    return out


def sample_filtered(logits: torch.Tensor, out: torch.Tensor, rows: torch.Tensor, temperature: torch.Tensor,
                    u: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor) -> torch.Tensor:
    """Top-k / top-p draws for some rows of the logits: for each i, the token of logits row rows[i] by the
    reference's law for filtered sampling (weights exp((l - max) / T), the tokens by falling weight with the
    lower id first among equals, the top_k[i] likeliest, of those the fewest that reach top_p[i] of their
    total, the first at which u[i] of the kept mass is passed) goes into out[rows[i]].  top_k 0 or beyond the
    vocabulary and top_p 1 are no limits -- but a row with neither limit is not for this kernel: the law
    without filters walks the tokens in the order of their ids (sample)."""
    _dev("sample_filtered", logits, out, rows, temperature, u, top_k, top_p)
    n = rows.numel()
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelError("sample_filtered: logits must be float32 [rows, vocab]")
    if out.dtype != torch.int32 or out.numel() != logits.shape[0]:
        raise KernelError("sample_filtered: out must be int32, one for every logits row")
    for name, t, dtype in (("rows", rows, torch.int32), ("temperature", temperature, torch.float32), ("u", u, torch.float64),
                           ("top_k", top_k, torch.int32), ("top_p", top_p, torch.float64)):
        if t.dtype != dtype or t.numel() != n:
            raise KernelError(f"sample_filtered: {name} must be {dtype} [{n}]")
    vocab = logits.shape[1]
    library.call("bc4g_sample_filtered", _ptr(logits), _ptr(rows), _ptr(temperature), _ptr(u), _ptr(top_k), _ptr(top_p),
                 _ptr(out), n, vocab, _stream(), cost=lambda: (40.0 * n * vocab, n * vocab * 4))
    return out


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """A [n, k] weight in the fragment order the weight-streaming kernel reads:
    [ceil(n/16)][ceil(k/32)][64 lanes][8], lane l of a k-step holding row l % 16 of the block and
    k 8 * (l / 16) .. + 7 of the step; rows past n and k past the matrix are zeros."""
    n, k = w.shape
    nb, ks = -(-n // 16), -(-k // 32)
    padded = w
    if nb * 16 != n or ks * 32 != k:
        padded = torch.zeros((nb * 16, ks * 32), dtype=w.dtype, device=w.device)
        padded[:n, :k] = w
    return padded.view(nb, 16, ks, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(-1)


def unpack_weight(packed: torch.Tensor, n: int, k: int) -> torch.Tensor:
    """The [n, k] weight by rows from its packed form (pack_weight's inverse)."""
    nb, ks = -(-n // 16), -(-k // 32)
    return packed.view(nb, ks, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nb * 16, ks * 32)[:n, :k].contiguous()


class StreamedWeight:
    """A linear map's weight [n, k] as the kernels read it.  A bfloat16 weight on the device (k a multiple of 8) is
    kept packed in the weight-streaming kernel's order; where k is whole steps of 64 the tiled kernel reads that
    same copy, so the weight is held ONCE.  The rows are kept beside it only where a kernel needs them (k no
    multiple of 64: the tiled kernel's fallback) or where they cost nothing (``keep_rows``: a tensor that someone
    else holds anyway, the embedding table of a tied head); otherwise ``rows`` makes them from the packed copy when
    first asked (the plain float kernel for operands the matrix-core kernels refuse) and keeps them from then on.
    A weight the matrix-core kernels cannot take at all (float32, a CPU tensor) is its rows."""

    def __init__(self, rows: torch.Tensor, keep_rows: Optional[bool] = None):
        self.shape, self.dtype, self.device = rows.shape, rows.dtype, rows.device
        ok = rows.is_cuda and rows.dtype == torch.bfloat16 and rows.dim() == 2 and rows.shape[1] % 8 == 0
        self.packed = pack_weight(rows) if ok else None
        if keep_rows is None:
            keep_rows = not (ok and rows.shape[1] % 64 == 0)
        self._rows = rows if keep_rows or not ok else None
        # which kernel serves this weight at which number of rows: its own table, made from its shape
        self.plan = plan_for(int(rows.shape[0]), int(rows.shape[1])) if rows.dim() == 2 else None

    @property
    def rows(self) -> torch.Tensor:
        if self._rows is None:
            self._rows = unpack_weight(self.packed, self.shape[0], self.shape[1])
        return self._rows

    @property
    def holds_rows(self) -> bool:
        return self._rows is not None

    # what the wrappers ask of an operand before they launch (answered without making the rows)
    @property
    def is_cuda(self) -> bool:
        return self.device.type == "cuda"

    def dim(self) -> int:
        return len(self.shape)

    def is_contiguous(self) -> bool:
        return True

    def stride(self):
        return (self.shape[1], 1)

    def data_ptr(self) -> int:
        return (self.packed if self._rows is None else self._rows).data_ptr()

    def element_size(self) -> int:
        return 2 if self.dtype == torch.bfloat16 else 4


def _weight(w):
    """(the weight as an operand to check -- shape, dtype, device --, its packed copy or None) of a weight given as
    a tensor or a StreamedWeight."""
    if isinstance(w, StreamedWeight):
        return w, w.packed
    return w, None


def _rows(w) -> torch.Tensor:
    return w.rows if isinstance(w, StreamedWeight) else w


def _tiled_weight(w, packed, a: Optional[torch.Tensor] = None):
    """(address, 1 if packed else 0) of a weight for the tiled kernel: the packed copy for the kernel with operands
    straight into LDS (k in whole steps of 64, x on a 16-byte boundary; a bare tensor is packed for the call: tests
    only), else the rows for the kernel that stages its tiles through registers."""
    if w.shape[1] % 64 == 0 and w.dtype == torch.bfloat16 and (a is None or a.data_ptr() % 16 == 0):
        if packed is None:
            packed = pack_weight(_rows(w))        # (given back to the allocator in stream order, after the launch)
        return packed.data_ptr(), 1
    return _rows(w).data_ptr(), 0


SKINNY_MAX_ROWS = 64                # rows the weight-streaming kernel takes in one launch
NORMED_STAGE_BYTES = 96 * 1024      # LDS the fused norm may fill with its rows of bf16(x * g)


@dataclasses.dataclass(frozen=True)
class LinearPlan:
    """Which kernel serves x W^T at which number of rows, for ONE weight [n, k].  A weight gets its plan when it is
    bound (StreamedWeight.plan; plan_for(n, k) for a bare tensor), from its own shape and the number of compute
    units; the ops below and the parts ask the plan and carry no row thresholds of their own, so a model of other
    widths gets thresholds of its own and a measured plan can take a computed one's place (set_plan).

    The rules a plan is computed by (each measured as a whole decode step at three shapes of this architecture,
    not as a loop over one product, whose weights would come from the 256 MB cache):
    - stream_rows.  Up to 64 rows the weight is streamed once by gemm_skinny: with one or two rows of tiles a tiled
      product is as long as its chain of k-steps, which the streaming kernel's eight waves cut into eight.  But every
      one of the streaming kernel's workgroups reads all the rows of x, and an output with 64 x 64 tiles enough for
      every other CU and more (n >= 32 tiles' worth of columns per CU pair: 8,192 on 256 CUs) fills the chip tiled:
      such a weight goes to the tiled kernel from 24 rows on.
    - fused_norm_rows.  Up to 8 rows the RMSNorm before the product is fused into the streaming kernel (it takes 16,
      but every workgroup stages all the rows, and from 9 on a norm kernel of its own is faster), as long as the
      staged rows fit LDS.
    - parts_rows.  For 10 to 256 rows a product that adds into the residual stream cuts k over workgroups (64 x 64
      tiles, the parts added up by a second kernel that norms the stream for the next product): a tile's workgroup
      would walk all of k alone and the streaming kernel's workgroups all read all of x.  Up to 64 rows only for
      weights of 2^24 elements and more (for smaller ones the streaming kernel wins there).
    - qkv_stream_rows.  The product with rotation and cache write in its epilogue stays with the streaming kernel up
      to 47 rows where the output is wide (every query head with keys of its own), to 64 otherwise.
    """
    n: int
    k: int
    stream_rows: int
    fused_norm_rows: int
    parts_rows: Tuple[int, int]
    qkv_stream_rows: int

    def streams(self, m: int) -> bool:
        """Whether the weight-streaming kernel takes a product of m rows."""
        return m <= self.stream_rows

    def fuses_norm(self, m: int) -> bool:
        return 0 < m <= self.fused_norm_rows

    def parts(self, m: int) -> int:
        """Into how many parts an adding product of m rows cuts k over workgroups (1: it does not)."""
        lo, hi = self.parts_rows
        if not (lo <= m <= hi):
            return 1
        tiles = -(-m // 64) * -(-self.n // 64)
        best = 1
        for parts in (2, 4, 8):
            if self.k % (64 * parts) == 0 and self.k // (64 * parts) >= PARTS_MIN_STEPS and tiles * parts <= PARTS_WORKGROUPS:
                best = parts
        return best

    def tiled_finishes_norm(self, m: int) -> bool:
        """Whether a SwiGLU product of m rows goes to the tiled kernel and can finish a prepared norm there."""
        return TILED_PRENORMED and not self.streams(m) and self.k % 64 == 0 and self.n % 16 == 0

    def wants_prepared(self, m: int, swiglu: bool = False) -> bool:
        """Whether a part whose first product is this weight's is better served, at m rows, by a norm that the
        product before prepared than by fusing the norm or running it.  A q|k|v product reads prepared bfloat16 rows
        faster than it stages float ones for a fused norm, and beyond the fused norm's rows a prepared norm saves
        the norm's own kernel: always.  A SwiGLU product has many more workgroups, each of which adds up the
        prepared parts: with few rows the fused norm costs little; from 5 rows to the fused norm's last, prepared
        rows beat float rows staged in every workgroup; beyond, up to 63 rows, a norm kernel of its own is the
        faster way for the streaming kernel -- while the tiled kernel, where the product goes there, adds the parts
        up once a tile and takes them; at 64 rows and more the streaming kernel takes them too."""
        if not swiglu:
            return True
        if m <= SKINNY_MAX_ROWS and self.tiled_finishes_norm(m):
            return True
        return 5 <= m <= self.fused_norm_rows or (m >= 64 and self.streams(m))


PARTS_MIN_STEPS = 4                 # k-steps of 64 a part keeps at least
PARTS_WORKGROUPS = 256              # as many parts (2, 4 or 8) as bring the 64 x 64 tiles to this many
TILED_PRENORMED = True
_PLANS: Dict[Tuple[int, int], LinearPlan] = {}


def compute_plan(n: int, k: int, cus: int = 256) -> LinearPlan:
    """The plan of a weight [n, k] by the rules LinearPlan states."""
    wide = k % 64 == 0 and n >= 32 * cus             # (the tiled kernel's small tiles need k in steps of 64)
    fused = 0
    for rows in range(1, 9):
        if (-(-rows // 4) * 4) * (k + 8) * 2 <= NORMED_STAGE_BYTES:     # rows rounded up to 4, each k + 8 bfloat16
            fused = rows
    if k % 64 or n % 8 or n > 8192:
        parts_rows = (1, 0)
    else:
        parts_rows = (10 if n * k >= (1 << 24) else SKINNY_MAX_ROWS + 1, 256)
    return LinearPlan(n=n, k=k, stream_rows=23 if wide else SKINNY_MAX_ROWS, fused_norm_rows=fused,
                      parts_rows=parts_rows, qkv_stream_rows=47 if wide else SKINNY_MAX_ROWS)


def plan_for(n: int, k: int) -> LinearPlan:
    """The plan every weight of this shape shares: computed at first sight, or what set_plan put there."""
    plan = _PLANS.get((n, k))
    if plan is None:
        plan = _PLANS[(n, k)] = compute_plan(n, k)
    return plan


def set_plan(plan: LinearPlan) -> None:
    """Put a plan (a measured one, say) in the place of the computed one for weights of its shape.  Weights bound
    before keep the plan they were bound with."""
    _PLANS[(plan.n, plan.k)] = plan


def _plan(w) -> LinearPlan:
    plan = getattr(w, "plan", None)
    return plan if plan is not None else plan_for(int(w.shape[0]), int(w.shape[1]))


def streams_weights(m: int, n: int, k: int) -> bool:
    """Whether the weight-streaming kernel takes a product of m rows, n outputs and this k."""
    return plan_for(n, k).streams(m)


EPI_STORE_BF16, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU = 0, 1, 2, 3


def _fast_operands(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
            and a.shape[1] == w.shape[1] and a.shape[1] % 8 == 0 and a.shape[0] > 0)


def gemm_fast(a: torch.Tensor, w, out_dtype=None,
              accumulate_into: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """The matrix-core product where a kernel takes these operands (bfloat16, k a multiple of
    8), else None (the caller then uses the plain float kernel).  Up to 64 rows the weights
    are streamed once (a decode step); a wide output goes to the tiled kernel from 24 rows on,
    everything from 65."""
    w, packed = _weight(w)
    if not _fast_operands(a, w):
        return None
    _dev("gemm", a, w, accumulate_into)
    m, k = a.shape
    n = w.shape[0]
    if accumulate_into is not None:
        out, epi = accumulate_into, EPI_ACCUM_F32
        if out.dtype != torch.float32 or tuple(out.shape) != (m, n):
            raise KernelError(f"gemm: accumulate_into must be float32 [{m}, {n}], got {out.dtype} {tuple(out.shape)}")
    else:
        out_dtype = out_dtype or a.dtype
        if out_dtype not in (torch.bfloat16, torch.float32):
            return None
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
        epi = EPI_STORE_BF16 if out_dtype == torch.bfloat16 else EPI_STORE_F32
    out_bytes = 8 if accumulate_into is not None else out.element_size()
    if streams_weights(m, n, k):
        packed = packed if packed is not None else pack_weight(_rows(w))      # (packing per call: tests only)
        for r0 in range(0, m, SKINNY_MAX_ROWS):                        # the weights once for every 64 rows
            rows = min(SKINNY_MAX_ROWS, m - r0)
            library.call("bc4g_gemm_skinny", _ptr(a[r0:]), _ptr(packed), _ptr(out[r0:]), epi, rows, n, k, _stream(),
                         cost=_skinny_cost(rows, n, k, 2, out_bytes))
    else:
        library.call("bc4g_gemm_mfma", _ptr(a), *_tiled_weight(w, packed, a), _ptr(out), epi, m, n, k, _stream(),
                     cost=_tiled_cost(m, n, k, out_bytes))
    return out


def _normed_rows_fit(n_rows: int, k: int, n: int = 0) -> bool:
    """Whether an RMSNorm before a product of these rows is fused into the streaming kernel: few rows (the plan's
    fused_norm_rows: at most 8), which fit LDS rounded up to 4 with k + 8 bfloat16 each (8 rows do up to k = 6,136)."""
    return plan_for(n or k, k).fuses_norm(n_rows)


def gemm_normed_supported(x: torch.Tensor, n_rows: int, g: torch.Tensor, w) -> bool:
    """Whether RMSNorm can be fused into the product: few rows, bfloat16 weights, k a multiple of 8."""
    w, _ = _weight(w)
    return (x.is_cuda and x.dtype == torch.float32 and w.dtype == torch.bfloat16 and x.shape[1] == w.shape[1]
            and _normed_rows_fit(n_rows, x.shape[1], w.shape[0]) and x.shape[1] % 8 == 0 and g.dtype in _CODE)


def gemm_normed(x: torch.Tensor, rows: Optional[torch.Tensor], n_rows: int, g: torch.Tensor, eps: float,
                w, epilogue: int) -> torch.Tensor:
    """rmsnorm(x[rows]) W^T with the norm fused into the product (see gemm_skinny.hip): epilogue
    EPI_STORE_BF16, EPI_STORE_F32 or EPI_SWIGLU (w = gate rows then up rows)."""
    w, packed = _weight(w)
    packed = packed if packed is not None else pack_weight(_rows(w))
    _dev("gemm_normed", x, rows, g, w)
    k, n = x.shape[1], w.shape[0]
    if tuple(g.shape) != (k,):
        raise KernelError(f"gemm_normed: norm scale must be [{k}], got {tuple(g.shape)}")
    if rows is not None:
        _i32("gemm_normed", "rows", rows, n_rows)
    elif n_rows != x.shape[0]:
        raise KernelError("gemm_normed: without row indices every row of x is used")
    if epilogue == EPI_SWIGLU:
        out = torch.empty((n_rows, n // 2), dtype=torch.bfloat16, device=x.device)
    elif epilogue == EPI_STORE_BF16:
        out = torch.empty((n_rows, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == EPI_STORE_F32:
        out = torch.empty((n_rows, n), dtype=torch.float32, device=x.device)
    else:
        raise KernelError(f"gemm_normed: epilogue {epilogue} is not supported")
    library.call("bc4g_gemm_skinny_normed", _ptr(x), _ptr(rows), _ptr(g), _code(g, "gemm_normed"), float(eps),
                 _ptr(packed), _ptr(out), epilogue, n_rows, n, k, _stream(),
                 cost=_skinny_cost(n_rows, n, k, 4, out.element_size() * out.shape[1] / n))
    return out


def gemm_swiglu(a: torch.Tensor, w_gate_up, interleaved: bool = False) -> torch.Tensor:
    """silu(a Wg^T) * (a Wu^T), [M, I], for w_gate_up [2I, K].  interleaved: every 16 rows of the
    weight are eight gate rows and the eight up rows of the same outputs -- then the activation
    is applied to the float sums inside the product's kernel.  Otherwise the product is stored
    and the activation kernel follows."""
    rows, packed = _weight(w_gate_up)
    if interleaved and _fast_operands(a, rows) and rows.shape[0] % 16 == 0:
        _dev("gemm_swiglu", a, rows)
        m, k = a.shape
        n = rows.shape[0]
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=a.device)
        if streams_weights(m, n, k):
            packed = packed if packed is not None else pack_weight(_rows(rows))
            for r0 in range(0, m, SKINNY_MAX_ROWS):
                part = min(SKINNY_MAX_ROWS, m - r0)
                library.call("bc4g_gemm_skinny", _ptr(a[r0:]), _ptr(packed), _ptr(out[r0:]), EPI_SWIGLU, part, n, k,
                             _stream(), cost=_skinny_cost(part, n, k, 2, 1))
        else:
            library.call("bc4g_gemm_mfma", _ptr(a), *_tiled_weight(rows, packed, a), _ptr(out), EPI_SWIGLU, m, n, k, _stream(),
                         cost=_tiled_cost(m, n, k, 1))
        return out
    gu = gemm_fast(a, w_gate_up, a.dtype)
    if gu is None:
        gu = gemm_generic(a, w_gate_up, a.dtype)
    return swiglu(gu, interleaved)


class Fresh:
    """Stands for a float32 [rows, n] sum that does not exist yet, where a part expects the stream it adds to: the first
    product "added" to it is simply stored, and the result is found in ``tensor`` (parts.linear.linear).  A block that
    norms a sublayer's output before adding it to the stream hands this to parts that add through one last product, and
    saves clearing a buffer and reading it back."""

    def __init__(self):
        self.tensor: Optional[torch.Tensor] = None


class Prenormed:
    """What a product that added into the residual stream left for the RMSNorm after it
    (gemm_accumulate_emit): ``xb`` = bfloat16(residual * g) [m, width] and ``parts`` [blocks, m], block
    b's share (16 columns) of every row's sum of squares.  A product that takes it
    (gemm_prenormed, gemm_qkv_rope) applies the row's rsqrt(sum of parts / width + eps) to its sums."""

    def __init__(self, xb: torch.Tensor, parts: torch.Tensor, eps: float):
        self.xb, self.parts, self.eps = xb, parts, float(eps)


class Finished:
    """The RMSNorm after a product that added into the residual stream, already computed by that product's
    second kernel (gemm_parts_accumulate_norm): ``tensor`` [m, width] in bfloat16."""

    def __init__(self, tensor: torch.Tensor):
        self.tensor = tensor


def parts_of_k(m: int, n: int, k: int) -> int:
    """Into how many parts gemm_parts_accumulate_norm cuts k (1: it does not take the product)."""
    return plan_for(n, k).parts(m)


def gemm_parts_supported(a: torch.Tensor, w, residual: torch.Tensor, g: torch.Tensor) -> bool:
    """Whether gemm_parts_accumulate_norm takes these operands: bfloat16, 10 to 256 rows, a k that several
    workgroups can share, a plain RMSNorm after it."""
    w, _ = _weight(w)
    return (_fast_operands(a, w) and residual.dtype == torch.float32 and residual.is_contiguous()
            and tuple(residual.shape) == (a.shape[0], w.shape[0]) and g.dtype in _CODE and tuple(g.shape) == (w.shape[0],)
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and residual.data_ptr() % 16 == 0 and a.is_contiguous()
            and w.is_contiguous() and parts_of_k(a.shape[0], w.shape[0], w.shape[1]) > 1)


def gemm_parts_accumulate_norm(a: torch.Tensor, w, residual: torch.Tensor, g: torch.Tensor, eps: float,
                               checked: bool = False) -> Finished:
    """residual += a w^T and the RMSNorm (scale g, eps) of the result, in two kernels: the tiled product with k cut
    into parts over workgroups, each part's sums stored apart; then one that adds the parts to the residual in
    order and norms it.  For a few dozen rows and a square or long weight, where a 64 x 64 tile's workgroup
    would walk all of k alone and the weight-streaming kernel's workgroups all read all of x."""
    w, packed = _weight(w)
    _dev("gemm_parts_accumulate_norm", a, w, residual, g)
    m, k = a.shape
    n = w.shape[0]
    n_parts = parts_of_k(m, n, k)
    if n_parts < 2 or not (checked or gemm_parts_supported(a, w, residual, g)):     # (checked: the caller has just asked)
        raise KernelError(f"gemm_parts_accumulate_norm: not for [{m}, {k}] x [{n}, {k}]^T")
    parts = torch.empty((n_parts, m, n), dtype=torch.float32, device=a.device)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    library.call("bc4g_gemm_mfma_parts", _ptr(a), *_tiled_weight(w, packed), _ptr(parts), m, n, k, n_parts, _stream(),
                 cost=_gemm_cost(m, n, k, 2, 2, 4 * n_parts, x_readers=-(-n // 64), w_readers=-(-m // 64)))
    library.call("bc4g_rmsnorm_sum", _ptr(residual), _ptr(parts), n_parts, _ptr(g), _code(g, "rmsnorm_sum"), _ptr(out),
                 _code(out, "rmsnorm_sum"), m, n, float(eps), _stream(),
                 cost=lambda: (3.0 * m * n + n_parts * m * n, m * n * (4 * n_parts + 8 + 2) + n * g.element_size()))
    return Finished(out)


def gemm_emit_supported(a: torch.Tensor, w, residual: torch.Tensor, g: torch.Tensor) -> bool:
    """Whether the adding product of these operands can prepare the next RMSNorm: the
    weight-streaming kernel serves it (bfloat16, few rows: streams_weights)."""
    w, _ = _weight(w)
    return (_fast_operands(a, w) and 0 < a.shape[0] and streams_weights(a.shape[0], w.shape[0], w.shape[1]) and residual.dtype == torch.float32
            and g.dtype in _CODE and tuple(g.shape) == (w.shape[0],))


def gemm_accumulate_emit(a: torch.Tensor, w, residual: torch.Tensor, g: torch.Tensor, eps: float) -> Prenormed:
    """residual += a w^T, and the next RMSNorm (scale g, eps) prepared: see Prenormed."""
    w, packed = _weight(w)
    packed = packed if packed is not None else pack_weight(_rows(w))
    _dev("gemm_accumulate_emit", a, w, residual, g)
    m, k = a.shape
    n = w.shape[0]
    if tuple(residual.shape) != (m, n) or residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError(f"gemm_accumulate_emit: the residual must be contiguous float32 [{m}, {n}]")
    if tuple(g.shape) != (n,):
        raise KernelError(f"gemm_accumulate_emit: norm scale must be [{n}], got {tuple(g.shape)}")
    xb = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    parts = torch.empty((-(-n // 16), m), dtype=torch.float32, device=a.device)
    for r0 in range(0, m, SKINNY_MAX_ROWS):
        rows = min(SKINNY_MAX_ROWS, m - r0)
        library.call("bc4g_gemm_skinny_emit", _ptr(a[r0:]), _ptr(packed), _ptr(residual[r0:]), _ptr(g),
                     _code(g, "gemm_accumulate_emit"), _ptr(xb[r0:]), _ptr(parts[:, r0:]), m, rows, n, k, _stream(),
                     cost=_skinny_cost(rows, n, k, 2, 10))
    return Prenormed(xb, parts, eps)


def tiled_takes_prenormed(n_rows: int, n: int, k: int) -> bool:
    """Whether a SwiGLU product of these sizes that goes to the tiled kernel can finish a prepared norm there."""
    return plan_for(n, k).tiled_finishes_norm(n_rows)


def gemm_prenormed_supported(pre: Prenormed, w, epilogue: Optional[int] = None) -> bool:
    w, _ = _weight(w)
    if not _fast_operands(pre.xb, w):
        return False
    m, (n, k) = pre.xb.shape[0], w.shape
    return streams_weights(m, n, k) or (epilogue == EPI_SWIGLU and tiled_takes_prenormed(m, n, k)
                                        and _ptr(pre.xb) % 16 == 0 and _ptr(w) % 16 == 0)


def gemm_prenormed(pre: Prenormed, w, epilogue: int) -> torch.Tensor:
    """rmsnorm(residual) w^T from what gemm_accumulate_emit left: epilogue EPI_STORE_BF16,
    EPI_STORE_F32 or EPI_SWIGLU (w in blocks of eight gate and eight up rows)."""
    w, packed = _weight(w)
    tiled_w = _tiled_weight(w, packed)
    packed = packed if packed is not None else pack_weight(_rows(w))
    _dev("gemm_prenormed", pre.xb, pre.parts, w)
    m, k = pre.xb.shape
    n = w.shape[0]
    if epilogue == EPI_SWIGLU:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=w.device)
    elif epilogue == EPI_STORE_BF16:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=w.device)
    elif epilogue == EPI_STORE_F32:
        out = torch.empty((m, n), dtype=torch.float32, device=w.device)
    else:
        raise KernelError(f"gemm_prenormed: epilogue {epilogue} is not supported")
    if not streams_weights(m, n, k):
        if epilogue != EPI_SWIGLU:
            raise KernelError("gemm_prenormed: the tiled kernel finishes a prepared norm in its SwiGLU epilogue only")
        library.call("bc4g_gemm_mfma_swiglu_scaled", _ptr(pre.xb), _ptr(pre.parts), pre.parts.shape[0], pre.parts.shape[1], pre.eps,
                     *tiled_w, _ptr(out), m, n, k, _stream(), cost=_tiled_cost(m, n, k, 1))
        return out
    for r0 in range(0, m, SKINNY_MAX_ROWS):
        rows = min(SKINNY_MAX_ROWS, m - r0)
        library.call("bc4g_gemm_skinny_prenormed", _ptr(pre.xb[r0:]), _ptr(pre.parts[:, r0:]), pre.parts.shape[0], m,
                     pre.eps, _ptr(packed), _ptr(out[r0:]), epilogue, rows, n, k, _stream(),
                     cost=_skinny_cost(rows, n, k, 2, out.element_size() * out.shape[1] / n))
    return out


def gemm_qkv_rope_supported(x: torch.Tensor, n_rows: int, normed: bool, w, head_dim: int,
                            rotary_dim: int) -> bool:
    """Whether the q|k|v product of these rows can rotate and write the cache in its epilogue."""
    w, _ = _weight(w)
    plan = plan_for(int(w.shape[0]), int(x.shape[1]))
    rows_ok = plan.fuses_norm(n_rows) if normed else n_rows <= SKINNY_MAX_ROWS
    if not normed and n_rows > plan.qkv_stream_rows:
        return False                  # a wide q|k|v output: the tiled kernel's epilogue does the same
    return (x.is_cuda and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and 0 < n_rows and rows_ok
            and head_dim % 16 == 0 and rotary_dim in (0, head_dim)
            and x.dtype == (torch.float32 if normed else torch.bfloat16))


def gemm_qkv_rope(x: torch.Tensor, g: Optional[torch.Tensor], eps: float, w,
                  positions: torch.Tensor, slot_map: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                  v_cache: Optional[torch.Tensor], n_heads: int, n_kv_heads: int, head_dim: int, rotary_dim: int,
                  theta: float, write_kv: bool = True, pre: Optional[Prenormed] = None) -> torch.Tensor:
    """The q|k|v product of a decode step with rotary positions and the cache write in its
    epilogue (w in the reordered head layout).  With g the input is the float residual stream
    and RMSNorm is fused; with ``pre`` (x = pre.xb) the norm was prepared by the product before.
    Returns the rotated queries [M, heads * head_dim]."""
    w, packed = _weight(w)
    packed = packed if packed is not None else pack_weight(_rows(w))
    _dev("gemm_qkv_rope", x, g, w, positions, slot_map, k_cache, v_cache)
    m, k = x.shape
    n = (n_heads + 2 * n_kv_heads) * head_dim
    if tuple(w.shape) != (n, k):
        raise KernelError(f"gemm_qkv_rope: weight must be [{n}, {k}], got {tuple(w.shape)}")
    _i32("gemm_qkv_rope", "positions", positions, m)
    page_tokens = 0
    if write_kv:
        _check_cache("gemm_qkv_rope", k_cache, v_cache, n_kv_heads, head_dim, torch.bfloat16)
        _i32("gemm_qkv_rope", "slot_map", slot_map, m)
        page_tokens = k_cache.shape[2]
    if g is not None and (tuple(g.shape) != (k,) or x.dtype != torch.float32):
        raise KernelError("gemm_qkv_rope: the fused norm needs a float32 input and a scale of its width")
    q = torch.empty((m, n_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    if pre is not None and (g is not None or x is not pre.xb):
        raise KernelError("gemm_qkv_rope: a prepared norm comes with its own rows and without a scale")
    parts = pre.parts if pre is not None else None
    library.call("bc4g_gemm_skinny_qkv", _ptr(x), _ptr(g), _code(g, "gemm_qkv_rope") if g is not None else 0,
                 float(pre.eps if pre is not None else eps), _ptr(parts), parts.shape[0] if pre is not None else 0,
                 parts.shape[1] if pre is not None else 0, _ptr(packed), _ptr(q), _ptr(positions), _ptr(slot_map),
                 _ptr(k_cache), _ptr(v_cache), m, k, n_heads, n_kv_heads, head_dim, int(rotary_dim), float(theta),
                 page_tokens, 1 if write_kv else 0, _stream(), cost=_skinny_cost(m, n, k, x.element_size(), 2))
    return q


TILED_QKV_ROPE = True               # (off: the product, then a kernel that rotates and writes the cache)


def gemm_qkv_rope_tiled_supported(x: torch.Tensor, w, head_dim: int, rotary_dim: int) -> bool:
    """Whether the tiled kernel takes the q|k|v product of these (many) rows with rotation and cache write in its
    epilogue: bfloat16, operands straight into LDS, heads in blocks of 16, the whole head rotated or none of it."""
    w, _ = _weight(w)
    return (TILED_QKV_ROPE and x.is_cuda and _fast_operands(x, w) and not streams_weights(x.shape[0], w.shape[0], w.shape[1])
            and x.shape[1] % 64 == 0 and x.is_contiguous() and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and head_dim % 16 == 0 and rotary_dim in (0, head_dim))


def gemm_qkv_rope_tiled(x: torch.Tensor, w, table: Optional[torch.Tensor], slot_map: Optional[torch.Tensor],
                        k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], n_heads: int, n_kv_heads: int,
                        head_dim: int, write_kv: bool = True) -> torch.Tensor:
    """The q|k|v product of a prompt portion with rotary positions (``table``: rope_table() of the rows' positions;
    None: no rotation) and the cache write in its epilogue (w in the reordered head layout).  Returns the rotated
    queries [M, heads * head_dim]."""
    w, packed = _weight(w)
    _dev("gemm_qkv_rope_tiled", x, w, table, slot_map, k_cache, v_cache)
    m, k = x.shape
    n = (n_heads + 2 * n_kv_heads) * head_dim
    if tuple(w.shape) != (n, k):
        raise KernelError(f"gemm_qkv_rope_tiled: weight must be [{n}, {k}], got {tuple(w.shape)}")
    if table is not None and (table.dtype != torch.float32 or tuple(table.shape) != (m, head_dim // 2, 2)
                              or not table.is_contiguous()):
        raise KernelError(f"gemm_qkv_rope_tiled: the table must be float32 [{m}, {head_dim // 2}, 2], "
                          f"got {table.dtype} {tuple(table.shape)}")
    page_tokens = 0
    if write_kv:
        _check_cache("gemm_qkv_rope_tiled", k_cache, v_cache, n_kv_heads, head_dim, torch.bfloat16)
        _i32("gemm_qkv_rope_tiled", "slot_map", slot_map, m)
        page_tokens = k_cache.shape[2]
    q = torch.empty((m, n_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    library.call("bc4g_gemm_mfma_qkv", _ptr(x), *_tiled_weight(w, packed), _ptr(q), _ptr(table), _ptr(slot_map), _ptr(k_cache), _ptr(v_cache),
                 m, n, k, n_heads, n_kv_heads, head_dim, page_tokens, 1 if write_kv else 0, _stream(),
                 cost=_tiled_cost(m, n, k, 2, qkv=True))
    return q


def attention_mfma_supported(qkv: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    return (qkv.dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256
            and k_cache.shape[2] % 16 == 0)


ATTENTION_STAGED_WAVES = 4      # waves of a workgroup whose tiles share every key tile through LDS


def attention_tile_tokens(n_heads: int, n_kv_heads: int) -> int:
    """Tokens of one request per 16-row tile of the matrix-core attention kernel."""
    return 16 // min(n_heads // n_kv_heads, 16)


def attention_q_tiles(head_dim: int) -> int:
    """16-row tiles a wave of the matrix-core attention kernel takes for prompt portions."""
    return 4 if head_dim <= 64 else (2 if head_dim <= 128 else 1)


ATTENTION_MAX_SPLITS = 64
ATTENTION_PROMPT_GROUPS = 512     # workgroups a prompt step should bring where the caller cuts every walk alike
ATTENTION_SLOTS = 512             # workgroups of the prompt form the GPU holds at a time (two a CU: the kernel's registers)
ATTENTION_MAX_PROMPT_SPLITS = 8
ATTENTION_SHARE_SLACK = 1.5       # a part of a prompt's walk may be this much longer than an even share of all tiles
                                  # (2,048-token prompts in the model: 1.25 to 2 within 1 %, 1 and 3 are 2-5 % longer)
ATTENTION_MIN_WALK = 4            # 32-key tiles a part of a prompt's keys should hold at least
ATTENTION_APART_CONTEXT = 256     # cached tokens from which on a single-tile request beside prompt portions gets a
                                  # launch of the decode form for itself
ATTENTION_SHARED_WALK = 1         # 32-key tiles a wave walks where a workgroup's waves share one tile's keys:
                                  # a CU pulls only so much from memory, so few workgroups with long walks are slow
ATTENTION_WORTH_A_CUT = 2
ATTENTION_ENOUGH_GROUPS = 256     # workgroups of that kind from which on the keys are not cut further


def attention_shared_waves(head_dim: int) -> int:
    """Waves that share one tile's keys in the decode form of the matrix-core attention kernel."""
    return 8 if head_dim <= 128 else 4



def attention_splits(n_tiles: int, n_heads: int, n_kv_heads: int, max_kv_len: int, shared_waves: int = 0) -> int:
    """Into how many parts the keys are cut over workgroups so that the GPU has enough of them.
    n_tiles counts waves' tiles.  Prompt forms (four waves a workgroup): towards
    ATTENTION_PROMPT_GROUPS workgroups, while a part keeps ATTENTION_MIN_WALK tiles of 32 keys (the
    engine's steps bring a work list instead: prompt_work_list).
    With ``shared_waves`` a workgroup is one tile whose waves already cut the keys between them;
    the keys are cut further only while a wave would walk more than ATTENTION_SHARED_WALK tiles."""
    group = n_heads // n_kv_heads
    waves = n_tiles * n_kv_heads * (-(-group // 16))
    key_tiles = max(1, -(-max_kv_len // 32))
    if shared_waves:
        walk = -(-key_tiles // shared_waves)
        parts = max(1, min(-(-walk // ATTENTION_SHARED_WALK), ATTENTION_ENOUGH_GROUPS // max(waves, 1),
                           ATTENTION_MAX_SPLITS))
        # a cut that shortens a wave's walk by less than ATTENTION_WORTH_A_CUT tiles does not pay for the merge kernel
        # (32 requests at 548 tokens of context, two parts: a wave walks 2 tiles instead of 3, a step 1.209 against 1.165 ms)
        return parts if walk - -(-walk // parts) >= ATTENTION_WORTH_A_CUT else 1
    groups = max(1, -(-waves // ATTENTION_STAGED_WAVES))
    return max(1, min(-(-ATTENTION_PROMPT_GROUPS // groups), ATTENTION_MAX_PROMPT_SPLITS,
                      key_tiles // ATTENTION_MIN_WALK))


def attention_mfma(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                   seq_start: torch.Tensor, seq_ctx: torch.Tensor, tile_start: torch.Tensor, n_tiles: int,
                   n_heads: int, n_kv_heads: int, head_dim: int, window: int, scale: float,
                   n_splits: int, q_tiles: int = 1, form: int = 0, work=None,
                   out: Optional[torch.Tensor] = None, row_seq: Optional[torch.Tensor] = None,
                   single_rows: bool = False, items: Optional[torch.Tensor] = None, n_items: int = 0,
                   row_parts: Optional[torch.Tensor] = None) -> torch.Tensor:
    """form 0: four independent waves a workgroup, tile_start counts pieces of q_tiles tiles; 1: one
    tile a workgroup, its waves share the keys (q_tiles 1); 2: four waves a workgroup that walk their
    keys together through LDS, tile_start counts pieces of 4 * q_tiles tiles (ATTENTION_STAGED_WAVES).
    Requests without pieces are left out; with ``out`` (the result of another launch over the other
    requests) and ``row_seq`` (each row's request) their rows of it stay as they are.
    ``single_rows`` (form 1): the caller knows that every request brings exactly one row (a decode
    step), and the kernel then looks nothing up before it asks for the block table and the query.
    ``items`` (form 2; prompt_work_list): a work list of n_items workgroups in the order in which they
    are to start, each a piece, a part and the number of parts of that piece's keys; ``row_parts`` [T]:
    into how many parts each row's keys are cut; n_splits is then the most parts of any piece."""
    _dev("attention_mfma", qkv, k_cache, v_cache, block_table, seq_start, seq_ctx, tile_start)
    t = qkv.shape[0]
    _check_queries("attention_mfma", qkv, n_heads, n_kv_heads, head_dim)
    if qkv.dtype != torch.bfloat16:
        raise KernelError(f"attention_mfma: queries must be bfloat16, got {qkv.dtype}")
    _check_cache("attention_mfma", k_cache, v_cache, n_kv_heads, head_dim, qkv.dtype)
    if block_table.dim() != 2 or block_table.dtype != torch.int32:
        raise KernelError("attention_mfma: block_table must be int32 [requests, pages]")
    n_seqs = block_table.shape[0]
    _i32("attention_mfma", "seq_start", seq_start, n_seqs + 1)
    _i32("attention_mfma", "seq_ctx", seq_ctx, n_seqs)
    _i32("attention_mfma", "tile_start", tile_start, n_seqs + 1)
    if out is None:
        out = torch.empty((t, n_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    elif out.dtype != qkv.dtype or tuple(out.shape) != (t, n_heads * head_dim) or not out.is_contiguous():
        raise KernelError(f"attention_mfma: out must be {qkv.dtype} [{t}, {n_heads * head_dim}]")
    if row_seq is not None:
        _dev("attention_mfma", row_seq)
        _i32("attention_mfma", "row_seq", row_seq, t)
    if items is not None:
        _dev("attention_mfma", items, row_parts)
        _i32("attention_mfma", "items", items, n_items)
        _i32("attention_mfma", "row_parts", row_parts, t)
    part_o = part_ml = None
    if n_splits > 1:
        part_o = torch.empty((n_splits, t, n_heads, head_dim), dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty((n_splits, t, n_heads, 2), dtype=torch.float32, device=qkv.device)
    library.call("bc4g_attention_mfma", _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(k_cache),
                 _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(seq_start), _ptr(seq_ctx),
                 _ptr(tile_start), n_seqs, n_tiles, t, n_heads, n_kv_heads, head_dim, k_cache.shape[2],
                 int(window), float(scale), attention_tile_tokens(n_heads, n_kv_heads), int(q_tiles),
                 int(form), int(n_splits), _ptr(items), int(n_items), _ptr(row_parts), 1 if single_rows else 0,
                 _ptr(row_seq), _stream(), cost=work)
    return out


_DECODE_TILE_STARTS: dict = {}


def prompt_work_list(batch, piece_starts, piece: int, head_blocks: int, window: int):
    """The prompt form's workgroups for a batch, in the order in which they should start, and into how many parts
    each row's keys are cut: (packed items, parts per row, most parts).  ``piece_starts`` [S + 1]: the first piece
    of every request (a piece = the ``piece`` consecutive rows a workgroup takes); ``head_blocks``: workgroups
    that take the same piece for different heads.

    Under the causal mask a piece's walk over the keys is as long as its position: walks of 1 to 64 tiles of
    32 keys in a 2,048-token prompt.  A workgroup takes about as long as its walk (1.6-1.9 us a tile, with a
    second workgroup beside it on the CU or without, plus 6 us before and after), and a CU holds two at a
    time.  So the walks are cut into parts of at most half more than an even share of all tiles per place
    (eight parts at most: every part of a row leaves float partial outputs), and the list starts with the
    longest: what is short fills in behind them (list scheduling).  Measured against every walk in two parts
    in the grid's own order, attention and merge: head size 64, 2,048 tokens 69 -> 57 us, 4,096 212 -> 180, 8,192
    (no walk cut, no merge) 597 -> 512; head size 128, 2,048 tokens 126 -> 98, 8,192 1,027 -> 890."""
    start = batch.seq_start
    pieces = []                                        # (tiles of 32 keys, piece, request, first row, rows)
    for s in range(batch.n_seqs):
        ctx0, new = batch.seq_ctx[s], start[s + 1] - start[s]
        for j in range(piece_starts[s + 1] - piece_starts[s]):
            first, last = ctx0 + j * piece, ctx0 + min(new, (j + 1) * piece) - 1
            lo = max(0, first - window + 1) if window > 0 else 0
            pieces.append((last // 32 - lo // 32 + 1, piece_starts[s] + j, start[s] + j * piece, min(new, (j + 1) * piece) - j * piece))
    share = sum(p[0] for p in pieces) * head_blocks / ATTENTION_SLOTS
    longest = max(ATTENTION_MIN_WALK, math.ceil(ATTENTION_SHARE_SLACK * share))
    items, row_parts, most = [], [1] * batch.n_tokens, 1
    for tiles, index, row, rows in pieces:
        parts = int(max(1, min(ATTENTION_MAX_PROMPT_SPLITS, -(-tiles // longest))))
        most = max(most, parts)
        row_parts[row:row + rows] = [parts] * rows
        items.extend((-(-tiles // parts), index | (z << 20) | (parts << 24)) for z in range(parts))
    items.sort(key=lambda it: -it[0])
    return [it[1] for it in items], row_parts, most


def attention_plan(batch, n_heads: int, n_kv_heads: int, head_dim: int, window: int = 0):
    """What the matrix-core attention kernel needs to know about a batch before it is launched, worked
    out on the host when the batch is described (``batch``: the step's HostBatch): how every request's
    rows are cut into pieces.  Returns (int32 arrays to go up with the batch, notes for attention()).

    While every request brings one tile of rows at most (decoded tokens), a workgroup is one tile and
    its waves share the tile's keys.  Else four waves with consecutive tiles of a request walk their
    keys together -- but a request that brings a single tile beside them (a decoded token in a step with
    prompt portions) would walk its whole context with one wave: from ATTENTION_APART_CONTEXT cached
    tokens on those requests get a launch of their own in the other form, into the same output."""
    tpt = attention_tile_tokens(n_heads, n_kv_heads)
    S, start = batch.n_seqs, batch.seq_start
    if batch.max_q_len <= tpt:
        if batch.n_tokens == S:                       # one row a request: the same array for every such step
            tiles = _DECODE_TILE_STARTS.get(S)
            if tiles is None:
                tiles = _DECODE_TILE_STARTS[S] = list(range(S + 1))
            return {"tiles": tiles}, dict(form="decode", n_tiles=S)
        return {"tiles": list(range(S + 1))}, dict(form="decode", n_tiles=S)
    piece = tpt * attention_q_tiles(head_dim) * ATTENTION_STAGED_WAVES
    new = [start[s + 1] - start[s] for s in range(S)]
    short = [s for s in range(S) if new[s] <= tpt]
    apart = bool(short) and max(batch.seq_ctx[s] for s in short) >= ATTENTION_APART_CONTEXT
    long_starts, short_starts = [0], [0]
    for s in range(S):
        is_short = new[s] <= tpt
        long_starts.append(long_starts[-1] + (0 if apart and is_short else -(-new[s] // piece)))
        short_starts.append(short_starts[-1] + (-(-new[s] // tpt) if apart and is_short else 0))
    arrays = {"tiles": long_starts}
    notes = dict(form="prompt", n_tiles=long_starts[-1], apart=apart)
    if 0 < long_starts[-1] < (1 << 20):
        group = n_heads // n_kv_heads
        items, row_parts, most = prompt_work_list(batch, long_starts, piece, n_kv_heads * -(-group // 16), window)
        if len(items) <= 65535:
            arrays.update(items=items, row_parts=row_parts)
            notes.update(n_items=len(items), most_parts=most)
    if apart:
        arrays["short_tiles"] = short_starts
        notes.update(n_short=short_starts[-1], longest_short=max(batch.seq_ctx[s] for s in short) + tpt)
    return arrays, notes


def attention(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
              ctx, plan, n_heads: int, n_kv_heads: int, head_dim: int, window: int, scale: float) -> torch.Tensor:
    """Attention of a step's rows over the cache: the matrix-core kernel where it takes the
    sizes (bfloat16, head size a multiple of 16 up to 256, pages of a multiple of 16 tokens),
    else the plain float kernel.  ``plan``: (device arrays, notes) of attention_plan() for this
    batch.  The number of parts the keys are cut into follows from ctx.max_kv_len: in a captured
    step that is the bound of the graph's context bucket, so the choice holds for every replay."""
    work = lambda: attention_work(ctx, n_heads, n_kv_heads, head_dim, window, qkv.element_size())
    if attention_mfma_supported(qkv, k_cache, head_dim):
        if plan is None:
            raise KernelError("attention: the matrix-core kernel needs the batch's attention_plan()")
        arrays, notes = plan
        args = (qkv, k_cache, v_cache, block_table, ctx.seq_start_dev, ctx.seq_ctx_dev)
        sizes = (n_heads, n_kv_heads, head_dim, window, scale)
        if notes["form"] == "decode":
            n_tiles = notes["n_tiles"]
            n_splits = attention_splits(n_tiles, n_heads, n_kv_heads, ctx.max_kv_len, attention_shared_waves(head_dim))
            return attention_mfma(*args, arrays["tiles"], n_tiles, *sizes, n_splits, 1, 1, work=work,
                                  single_rows=ctx.max_q_len == 1 and ctx.n_tokens == ctx.n_seqs)
        q_tiles = attention_q_tiles(head_dim)
        apart = notes["apart"]
        if "items" in arrays:       # the pieces' parts in the order the host chose, longest walks first
            out = attention_mfma(*args, arrays["tiles"], notes["n_tiles"], *sizes, notes["most_parts"], q_tiles, 2, work=work,
                                 row_seq=ctx.row_seq if apart else None, items=arrays["items"], n_items=notes["n_items"],
                                 row_parts=arrays["row_parts"])
        else:
            n_splits = attention_splits(notes["n_tiles"] * ATTENTION_STAGED_WAVES, n_heads, n_kv_heads, ctx.max_kv_len)
            out = attention_mfma(*args, arrays["tiles"], notes["n_tiles"], *sizes, n_splits, q_tiles, 2, work=work,
                                 row_seq=ctx.row_seq if apart else None)
        if apart:
            n_splits = attention_splits(notes["n_short"], n_heads, n_kv_heads, notes["longest_short"],
                                        attention_shared_waves(head_dim))
            attention_mfma(*args, arrays["short_tiles"], notes["n_short"], *sizes, n_splits, 1, 1, out=out,
                           row_seq=ctx.row_seq)
        return out
    return attention_generic(qkv, k_cache, v_cache, block_table, ctx.row_seq, ctx.positions,
                             n_heads, n_kv_heads, head_dim, window, scale, work=work)


def attention_work(ctx, n_heads: int, n_kv_heads: int, head_dim: int, window: int, elem: int):
    """(operations, bytes moved at least, bytes asked for in all) of a step's attention, for the profiler: two
    products of head_dim per query head and visible key; every visible key and value read once per
    request, queries read and outputs written once.  Asked for in all: every piece of a request's new
    rows (the rows one workgroup of the matrix-core kernel's prompt form takes) walks the keys up to its
    last row by itself."""
    pairs = keys = walked = 0
    piece = attention_tile_tokens(n_heads, n_kv_heads) * attention_q_tiles(head_dim) * ATTENTION_STAGED_WAVES
    for s in range(ctx.n_seqs):
        cached, new = ctx.seq_ctx[s], ctx.seq_start[s + 1] - ctx.seq_start[s]
        if window > 0:
            pairs += sum(min(window, cached + i + 1) for i in range(new))
            keys += min(cached + new, window + new - 1)
            walked += sum(min(cached + min(new, j + piece), window + piece - 1) for j in range(0, new, piece))
        else:
            pairs += new * cached + new * (new + 1) // 2
            keys += cached + new
            walked += sum(cached + min(new, j + piece) for j in range(0, new, piece))
    rows = 2 * ctx.n_tokens * n_heads * head_dim
    return (4.0 * pairs * n_heads * head_dim, (2 * keys * n_kv_heads * head_dim + rows) * elem,
            (2 * walked * n_kv_heads * head_dim + rows) * elem)


# ---- a norm added to the stream, xIELU, state-carrying mixers, latent attention ----------------------------------------

def _f32(what: str, name: str, t: Optional[torch.Tensor], shape) -> None:
    if t is not None and (t.dtype != torch.float32 or tuple(t.shape) != tuple(shape)):
        raise KernelError(f"{what}: {name} must be float32 {tuple(shape)}, got {t.dtype} {tuple(t.shape)}")


def rmsnorm_add(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x += y * rsqrt(mean(y^2) + eps) * weight, row by row, in place on the float residual stream x [T, H];
    y [T, H] float32 or bfloat16, weight float32 [H] (as it multiplies)."""
    _dev("rmsnorm_add", x, y, weight)
    if x.dtype != torch.float32 or x.dim() != 2 or tuple(y.shape) != tuple(x.shape):
        raise KernelError(f"rmsnorm_add: x must be float32 [T, H] and y of its shape, got {x.dtype} {tuple(x.shape)} and {tuple(y.shape)}")
    n, hidden = x.shape
    _f32("rmsnorm_add", "weight", weight, (hidden,))
    library.call("bc4g_rmsnorm_add", _ptr(x), _ptr(y), _code(y, "rmsnorm_add"), _ptr(weight), n, hidden, float(eps), _stream(),
                 cost=lambda: (5.0 * n * hidden, n * hidden * (8 + y.element_size())))
    return x


def xielu(z: torch.Tensor, pq: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softplus(p) z^2 + z/2 for z > 0, (1/2 + softplus(q)) (e^z - 1 - z) + z/2 otherwise; pq = (p, q) float32 on the
    device.  ``out`` may be z itself."""
    _dev("xielu", z, pq, out)
    _f32("xielu", "pq", pq, (2,))
    if out is None:
        out = torch.empty_like(z)
    elif out.dtype != z.dtype or out.shape != z.shape:
        raise KernelError("xielu: out must have the input's dtype and shape")
    total = z.numel()
    library.call("bc4g_xielu", _ptr(z), _ptr(out), _code(z, "xielu"), _ptr(pq), total, _stream(),
                 cost=lambda: (6.0 * total, 2 * total * z.element_size()))
    return out


def _rows_of(what: str, name: str, t: torch.Tensor) -> int:
    """The row stride of a [T, C] tensor on the GPU whose rows may be parts of wider rows (columns of one product's
    output): the elements of a row lie side by side."""
    if not t.is_cuda or t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1) or t.stride(0) < t.shape[1]:
        raise KernelError(f"{what}: {name} must be [T, C] on the GPU with a row's elements side by side, got strides {t.stride()} "
                          f"for shape {tuple(t.shape)} on {t.device}")
    return t.stride(0)


def _check_grouping(what: str, ctx, n_rows: int) -> None:
    if ctx.n_tokens != n_rows:
        raise KernelError(f"{what}: {n_rows} rows for a step of {ctx.n_tokens}")
    _i32(what, "row_seq", ctx.row_seq, n_rows)
    _i32(what, "seq_start", ctx.seq_start_dev, ctx.n_seqs + 1)
    _i32(what, "seq_slots", ctx.seq_slots_dev, ctx.n_seqs)


def causal_conv(x: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], ctx, in_bias: Optional[torch.Tensor] = None,
                out_bias: Optional[torch.Tensor] = None, add_input: bool = False) -> torch.Tensor:
    """A causal convolution over time on each channel of x [T, C], continued from every request's state
    [slots, taps - 1, C] (x's dtype), which then receives the request's last taps - 1 inputs.  weight float32
    [taps, C]: by taps (a checkpoint's [C, taps] transposed; its last row is the current token's); a row's input is
    x + in_bias; out_bias is added to the sum, and with ``add_input`` x itself.  ``ctx``: the step's context (which rows
    belong to which request and slot)."""
    _dev("causal_conv", weight, state, in_bias, out_bias)
    in_row = _rows_of("causal_conv", "x", x)             # (x may be a part of one product's wider rows)
    if x.dim() != 2 or weight.dim() != 2 or weight.shape[1] != x.shape[1]:
        raise KernelError(f"causal_conv: x {tuple(x.shape)} and weight {tuple(weight.shape)} (by taps) do not match")
    t, c = x.shape
    taps = weight.shape[0]
    _f32("causal_conv", "weight", weight, (taps, c))
    _f32("causal_conv", "in_bias", in_bias, (c,))
    _f32("causal_conv", "out_bias", out_bias, (c,))
    if taps > 1:
        if state is None or state.dtype != x.dtype or state.dim() != 3 or tuple(state.shape[1:]) != (taps - 1, c):
            raise KernelError(f"causal_conv: state must be {x.dtype} [slots, {taps - 1}, {c}]")
        if max(ctx.seq_slots, default=0) >= state.shape[0]:
            raise KernelError(f"causal_conv: a slot beyond the state's {state.shape[0]}")
    _check_grouping("causal_conv", ctx, t)
    out = torch.empty((t, c), dtype=x.dtype, device=x.device)
    library.call("bc4g_causal_conv", _ptr(x), _code(x, "causal_conv"), _ptr(in_bias), _ptr(weight), _ptr(out_bias),
                 1 if add_input else 0, _ptr(out), _ptr(state), _ptr(ctx.row_seq), _ptr(ctx.seq_start_dev),
                 _ptr(ctx.seq_slots_dev), t, ctx.n_seqs, c, taps, in_row, _stream(),
                 cost=lambda: (2.0 * t * c * taps, 2 * t * c * x.element_size()))
    return out


def rmsnorm_shift(x: torch.Tensor, weight: torch.Tensor, eps: float, mix: torch.Tensor, state: torch.Tensor, ctx,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """An RMS norm of the float32 stream x [T, H] and the token shift behind it in one launch: h = norm(x) (rounded to
    ``out_dtype``), out[t] = h[t] + (h[t - 1] - h[t]) * mix along a request's rows.  ``state`` [slots, 1, H] (``out_dtype``)
    holds every request's last h so far -- h[-1] for its first row of this step -- and receives the last h of this step.
    weight, mix: float32 [H]."""
    _dev("rmsnorm_shift", x, weight, mix, state)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous():
        raise KernelError(f"rmsnorm_shift: x must be float32 [T, H], got {x.dtype} {tuple(x.shape)}")
    t, hidden = x.shape
    _f32("rmsnorm_shift", "weight", weight, (hidden,))
    _f32("rmsnorm_shift", "mix", mix, (hidden,))
    if state.dtype != out_dtype or state.dim() != 3 or tuple(state.shape[1:]) != (1, hidden) or not state.is_contiguous():
        raise KernelError(f"rmsnorm_shift: state must be {out_dtype} [slots, 1, {hidden}], got {state.dtype} {tuple(state.shape)}")
    if max(ctx.seq_slots, default=0) >= state.shape[0]:
        raise KernelError(f"rmsnorm_shift: a slot beyond the state's {state.shape[0]}")
    _check_grouping("rmsnorm_shift", ctx, t)
    out = torch.empty((t, hidden), dtype=out_dtype, device=x.device)
    library.call("bc4g_rmsnorm_shift", _ptr(x), _ptr(weight), _ptr(mix), _ptr(out), _ptr(state), _code(out, "rmsnorm_shift"),
                 _ptr(ctx.row_seq), _ptr(ctx.seq_start_dev), _ptr(ctx.seq_slots_dev), t, hidden, float(eps), _stream(),
                 cost=lambda: (8.0 * t * hidden, t * hidden * (4 + out.element_size())))
    return out


RGLRU_CHUNK = 64            # rows of a request that one thread of the recurrence walks


def rglru(u: torch.Tensor, y: torch.Tensor, w_gates: torch.Tensor, ra_b: torch.Tensor, ri_b: torch.Tensor,
          lam: torch.Tensor, y_bias: Optional[torch.Tensor], state: torch.Tensor, ctx) -> torch.Tensor:
    """The real-gated linear recurrent unit over a step's rows: u, y [T, W]; w_gates [blocks, 2 bs, bs] (of every block
    the matrix of the recurrence gate, then that of the input gate, each [out, in]); biases and lam float32 [W]; state
    float32 [slots, W].  The gates' sums are a product per block (float32 out), the gates, the decay and the state
    float32.  Returns S_t * gelu_tanh(y + y_bias) in u's dtype."""
    _dev("rglru", u, w_gates, ra_b, ri_b, lam, y_bias, state)
    y_row = _rows_of("rglru", "y", y)                     # (y may be a part of one product's wider rows)
    if u.dim() != 2 or y.shape != u.shape or y.dtype != u.dtype:
        raise KernelError(f"rglru: u and y must be alike [T, W], got {tuple(u.shape)} and {tuple(y.shape)}")
    t, w = u.shape
    if w_gates.dim() != 3 or w_gates.shape[1] != 2 * w_gates.shape[2] or w_gates.shape[0] * w_gates.shape[2] != w:
        raise KernelError(f"rglru: gate matrices {tuple(w_gates.shape)} do not cut {w} channels into blocks of [2 bs, bs]")
    for name, v in (("ra_b", ra_b), ("ri_b", ri_b), ("lam", lam), ("y_bias", y_bias)):
        _f32("rglru", name, v, (w,))
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != w or max(ctx.seq_slots, default=0) >= state.shape[0]:
        raise KernelError(f"rglru: state must be float32 [slots, {w}] with a row for every slot of the step")
    _check_grouping("rglru", ctx, t)
    blocks, bs = w_gates.shape[0], w_gates.shape[2]
    pre = torch.empty((t, blocks, 2 * bs), dtype=torch.float32, device=u.device)
    heads_gemm(u.view(t, blocks, bs), w_gates, pre, k=bs, n=2 * bs)
    most = max(int(ctx.seq_start[s + 1] - ctx.seq_start[s]) for s in range(ctx.n_seqs))
    chunks = -(-most // RGLRU_CHUNK)
    scratch = torch.empty((2 * chunks + 1, ctx.n_seqs, w), dtype=torch.float32, device=u.device)
    out = torch.empty_like(u)
    library.call("bc4g_rglru_scan", _ptr(pre), _ptr(u), _ptr(y), _code(y, "rglru"), _ptr(ra_b), _ptr(ri_b), _ptr(lam), _ptr(y_bias),
                 _ptr(out), _ptr(state), _ptr(scratch[:chunks]), _ptr(scratch[chunks:2 * chunks]), _ptr(scratch[2 * chunks]),
                 _ptr(ctx.seq_start_dev), _ptr(ctx.seq_slots_dev), t, ctx.n_seqs, most, w, blocks, y_row, _stream(),
                 cost=lambda: (40.0 * t * w, t * w * (16 + 5 * u.element_size())))
    return out


LATENT_MAX_ROW = 1024       # numbers of a latent cache row (latent + rotated key part) the attention kernel takes
LATENT_MFMA = True          # (off: the plain kernel also where the matrix-core kernel takes the sizes)
LATENT_ENOUGH_GROUPS = 256  # workgroups from which on the keys are not cut into parts
LATENT_MAX_SPLITS = 64


def attention_latent_mfma_takes(cache: torch.Tensor, rank: int, rot: int) -> bool:
    """Whether the matrix-core kernel serves this cache: bfloat16, rows of whole k-steps of 32, a latent of whole
    blocks of 16, within what a wave's registers hold."""
    dk = rank + rot
    return (LATENT_MFMA and cache.dtype == torch.bfloat16 and dk % 32 == 0 and rank % 16 == 0 and dk <= 576 and 0 < rank <= 512
            and cache.data_ptr() % 16 == 0)


def latent_splits(seq_start, heads: int, max_kv_len: int) -> int:
    """Into how many parts the matrix-core kernel cuts every walk over the keys: one where the step's rows fill the
    GPU by themselves (a workgroup takes four tiles of 16 (token, head) pairs of one request), else as many as bring
    the workgroups to twice that, while a part keeps a key tile of 32."""
    hb = min(heads, 16)
    tpt, n_hg = 16 // hb, -(-heads // hb)
    tiles = [-(-int(seq_start[s + 1] - seq_start[s]) // tpt) * n_hg for s in range(len(seq_start) - 1)]
    # (no request with four tiles: a workgroup a tile, else four tiles a workgroup)
    groups = sum(tiles) if max(tiles, default=0) < 4 else sum(-(-n // 4) for n in tiles)
    if groups >= LATENT_ENOUGH_GROUPS or groups == 0:
        return 1
    key_tiles = -(-max_kv_len // 32)
    return max(1, min(-(-2 * LATENT_ENOUGH_GROUPS // groups), key_tiles, LATENT_MAX_SPLITS))


def latent_angles(positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """(cos, sin) of every row's angles position * base^(-2i / dims), float32 [T, dims / 2, 2], worked out in double:
    made once a step and read by every layer that rotates alike."""
    _dev("latent_angles", positions)
    t = positions.shape[0]
    _i32("latent_angles", "positions", positions, t)
    table = torch.empty((t, dims // 2, 2), dtype=torch.float32, device=positions.device)
    library.call("bc4g_latent_angles", _ptr(positions), _ptr(table), t, int(dims), float(base), _stream(),
                 cost=lambda: (0.0, t * dims * 4))
    return table


def latent_prepare(q: torch.Tensor, dkv: torch.Tensor, g: torch.Tensor, eps: float, angles: Optional[torch.Tensor],
                   slot_map: Optional[torch.Tensor], cache: Optional[torch.Tensor], q_lat: torch.Tensor, heads: int, plain: int,
                   rot: int, rank: int, dims: int) -> None:
    """Writes [rmsnorm(dkv[:, :rank]) * g | rotate(dkv[:, rank:])] into every row's cache slot (``cache`` None: nowhere)
    and every head's rotated query part into q_lat[:, h, rank:].  ``angles``: latent_angles of the rows (None where
    nothing is rotated, dims 0)."""
    _dev("latent_prepare", g, angles, slot_map, cache, q_lat)
    q_row, dkv_row = _rows_of("latent_prepare", "q", q), _rows_of("latent_prepare", "dkv", dkv)   # (parts of one product's rows)
    t = q.shape[0]
    if q.dtype != dkv.dtype or tuple(q.shape) != (t, heads * (plain + rot)) or tuple(dkv.shape) != (t, rank + rot):
        raise KernelError(f"latent_prepare: q {tuple(q.shape)} / dkv {tuple(dkv.shape)} do not fit heads={heads} plain={plain} rot={rot} rank={rank}")
    _f32("latent_prepare", "g", g, (rank,))
    _f32("latent_prepare", "q_lat", q_lat, (t, heads, rank + rot))
    if dims:
        _f32("latent_prepare", "angles", angles, (t, dims // 2, 2))
    if cache is not None:
        if cache.dtype != q.dtype or cache.dim() != 3 or cache.shape[2] != rank + rot:
            raise KernelError(f"latent_prepare: the cache must be {q.dtype} [pages, page_tokens, {rank + rot}], got {cache.dtype} {tuple(cache.shape)}")
        _i32("latent_prepare", "slot_map", slot_map, t)
    library.call("bc4g_latent_prepare", _ptr(q), _ptr(dkv), _code(q, "latent_prepare"), _ptr(g), float(eps),
                 _ptr(angles) if dims else None, _ptr(slot_map) if cache is not None else None, _ptr(cache), _ptr(q_lat), t, heads,
                 plain, rot, rank, int(dims), q_row, dkv_row, _stream(), cost=lambda: (4.0 * t * (rank + (heads + 1) * rot), t * (q.element_size() * (heads + 2) * rot + 2 * rank * q.element_size())))


def heads_gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, k: int, n: int) -> None:
    """out[t, h, :n] = w[h] a[t, h, :k] for a [T, heads, >= k], w [heads, n, k], out [T, heads, >= n] (the last
    dimensions may be longer than k and n: parts of wider rows)."""
    _dev("heads_gemm", w, out)
    if a.dim() != 3 or out.dim() != 3 or w.dim() != 3 or a.shape[:2] != out.shape[:2] or a.shape[2] < k or out.shape[2] < n \
            or tuple(w.shape) != (a.shape[1], n, k):
        raise KernelError(f"heads_gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit k={k}, n={n}")
    if not a.is_cuda or a.stride(2) != 1 or a.stride(1) < k or a.stride(0) < a.stride(1):      # (a's rows may be parts of wider rows)
        raise KernelError(f"heads_gemm: a must lie on the GPU with a head's elements side by side, got strides {a.stride()}")
    t, heads = a.shape[0], a.shape[1]
    library.call("bc4g_heads_gemm", _ptr(a), _code(a, "heads_gemm"), a.stride(0), a.stride(1), _ptr(w), _code(w, "heads_gemm"),
                 _ptr(out), _code(out, "heads_gemm"), heads * out.shape[2], out.shape[2], t, n, k, heads, _stream(),
                 cost=lambda: (2.0 * t * heads * n * k, heads * n * k * w.element_size() + t * heads * (k * a.element_size() + n * out.element_size())))


def attention_latent(q_lat: torch.Tensor, cache: torch.Tensor, sink: Optional[torch.Tensor], block_table: torch.Tensor, ctx,
                     heads: int, rank: int, rot: int, page_tokens: int, window: int, scale: float) -> torch.Tensor:
    """Causal attention of every row over its request's latent cache rows; float32 [T, heads, rank] (the weighted
    sums of the latents, before the values' up-projection)."""
    _dev("attention_latent", q_lat, cache, sink, block_table)
    t = q_lat.shape[0]
    _f32("attention_latent", "q_lat", q_lat, (t, heads, rank + rot))
    _f32("attention_latent", "sink", sink, (heads,))
    if rank + rot > LATENT_MAX_ROW:
        raise KernelError(f"attention_latent: a cache row of {rank + rot} numbers is beyond {LATENT_MAX_ROW}")
    if cache.dim() != 3 or tuple(cache.shape[1:]) != (page_tokens, rank + rot):
        raise KernelError(f"attention_latent: the cache must be [pages, {page_tokens}, {rank + rot}], got {tuple(cache.shape)}")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] < ctx.n_seqs:
        raise KernelError("attention_latent: the block table must be int32 [requests, pages]")
    if block_table.shape[1] * page_tokens < ctx.max_kv_len and not ctx.captured:
        raise KernelError(f"attention_latent: the block table's {block_table.shape[1]} pages do not hold {ctx.max_kv_len} tokens")
    _i32("attention_latent", "row_seq", ctx.row_seq, t)
    _i32("attention_latent", "positions", ctx.positions, t)
    out = torch.empty((t, heads, rank), dtype=torch.float32, device=q_lat.device)
    if attention_latent_mfma_takes(cache, rank, rot):
        _i32("attention_latent", "seq_start", ctx.seq_start_dev, ctx.n_seqs + 1)
        _i32("attention_latent", "seq_ctx", ctx.seq_ctx_dev, ctx.n_seqs)
        n_splits = latent_splits(ctx.seq_start, heads, ctx.max_kv_len)
        most = max(int(ctx.seq_start[s + 1] - ctx.seq_start[s]) for s in range(ctx.n_seqs))
        part_o = part_ml = None
        if n_splits > 1:
            part_o = torch.empty((n_splits, t, heads, rank), dtype=torch.float32, device=q_lat.device)
            part_ml = torch.empty((n_splits, t, heads, 2), dtype=torch.float32, device=q_lat.device)
        library.call("bc4g_attention_latent_mfma", _ptr(q_lat), _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(cache), _ptr(sink),
                     _ptr(block_table), block_table.shape[1], _ptr(ctx.seq_start_dev), _ptr(ctx.seq_ctx_dev), ctx.n_seqs, t, most,
                     heads, rank, rot, page_tokens, int(window), float(scale), n_splits, _stream(),
                     cost=lambda: attention_latent_work(ctx, heads, rank, rot, window, cache.element_size()))
        return out
    library.call("bc4g_attention_latent", _ptr(q_lat), _ptr(out), _ptr(cache), _code(cache, "attention_latent"), _ptr(sink),
                 _ptr(block_table), block_table.shape[1], _ptr(ctx.row_seq), _ptr(ctx.positions), t, heads, rank, rot, page_tokens,
                 int(window), float(scale), _stream(), cost=lambda: attention_latent_work(ctx, heads, rank, rot, window, cache.element_size()))
    return out


def attention_latent_work(ctx, heads: int, rank: int, rot: int, window: int, elem: int):
    """(operations, bytes to read at least) of latent attention over a step's rows."""
    pairs = keys = 0
    for s in range(ctx.n_seqs):
        cached, new = int(ctx.seq_ctx[s]), int(ctx.seq_start[s + 1] - ctx.seq_start[s])
        if window > 0:
            pairs += sum(min(window, cached + i + 1) for i in range(new))
            keys += min(cached + new, window + new - 1)
        else:
            pairs += new * cached + new * (new + 1) // 2
            keys += cached + new
    return 2.0 * pairs * heads * (2 * rank + rot), float(keys * (rank + rot) * elem)


# ---- a residual stream in several copies, a pointwise norm, clamped gated units -----------------------------------------

MAX_STREAMS = 16            # copies of the residual stream the kernels take


def _streams(what: str, x: torch.Tensor):
    if x.dtype != torch.float32 or x.dim() != 3 or not (1 <= x.shape[1] <= MAX_STREAMS):
        raise KernelError(f"{what}: the stream must be float32 [T, copies (at most {MAX_STREAMS}), H], got {x.dtype} {tuple(x.shape)}")
    return x.shape


def streams_fill(x: torch.Tensor, copies: int) -> torch.Tensor:
    """[T, H] float32 -> [T, copies, H], every copy equal to x."""
    _dev("streams_fill", x)
    if x.dtype != torch.float32 or x.dim() != 2 or copies < 1:
        raise KernelError(f"streams_fill: x must be float32 [T, H], got {x.dtype} {tuple(x.shape)}")
    t, hidden = x.shape
    out = torch.empty((t, copies, hidden), dtype=torch.float32, device=x.device)
    library.call("bc4g_streams_fill", _ptr(x), _ptr(out), t, copies, hidden, _stream(),
                 cost=lambda: (0.0, 4.0 * t * hidden * (1 + copies)))
    return out


def streams_read(x: torch.Tensor, read: Optional[torch.Tensor], pointwise, out_dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None, n_rows: Optional[int] = None) -> torch.Tensor:
    """sum_s read[s] x[:, s] of the copies x [T, n, H] (``read`` None: every copy counts once), at ``rows`` only if
    given; with ``pointwise`` = (alpha [1], g [H], b [H], out_scale) the norm (tanh(alpha u) g + b) out_scale of it."""
    t, n, hidden = _streams("streams_read", x)
    alpha, g, b, out_scale = pointwise if pointwise is not None else (None, None, None, 1.0)
    _dev("streams_read", x, read, alpha, g, b, rows)
    _f32("streams_read", "read", read, (n,))
    _f32("streams_read", "alpha", alpha, (1,))
    _f32("streams_read", "g", g, (hidden,))
    _f32("streams_read", "b", b, (hidden,))
    if rows is not None:
        t = rows.numel() if n_rows is None else n_rows
        _i32("streams_read", "rows", rows, t)
    out = torch.empty((t, hidden), dtype=out_dtype, device=x.device)
    library.call("bc4g_streams_read", _ptr(x), _ptr(rows), _ptr(read), _ptr(alpha), _ptr(g), _ptr(b), float(out_scale), _ptr(out),
                 _code(out, "streams_read"), t, n, hidden, _stream(),
                 cost=lambda: (2.0 * t * hidden * (n + 2), t * hidden * (4 * n + out.element_size())))
    return out


def streams_write(x: torch.Tensor, y: torch.Tensor, mix: torch.Tensor, write: torch.Tensor,
                  next_read: Optional[torch.Tensor] = None, pointwise=None, out_dtype: Optional[torch.dtype] = None):
    """x'[:, t] = sum_s mix[s, t] x[:, s] + write[t] y in place on the copies x [T, n, H] (y float32 [T, H]); with
    ``next_read`` also returns the next reader's input from the new copies (see streams_read; the norm's out_scale is 1)."""
    t, n, hidden = _streams("streams_write", x)
    alpha, g, b, _ = pointwise if pointwise is not None else (None, None, None, 1.0)
    _dev("streams_write", x, y, mix, write, next_read, alpha, g, b)
    _f32("streams_write", "y", y, (t, hidden))
    _f32("streams_write", "mix", mix, (n, n))
    _f32("streams_write", "write", write, (n,))
    _f32("streams_write", "next_read", next_read, (n,))
    _f32("streams_write", "alpha", alpha, (1,))
    _f32("streams_write", "g", g, (hidden,))
    _f32("streams_write", "b", b, (hidden,))
    out = None
    if next_read is not None:
        out = torch.empty((t, hidden), dtype=out_dtype or torch.float32, device=x.device)
    library.call("bc4g_streams_write", _ptr(x), _ptr(y), _ptr(mix), _ptr(write), _ptr(next_read), _ptr(alpha), _ptr(g), _ptr(b),
                 _ptr(out), _code(out, "streams_write") if out is not None else F32, t, n, hidden, _stream(),
                 cost=lambda: (2.0 * t * hidden * n * (n + 2), t * hidden * (8 * n + 4 + (out.element_size() if out is not None else 0))))
    return out


def clamped_glu(gu: torch.Tensor, limit: float, slope: float) -> torch.Tensor:
    """gu [T, 2I] (a row's gates, then its ups) -> g sigmoid(slope g) (u + 1) with g = min(gate, limit),
    u = clamp(up, -limit, limit), [T, I]."""
    _dev("clamped_glu", gu)
    if gu.dim() != 2 or gu.shape[1] % 2:
        raise KernelError(f"clamped_glu: input must be [T, 2I], got {tuple(gu.shape)}")
    t, inter = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((t, inter), dtype=gu.dtype, device=gu.device)
    library.call("bc4g_clamped_glu", _ptr(gu), _ptr(out), _code(gu, "clamped_glu"), float(limit), float(slope), t, inter, _stream(),
                 cost=lambda: (8.0 * t * inter, 3 * t * inter * gu.element_size()))
    return out


# ---- heads: rotation tables, preparation, finishing; linear attention with a decayed state; attention with two maps -----

HEADS_MAX_DIM = 256         # elements of a head that heads_prepare, heads_finish, decay_scan and attention_maps take
DECAY_SCAN_CHUNK = 32       # rows of a request that one workgroup of the scan walks

ACT_NONE, ACT_SILU, ACT_SIGMOID = 0, 1, 2
ATTENTION_MAPS_FULL = 4096   # (row, head) pairs from which on one wave walks a row's keys alone


def _part_of_rows(what: str, name: str, t: torch.Tensor, width: int) -> int:
    """The row stride of a [T, >= width] tensor on the GPU that may be a part of one product's wider rows."""
    if not t.is_cuda or t.dim() != 2 or t.shape[1] < width or (t.shape[1] > 1 and t.stride(1) != 1) or t.stride(0) < t.shape[1]:
        raise KernelError(f"{what}: {name} must be [T, {width}] on the GPU with a row's elements side by side, got shape "
                          f"{tuple(t.shape)} with strides {t.stride()} on {t.device}")
    return t.stride(0)


def rotary_table(positions: torch.Tensor, freqs: torch.Tensor, amplitude: float = 1.0) -> torch.Tensor:
    """[T, half, 2] float32: cos and sin of positions[t] * freqs[i] (freqs float64 [half] on the device), times
    ``amplitude``; the angles are worked out in double."""
    _dev("rotary_table", positions, freqs)
    n, half = positions.numel(), freqs.numel()
    _i32("rotary_table", "positions", positions, n)
    if freqs.dtype != torch.float64 or freqs.dim() != 1 or half < 1:
        raise KernelError(f"rotary_table: freqs must be float64 [half], got {freqs.dtype} {tuple(freqs.shape)}")
    table = torch.empty((n, half, 2), dtype=torch.float32, device=positions.device)
    library.call("bc4g_rotary_table", _ptr(positions), _ptr(freqs), float(amplitude), _ptr(table), n, half, _stream(),
                 cost=lambda: (40.0 * n * half, 8.0 * n * half))
    return table


class _PrepareSection(ctypes.Structure):
    """One section of heads_prepare_many, as the library's ``bc4g_prepare_section``."""
    _fields_ = [("src", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("norm_w", ctypes.c_void_p), ("table", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("slot_map", ctypes.c_void_p), ("in_row", ctypes.c_long), ("out_row", ctypes.c_long),
                ("page_stride", ctypes.c_long), ("head_stride", ctypes.c_long), ("token_stride", ctypes.c_long),
                ("in_dtype", ctypes.c_int), ("out_dtype", ctypes.c_int), ("half", ctypes.c_int), ("page_tokens", ctypes.c_int),
                ("heads", ctypes.c_int), ("dim", ctypes.c_int), ("eps", ctypes.c_float), ("factor", ctypes.c_float),
                ("pairing", ctypes.c_int), ("unit_after", ctypes.c_int), ("norm_rows", ctypes.c_int)]


def heads_section(x: torch.Tensor, heads: int, dim: int, out: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                  norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0, table: Optional[torch.Tensor] = None,
                  factor: float = 1.0, slot_map: Optional[torch.Tensor] = None, page_tokens: int = 0,
                  neighbours: bool = False, unit_after: bool = False, norm_rows: bool = False):
    """One section for heads_prepare_many: every head of x [T, heads * dim] (may be a part of wider rows): + bias, RMS norm
    over the head with ``norm_weight`` [dim], rotation by ``table`` [T, half, 2] (element i with element i + half, or with
    ``neighbours`` element 2i with element 2i + 1), with ``unit_after`` division by sqrt(mean(head^2) + eps) of the head as
    it stands then, times ``factor``.  With ``norm_rows`` the norm before the rotation is taken over the whole row, all heads
    at once, and ``norm_weight`` is [heads * dim].  ``out``: [T, heads, dim] (float32 or bfloat16), or with ``slot_map`` a cache
    [pages, heads, page_tokens, dim] whose slot page * page_tokens + offset receives the row.  Checked here; the tensors
    must live until the launch."""
    _dev("heads_prepare", bias, norm_weight, table, out, slot_map)
    in_row = _part_of_rows("heads_prepare", "x", x, heads * dim)
    t = x.shape[0]
    _f32("heads_prepare", "bias", bias, (heads * dim,))
    _f32("heads_prepare", "norm_weight", norm_weight, (heads * dim,) if norm_rows else (dim,))
    half = 0
    if table is not None:
        half = table.shape[1]
        _f32("heads_prepare", "table", table, (t, half, 2))
    if dim > HEADS_MAX_DIM or 2 * half > dim:
        raise KernelError(f"heads_prepare: heads of {dim} elements (at most {HEADS_MAX_DIM}) with {half} rotated pairs")
    if slot_map is not None:
        _i32("heads_prepare", "slot_map", slot_map, t)
        if out.dim() != 4 or tuple(out.shape[1:]) != (heads, page_tokens, dim):
            raise KernelError(f"heads_prepare: the cache must be [pages, {heads}, {page_tokens}, {dim}], got {tuple(out.shape)}")
        page_stride, head_stride, token_stride, out_row = heads * page_tokens * dim, page_tokens * dim, dim, 0
    else:
        if tuple(out.shape) != (t, heads, dim):
            raise KernelError(f"heads_prepare: out must be [{t}, {heads}, {dim}], got {tuple(out.shape)}")
        page_stride = head_stride = token_stride = 0
        out_row = heads * dim
    section = _PrepareSection(_ptr(x), _ptr(bias), _ptr(norm_weight), _ptr(table), _ptr(out), _ptr(slot_map), in_row, out_row,
                              page_stride, head_stride, token_stride, _code(x, "heads_prepare"), _code(out, "heads_prepare"), half,
                              page_tokens, heads, dim, float(eps), float(factor), 1 if neighbours else 0, 1 if unit_after else 0,
                              1 if norm_rows and norm_weight is not None else 0)
    return section, t, t * heads * dim, x.element_size() + out.element_size()


def heads_prepare_many(sections) -> None:
    """Up to four sections (heads_section) of the same step's rows in one launch: the queries, keys and values of an
    attention layer, say."""
    if not 1 <= len(sections) <= 4 or len({s[1] for s in sections}) != 1:
        raise KernelError(f"heads_prepare: {len(sections)} sections (1 to 4) of {sorted({s[1] for s in sections})} rows")
    array = (_PrepareSection * len(sections))(*[s[0] for s in sections])
    library.call("bc4g_heads_prepare_many", ctypes.cast(array, ctypes.c_void_p), len(sections), sections[0][1], _stream(),
                 cost=lambda: (8.0 * sum(s[2] for s in sections), sum(s[2] * s[3] for s in sections)))


def heads_prepare(x: torch.Tensor, heads: int, dim: int, out: torch.Tensor, **how) -> torch.Tensor:
    """One section alone (see heads_section); returns ``out``."""
    heads_prepare_many([heads_section(x, heads, dim, out, **how)])
    return out


def heads_finish(o: torch.Tensor, out_dtype: torch.dtype, *, weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                 factor: float = 1.0, gate: Optional[torch.Tensor] = None, act: int = ACT_NONE) -> torch.Tensor:
    """o float32 [T, heads, vdim] -> o / sqrt(mean(o^2) + eps) (* weight [vdim]) * factor * act(gate) per head, as
    [T, heads * vdim] in ``out_dtype``; gate [T, heads * vdim] may be a part of wider rows."""
    _dev("heads_finish", o, weight)
    if o.dtype != torch.float32 or o.dim() != 3 or o.shape[2] > HEADS_MAX_DIM:
        raise KernelError(f"heads_finish: o must be float32 [T, heads, vdim <= {HEADS_MAX_DIM}], got {o.dtype} {tuple(o.shape)}")
    t, heads, vdim = o.shape
    _f32("heads_finish", "weight", weight, (vdim,))
    gate_row = _part_of_rows("heads_finish", "gate", gate, heads * vdim) if gate is not None else 0
    if gate is not None and gate.shape[0] != t:
        raise KernelError(f"heads_finish: gate has {gate.shape[0]} rows, o {t}")
    out = torch.empty((t, heads * vdim), dtype=out_dtype, device=o.device)
    library.call("bc4g_heads_finish", _ptr(o), _ptr(weight), float(eps), float(factor), _ptr(gate),
                 _code(gate, "heads_finish") if gate is not None else F32, gate_row, int(act), _ptr(out), _code(out, "heads_finish"),
                 t, heads, vdim, _stream(),
                 cost=lambda: (10.0 * t * heads * vdim, t * heads * vdim * (4 + 2 * out.element_size())))
    return out


def decay_scan_chunks(batch) -> Tuple[list, int]:
    """(first chunk of every request among all chunks of the requests that bring two chunks or more, how many such
    chunks there are) for a step's HostBatch."""
    base, total = [], 0
    for s in range(batch.n_seqs):
        n = -(-int(batch.seq_start[s + 1] - batch.seq_start[s]) // DECAY_SCAN_CHUNK)
        base.append(total)
        if n >= 2:
            total += n
    return base, total


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, ctx, heads: int, dim: int, vdim: int, *,
               head_decay: Optional[torch.Tensor] = None, z: Optional[torch.Tensor] = None, z_bias: Optional[torch.Tensor] = None,
               inv_tau: float = 1.0, q_scale: float = 1.0, chunk_base: Optional[torch.Tensor] = None, n_chunks: int = 0) -> torch.Tensor:
    """S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T (q_t q_scale) per request and head over a step's rows; q, k
    [T, heads * dim], v [T, heads * vdim] (float32 or bfloat16, each may be a part of wider rows); state float32
    [slots, heads, dim, vdim] is read and left.  a_t = head_decay[head] (float32 [heads]) or, with gate logits z
    [T, heads * dim], sigmoid(z + z_bias)^inv_tau.  ``chunk_base`` (int32 [S] on the device) and ``n_chunks``:
    see decay_scan_chunks -- needed when a request brings more than DECAY_SCAN_CHUNK rows.  Returns float32 [T, heads, vdim]."""
    _dev("decay_scan", head_decay, z_bias, state, chunk_base)
    t = q.shape[0]
    q_row = _part_of_rows("decay_scan", "q", q, heads * dim)
    k_row = _part_of_rows("decay_scan", "k", k, heads * dim)
    v_row = _part_of_rows("decay_scan", "v", v, heads * vdim)
    z_row = _part_of_rows("decay_scan", "z", z, heads * dim) if z is not None else 0
    if k.shape[0] != t or v.shape[0] != t or (z is not None and z.shape[0] != t):
        raise KernelError("decay_scan: q, k, v and z must have the same number of rows")
    if (head_decay is None) == (z is None):
        raise KernelError("decay_scan: either a decay per head or gate logits per token")
    _f32("decay_scan", "head_decay", head_decay, (heads,))
    _f32("decay_scan", "z_bias", z_bias, (heads * dim,))
    if (state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, vdim)
            or max(ctx.seq_slots, default=0) >= state.shape[0]):
        raise KernelError(f"decay_scan: state must be float32 [slots, {heads}, {dim}, {vdim}] with a row for every slot of the step")
    if dim > HEADS_MAX_DIM:
        raise KernelError(f"decay_scan: {dim} key channels a head are beyond the kernel's {HEADS_MAX_DIM}")
    _check_grouping("decay_scan", ctx, t)
    most = max(int(ctx.seq_start[s + 1] - ctx.seq_start[s]) for s in range(ctx.n_seqs))
    chunk_state = chunk_decay = None
    if most > DECAY_SCAN_CHUNK:
        if chunk_base is None or n_chunks < 2:
            raise KernelError("decay_scan: a request brings several chunks of rows and the chunks' places are not given")
        _i32("decay_scan", "chunk_base", chunk_base, ctx.n_seqs)
        chunk_state = torch.empty((n_chunks, heads, dim, vdim), dtype=torch.float32, device=state.device)
        chunk_decay = torch.empty((n_chunks, heads, dim), dtype=torch.float32, device=state.device)
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=state.device)
    passes = 2 if most > DECAY_SCAN_CHUNK else 1
    library.call("bc4g_decay_scan", _ptr(q), _code(q, "decay_scan"), q_row, float(q_scale), _ptr(k), _code(k, "decay_scan"), k_row,
                 _ptr(v), _code(v, "decay_scan"), v_row, _ptr(head_decay), _ptr(z), _code(z, "decay_scan") if z is not None else F32,
                 z_row, _ptr(z_bias), float(inv_tau), _ptr(out), _ptr(state), _ptr(chunk_state), _ptr(chunk_decay),
                 _ptr(ctx.seq_start_dev), _ptr(ctx.seq_slots_dev), _ptr(chunk_base), t, ctx.n_seqs, most, heads, dim, vdim, _stream(),
                 cost=lambda: (passes * 4.0 * t * heads * dim * vdim,
                               t * heads * (2 * dim * q.element_size() + vdim * (v.element_size() + 4))
                               + 8.0 * ctx.n_seqs * heads * dim * vdim))
    return out


def attention_maps(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, ctx, out_dtype: torch.dtype,
                   n_heads: int, n_kv_heads: int, maps: int, dim: int, vdim: int, window: int, keep_first: int, scale: float, *,
                   lam: float = 0.0, normalize: bool = False, eps: float = 0.0, factor: float = 1.0,
                   gate: Optional[torch.Tensor] = None, act: int = ACT_SIGMOID, waves: int = 0,
                   sink: Optional[torch.Tensor] = None, far: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                   block: int = 0, cap: float = 0.0, point: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax attention with ``maps`` (1 or 2) score maps per query head over the same values: q float32
    [T, n_heads, maps, dim]; keys [pages, n_kv_heads * maps, page_tokens, dim], values [pages, n_kv_heads, page_tokens, vdim].
    A row at position p sees key j <= p if p - j < window or j < keep_first (window 0: every key).  o = a1 - lam a2,
    with ``normalize`` divided by sqrt(mean(o^2) + eps) over the head, times ``factor`` and act(gate); [T, n_heads * vdim].
    ``waves``: how many waves cut one row's keys among them (0: chosen here -- one where the rows fill the GPU, up to
    eight where few rows walk long contexts).  ``sink`` (float32 [n_heads]): exp(sink) joins every map's denominator, with
    no key and no value.  ``far`` = (r1, r2), float32 [n_heads] each: r1 ln(1 + r2 (p - j)) is taken off the scaled score.
    ``block`` (instead of a window): a row sees the keys j <= p of its own block of that many positions, counted from 0.
    ``cap``: the scaled score becomes cap tanh(score / cap).  ``point`` (float32 [n_heads], no sink then): no softmax -- a
    visible key weighs sigmoid(score + point[head]), nothing is normalised over keys."""
    _dev("attention_maps", q, k_cache, v_cache, block_table, sink, point, *(far or ()))
    _f32("attention_maps", "sink", sink, (n_heads,))
    _f32("attention_maps", "point", point, (n_heads,))
    if block < 0 or (block > 0 and (window > 0 or keep_first > 0)) or cap < 0 or (point is not None and sink is not None):
        raise KernelError(f"attention_maps: block {block} beside window {window} and {keep_first} kept keys, cap {cap}, or a sink "
                          "beside weights that are no softmax")
    for v in far or ():
        _f32("attention_maps", "far", v, (n_heads,))
    t = q.shape[0]
    if q.dtype != torch.float32 or tuple(q.shape) != (t, n_heads, maps, dim):
        raise KernelError(f"attention_maps: q must be float32 [T, {n_heads}, {maps}, {dim}], got {q.dtype} {tuple(q.shape)}")
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.dtype != v_cache.dtype:
        raise KernelError("attention_maps: caches must be [pages, heads, page_tokens, size] of one dtype")
    pages, _, page_tokens, _ = k_cache.shape
    if tuple(k_cache.shape[1:]) != (n_kv_heads * maps, page_tokens, dim) or tuple(v_cache.shape) != (pages, n_kv_heads, page_tokens, vdim):
        raise KernelError(f"attention_maps: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit {n_kv_heads} key/value heads, "
                          f"{maps} maps of {dim}, values of {vdim}")
    if ctx.n_tokens != t or block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.shape[0] < ctx.n_seqs:
        raise KernelError("attention_maps: the block table does not fit the step")
    _i32("attention_maps", "row_seq", ctx.row_seq, t)
    _i32("attention_maps", "positions", ctx.positions, t)
    gate_row = _part_of_rows("attention_maps", "gate", gate, n_heads * vdim) if gate is not None else 0
    out = torch.empty((t, n_heads * vdim), dtype=out_dtype, device=q.device)

    def cost():
        keys = pairs = 0
        for s in range(ctx.n_seqs):
            cached, new = int(ctx.seq_ctx[s]), int(ctx.seq_start[s + 1] - ctx.seq_start[s])
            if block > 0:
                pairs += sum((cached + i) % block + 1 for i in range(new))
                keys += min(cached + new, cached % block + new)
            elif window > 0:
                pairs += sum(min(window + keep_first, cached + i + 1) for i in range(new))
                keys += min(cached + new, window + keep_first + new - 1)
            else:
                pairs += new * cached + new * (new + 1) // 2
                keys += cached + new
        return (2.0 * pairs * n_heads * maps * (dim + vdim),
                keys * n_kv_heads * (maps * dim + vdim) * k_cache.element_size() + t * n_heads * (4 * maps * dim + vdim * out.element_size()))
    if waves <= 0:
        reach = min(ctx.max_kv_len, block) if block > 0 else ctx.max_kv_len if window <= 0 else min(ctx.max_kv_len, window + keep_first)
        tiles = max(1, -(-reach // 64))
        waves = 1 if t * n_heads >= ATTENTION_MAPS_FULL else min(8, tiles)
    library.call("bc4g_attention_maps", _ptr(q), n_heads * maps * dim, _ptr(k_cache), _ptr(v_cache), _code(k_cache, "attention_maps"),
                 _ptr(block_table), block_table.stride(0), _ptr(ctx.row_seq), _ptr(ctx.positions), float(lam), 1 if normalize else 0,
                 float(eps), float(factor), _ptr(gate), _code(gate, "attention_maps") if gate is not None else F32, gate_row, int(act),
                 _ptr(out), _code(out, "attention_maps"), t, n_heads, n_kv_heads, maps, dim, vdim, page_tokens, int(window),
                 int(keep_first), float(scale), int(waves), _ptr(sink), _ptr(far[0]) if far else None,
                 _ptr(far[1]) if far else None, int(block), float(cap), _ptr(point), _stream(), cost=cost)
    return out


TALK_MAX_HEADS = 64          # query heads whose weights attention_talk mixes
TALK_MAX_QUERIES = 8192      # heads * (dim rounded up: 64 up to 64, else 256) that a row's queries may take in its LDS
TALK_WORKGROUPS = 512        # a step of fewer rows cuts every row's keys into parts (whole tiles of 64) to bring this many
TALK_MAX_PARTS = 64
TALK_KEPT_BYTES = 1 << 30    # the most a step's first-walk scores may take to be kept for the second walk (else: computed twice)


def attention_talk_takes(n_heads: int, dim: int, vdim: int) -> bool:
    return (0 < n_heads <= TALK_MAX_HEADS and 0 < dim <= HEADS_MAX_DIM and 0 < vdim <= HEADS_MAX_DIM
            and n_heads * (64 if dim <= 64 else 256) <= TALK_MAX_QUERIES)


def attention_talk(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, ctx, out_dtype: torch.dtype,
                   n_heads: int, n_kv_heads: int, dim: int, vdim: int, window: int, scale: float, *,
                   sink: Optional[torch.Tensor] = None, far: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                   talk: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, parts: int = 0,
                   keep_scores: Optional[bool] = None) -> torch.Tensor:
    """Windowed softmax attention whose heads' weights are mixed before they meet the values: q float32 [T, n_heads, dim];
    keys [pages, n_kv_heads, page_tokens, dim], values [pages, n_kv_heads, page_tokens, vdim].  A row at position p sees key
    j <= p with p - j < window (0: every key).  score = q . k * scale - r1 ln(1 + r2 (p - j)) (``far`` = (r1, r2));
    w_g = exp(score_g) / (sum_j exp(score_g) + exp(sink_g)); head h weighs the values of its own key/value head by
    sum_g talk[h, g] w_g (``talk`` float32 [n_heads, n_heads]; none: its own weights) and is multiplied by
    sigmoid(gate[t, h]) (``gate`` [T, n_heads], may be a part of wider rows).  Returns [T, n_heads * vdim].
    ``parts``: into how many parts, a workgroup each, every row's keys are cut (0: chosen here -- one where the rows fill
    the GPU, more where few rows walk long contexts).  ``keep_scores``: whether the first walk's scores are kept in memory
    for the second (None: where they fit TALK_KEPT_BYTES)."""
    _dev("attention_talk", q, k_cache, v_cache, block_table, sink, talk, *(far or ()))
    t = q.shape[0]
    if q.dtype != torch.float32 or tuple(q.shape) != (t, n_heads, dim) or not q.is_contiguous():
        raise KernelError(f"attention_talk: q must be float32 [T, {n_heads}, {dim}], got {q.dtype} {tuple(q.shape)}")
    if not attention_talk_takes(n_heads, dim, vdim):
        raise KernelError(f"attention_talk: {n_heads} heads of {dim} with values of {vdim} are beyond the kernel")
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.dtype != v_cache.dtype:
        raise KernelError("attention_talk: caches must be [pages, heads, page_tokens, size] of one dtype")
    pages, _, page_tokens, _ = k_cache.shape
    if tuple(k_cache.shape[1:]) != (n_kv_heads, page_tokens, dim) or tuple(v_cache.shape) != (pages, n_kv_heads, page_tokens, vdim):
        raise KernelError(f"attention_talk: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit {n_kv_heads} key/value "
                          f"heads, keys of {dim}, values of {vdim}")
    if ctx.n_tokens != t or block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.shape[0] < ctx.n_seqs:
        raise KernelError("attention_talk: the block table does not fit the step")
    _i32("attention_talk", "row_seq", ctx.row_seq, t)
    _i32("attention_talk", "positions", ctx.positions, t)
    _f32("attention_talk", "sink", sink, (n_heads,))
    _f32("attention_talk", "talk", talk, (n_heads, n_heads))
    for v in far or ():
        _f32("attention_talk", "far", v, (n_heads,))
    gate_row = _part_of_rows("attention_talk", "gate", gate, n_heads) if gate is not None else 0
    if gate is not None and gate.shape[0] != t:
        raise KernelError(f"attention_talk: gate has {gate.shape[0]} rows, q {t}")
    out = torch.empty((t, n_heads * vdim), dtype=out_dtype, device=q.device)

    def cost():
        keys = pairs = 0
        for s in range(ctx.n_seqs):
            cached, new = int(ctx.seq_ctx[s]), int(ctx.seq_start[s + 1] - ctx.seq_start[s])
            if window > 0:
                pairs += sum(min(window, cached + i + 1) for i in range(new))
                keys += min(cached + new, window + new - 1)
            else:
                pairs += new * cached + new * (new + 1) // 2
                keys += cached + new
        mixing = n_heads if talk is not None else 0
        return (2.0 * pairs * n_heads * (dim + vdim + mixing),
                keys * n_kv_heads * (dim + vdim) * k_cache.element_size() + t * n_heads * (4 * dim + vdim * out.element_size()))
    if parts <= 0:
        reach = ctx.max_kv_len if window <= 0 else min(ctx.max_kv_len, window)
        parts = max(1, min(-(-reach // 64), TALK_MAX_PARTS, TALK_WORKGROUPS // max(1, t)))
    reach = ctx.max_kv_len if window <= 0 else min(ctx.max_kv_len, window)
    kept_row = 64 * max(1, -(-reach // 64))
    if keep_scores is None:
        keep_scores = 4 * t * n_heads * kept_row <= TALK_KEPT_BYTES
    kept = torch.empty((t, n_heads, kept_row), dtype=torch.float32, device=q.device) if keep_scores else None
    stats = partial = None
    if parts > 1:
        stats = torch.empty((t, parts, n_heads, 2), dtype=torch.float32, device=q.device)
        partial = torch.empty((t, parts, n_heads * vdim), dtype=torch.float32, device=q.device)
    library.call("bc4g_attention_talk", _ptr(q), n_heads * dim, _ptr(k_cache), _ptr(v_cache), _code(k_cache, "attention_talk"),
                 _ptr(block_table), block_table.stride(0), _ptr(ctx.row_seq), _ptr(ctx.positions), _ptr(sink),
                 _ptr(far[0]) if far else None, _ptr(far[1]) if far else None, _ptr(talk), _ptr(gate),
                 _code(gate, "attention_talk") if gate is not None else F32, gate_row, _ptr(out), _code(out, "attention_talk"),
                 t, n_heads, n_kv_heads, dim, vdim, page_tokens, int(window), float(scale), int(parts), _ptr(stats), _ptr(partial),
                 _ptr(kept), kept_row, _stream(), cost=cost)
    return out


# ---- activations and routing of a mixture of experts ------------------------------------------------------------------------

def gelu(z: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """z Phi(z), the exact gelu, element by element; ``out`` may be z itself."""
    _dev("gelu", z, out)
    if not z.is_contiguous():
        raise KernelError("gelu: the input's elements must lie side by side")
    if out is None:
        out = torch.empty_like(z)
    elif out.dtype != z.dtype or out.shape != z.shape or not out.is_contiguous():
        raise KernelError("gelu: out must have the input's dtype and shape")
    total = z.numel()
    library.call("bc4g_gelu", _ptr(z), _ptr(out), _code(z, "gelu"), total, _stream(),
                 cost=lambda: (10.0 * total, 2 * total * z.element_size()))
    return out


MOE_MAX_EXPERTS = 1024


def moe_route(logits: torch.Tensor, experts: int, top: int, groups: int = 1, keep: int = 1,
              correction: Optional[torch.Tensor] = None, want_chosen: bool = False, squash: bool = False,
              normalize: bool = False, factor: float = 1.0):
    """The choice of experts for every row: logits float32 [T, >= experts] (the first ``experts`` columns count; rows may
    be parts of wider rows).  s = softmax(logits); the choice goes by s + correction; only experts of the ``keep`` best of
    ``groups`` equal groups of neighbours (a group counts by its largest choice) can be chosen; the ``top`` largest win.
    ``squash``: s = sigmoid(logits), every expert by itself, instead of the softmax.  ``normalize``: the chosen experts'
    weights are their s divided by the sum of the chosen s (+ 1e-20).  ``factor`` multiplies the weights last.
    Returns weights float32 [T, experts] -- s of the chosen, zero elsewhere -- and, if asked, the chosen int32 [T, top]."""
    _dev("moe_route", correction)
    row = _part_of_rows("moe_route", "logits", logits, experts)
    if logits.dtype != torch.float32:
        raise KernelError(f"moe_route: logits must be float32, got {logits.dtype}")
    _f32("moe_route", "correction", correction, (experts,))
    t = logits.shape[0]
    weights = torch.empty((t, experts), dtype=torch.float32, device=logits.device)
    chosen = torch.empty((t, top), dtype=torch.int32, device=logits.device) if want_chosen else None
    library.call("bc4g_moe_route", _ptr(logits), row, _ptr(correction), _ptr(weights), _ptr(chosen), t, experts, groups, keep, top,
                 1 if squash else 0, 1 if normalize else 0, float(factor), _stream(),
                 cost=lambda: (8.0 * t * experts * (1 + top), 8.0 * t * experts))
    return (weights, chosen) if want_chosen else weights


def routed_gelu(z: torch.Tensor, weights: Optional[torch.Tensor], experts: int, ff: int, shared_ff: int = 0,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """z [T, experts * ff + shared_ff]: every expert's ff units, then the shared unit's.  Returns (``out`` may be z itself)
    weights[t, e] * gelu(z) with the exact gelu for expert e's units -- zero for the experts a row did not choose -- and
    gelu(z) for the shared unit's."""
    _dev("routed_gelu", z, weights, out)
    t = z.shape[0]
    if z.dim() != 2 or z.shape[1] != experts * ff + shared_ff:
        raise KernelError(f"routed_gelu: input must be [T, {experts * ff + shared_ff}], got {tuple(z.shape)}")
    if experts:
        _f32("routed_gelu", "weights", weights, (t, experts))
    if out is None:
        out = torch.empty_like(z)
    elif out.dtype != z.dtype or out.shape != z.shape:
        raise KernelError("routed_gelu: out must have the input's dtype and shape")
    library.call("bc4g_routed_gelu", _ptr(z), _ptr(out), _code(z, "routed_gelu"), _ptr(weights), t, experts, ff, shared_ff, _stream(),
                 cost=lambda: (12.0 * z.numel(), 2 * z.numel() * z.element_size()))
    return out


def routed_glu(gu: torch.Tensor, weights: Optional[torch.Tensor], experts: int, ff: int, limit: float, *, shared_ff: int = 0,
               shared_limit: float = 0.0, shared_logit: Optional[torch.Tensor] = None, slope: float = 1.702) -> torch.Tensor:
    """gu [T, experts * 2 ff + 2 shared_ff]: per expert its ff gates, then its ff ups, and last the shared unit's.  Returns
    [T, experts * ff + shared_ff]: weights[t, e] * g sigmoid(slope g) (u + 1) with g = min(gate, limit),
    u = clamp(up, -limit, limit); the shared unit (its own limit) times sigmoid(shared_logit[t]) (float32 [T, 1], may be a
    part of wider rows)."""
    _dev("routed_glu", gu, weights)
    t = gu.shape[0]
    if gu.dim() != 2 or gu.shape[1] != 2 * (experts * ff + shared_ff) or not gu.is_contiguous():
        raise KernelError(f"routed_glu: input must be [T, {2 * (experts * ff + shared_ff)}], got {tuple(gu.shape)}")
    if experts:
        _f32("routed_glu", "weights", weights, (t, experts))
    shared_row = 0
    if shared_ff:
        if shared_logit is None or shared_logit.dtype != torch.float32 or shared_logit.shape[0] != t:
            raise KernelError("routed_glu: the shared unit needs a float32 gate logit for every row")
        shared_row = _part_of_rows("routed_glu", "shared_logit", shared_logit, 1)
    out = torch.empty((t, experts * ff + shared_ff), dtype=gu.dtype, device=gu.device)
    library.call("bc4g_routed_glu", _ptr(gu), _ptr(out), _code(gu, "routed_glu"), _ptr(weights), _ptr(shared_logit), shared_row,
                 float(limit), float(shared_limit), float(slope), t, experts, ff, shared_ff, _stream(),
                 cost=lambda: (8.0 * out.numel(), 3 * out.numel() * gu.element_size()))
    return out
