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


def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, :] = float(table[ids[t], :]); ids must already be known to lie in [0, vocab)."""
    _dev("embed_gather", table, ids, out)
    vocab, hidden = table.shape
    n = ids.numel()
    _i32("embed_gather", "ids", ids, n)
    if out is None:
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    elif out.dtype != torch.float32 or tuple(out.shape) != (n, hidden):
        raise KernelError(f"embed_gather: out must be float32 [{n}, {hidden}]")
    library.call("bc4g_embed_gather", _ptr(table), _code(table, "embed_gather"), _ptr(ids), _ptr(out),
                 n, hidden, vocab, _stream(), cost=lambda: (0.0, n * hidden * (table.element_size() + 4)))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None, n_rows: Optional[int] = None) -> torch.Tensor:
    """RMSNorm of rows of the float residual stream x [T, H]; with ``rows`` (int32
    indices, the first n_rows are used) only those rows are normed."""
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
    out = torch.empty((n, hidden), dtype=out_dtype, device=x.device)
    library.call("bc4g_rmsnorm", _ptr(x), _ptr(rows), _ptr(weight), _code(weight, "rmsnorm"), _ptr(out),
                 _code(out, "rmsnorm"), n, hidden, float(eps), _stream(),
                 cost=lambda: (3.0 * n * hidden, n * hidden * (4 + out.element_size()) + hidden * weight.element_size()))
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
