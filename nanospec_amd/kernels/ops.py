"""Python faces of the HIP kernels.  Each function checks on the host that the operands have the
shapes, strides and types the kernel and its grid assume, then launches on the current stream.

A size a kernel does not take raises ``KernelRefused`` with the reason; nothing is computed
elsewhere instead.  Tensors are torch tensors on the GPU; only their addresses cross into C.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_size_t, c_uint32, c_void_p

import torch

from . import build

F32, BF16 = 0, 1


class KernelRefused(Exception):
    """A kernel was asked for a size or type it does not take."""


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelRefused(f"kernels take float32 or bfloat16 tensors, not {t.dtype}")


def _ptr(t):
    return c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # the handle without building a Stream object
_device_index = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream's handle; asked for at every launch, so by the shortest way that torch offers."""
    if _raw_stream is not None and _device_index is not None:
        return c_void_p(_raw_stream(_device_index()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelRefused("kernels run on GPU tensors only; there is no CPU path")


def _check(code: int, what: str) -> None:
    if code != 0:
        lib = build.core()
        lib.ns_error_string.restype = ctypes.c_char_p
        msg = lib.ns_error_string(c_int(code)).decode()
        raise KernelRefused(f"{what}: {msg} (code {code})")


_units: dict[int, int] = {}


def compute_units(device) -> int:
    """Compute units of the GPU a tensor lives on (256 on an MI355X); launch heuristics count workgroups against it."""
    index = torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if index not in _units:
        _units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _units[index]


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelRefused(f"{name} must be a contiguous int32 tensor")
    return t


# ------------------------------------------------------------------------------------------------ elementwise


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None, scale: float = 1.0) -> torch.Tensor:
    """out[i] = table[ids[i]] (times ``scale``, in 32-bit, rounded once).  ``ids`` int32; the caller has checked 0 <= id < vocab."""
    _gpu(table, ids)
    _i32(ids, "ids")
    n, hidden = ids.numel(), table.shape[1]
    if out is None:
        out = torch.empty((n, hidden), dtype=table.dtype, device=table.device)
    if not table.is_contiguous() or out.shape != (n, hidden) or out.dtype != table.dtype or not out.is_contiguous():
        raise KernelRefused("embed: table and out must be contiguous [*, hidden] of one dtype")
    _check(build.core().ns_embed(_ptr(out), _ptr(table), _ptr(ids), c_int(n), c_int(hidden), c_float(scale), c_int(_dtype_code(table)),
                                 _stream()), "embed")
    return out


def logit_transform(logits: torch.Tensor, scale: float = 1.0, softcap: float = 0.0) -> torch.Tensor:
    """32-bit logits in place: times ``scale``; with ``softcap`` > 0 then softcap * tanh(logit / softcap)."""
    _gpu(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1 or softcap < 0:
        raise KernelRefused("logit_transform takes float32 [rows, vocab] and a cap that is not negative")
    _check(build.core().ns_logit_transform(_ptr(logits), c_int(logits.shape[0]), c_int(logits.shape[1]), c_int(logits.stride(0)),
                                           c_float(scale), c_float(softcap), _stream()), "logit_transform")
    return logits


class PartialSums:
    """A product whose K was cut into ranges that have not been added up yet (``linear_wide(..., defer=True)``):
    ``ws`` holds float32 [ksplit, rows, n].  ``rmsnorm`` adds them while it reads them; ``reduce_partial`` makes the tensor."""

    def __init__(self, ws: torch.Tensor, ksplit: int, rows: int, n: int, dtype: torch.dtype) -> None:
        self.ws, self.ksplit, self.rows, self.n, self.dtype = ws, ksplit, rows, n, dtype
        self.shape = (rows, n)


def reduce_partial(p: PartialSums, out: torch.Tensor | None = None) -> torch.Tensor:
    """The sum of the ranges, in order, rounded to the product's dtype."""
    _gpu(p.ws, out)
    if out is None:
        out = torch.empty((p.rows, p.n), dtype=p.dtype, device=p.ws.device)
    if out.shape != (p.rows, p.n) or out.stride(1) != 1 or out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelRefused("reduce_partial: out has the wrong shape or dtype")
    _check(build.core().ns_wide_reduce(_ptr(out), _ptr(p.ws), c_int(p.rows), c_int(p.n), c_int(out.stride(0)), c_int(p.ksplit),
                                       c_int(1 if out.dtype == torch.float32 else 0), _stream()), "reduce_partial")
    return out


def rmsnorm(weight: torch.Tensor, eps: float, resid: torch.Tensor | None = None, x: "torch.Tensor | PartialSums | None" = None,
            rows: torch.Tensor | None = None, write_resid: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[i] = weight * norm(resid[r] + x[r]) with r = rows[i] (or i).  With ``write_resid`` the sum
    is also stored back into ``resid`` (not with ``rows``).  ``x`` may be a ``PartialSums``."""
    if isinstance(x, PartialSums):
        p, dim = x, weight.numel()
        ok = (weight.dtype == torch.bfloat16 and p.dtype == torch.bfloat16 and p.n == dim and dim % 4 == 0 and dim <= 16384
              and (resid is None or (resid.shape == (p.rows, dim) and resid.is_contiguous() and resid.dtype == weight.dtype)))
        if not ok:
            x = reduce_partial(p)
        else:
            _gpu(weight, resid, rows, p.ws)
            if rows is not None:
                _i32(rows, "rows")
            n = rows.numel() if rows is not None else p.rows
            if out is None:
                out = torch.empty((n, dim), dtype=weight.dtype, device=weight.device)
            if out.shape != (n, dim) or not out.is_contiguous() or out.dtype != weight.dtype:
                raise KernelRefused("rmsnorm: out has the wrong shape")
            _check(build.core().ns_rmsnorm_partial(_ptr(out), _ptr(resid), _ptr(p.ws), c_size_t(p.rows * dim), c_int(p.ksplit), _ptr(weight),
                                                   _ptr(rows), c_int(n), c_int(dim), c_float(eps), c_int(1 if write_resid else 0),
                                                   c_int(_dtype_code(weight)), _stream()), "rmsnorm")
            return out
    src = resid if resid is not None else x
    if src is None:
        raise KernelRefused("rmsnorm needs resid or x")
    _gpu(weight, resid, x, rows)
    dim = weight.numel()
    for t in (resid, x):
        if t is not None and (t.dim() != 2 or t.shape[1] != dim or not t.is_contiguous() or t.dtype != weight.dtype):
            raise KernelRefused(f"rmsnorm: operands must be contiguous [*, {dim}] of the weight's dtype")
    if resid is not None and x is not None and resid.shape != x.shape:
        raise KernelRefused("rmsnorm: resid and x differ in shape")
    if rows is not None:
        _i32(rows, "rows")
    n = rows.numel() if rows is not None else src.shape[0]
    if out is None:
        out = torch.empty((n, dim), dtype=weight.dtype, device=weight.device)
    if out.shape != (n, dim) or not out.is_contiguous() or out.dtype != weight.dtype:
        raise KernelRefused("rmsnorm: out has the wrong shape")
    _check(build.core().ns_rmsnorm(_ptr(out), _ptr(resid), _ptr(x), _ptr(weight), _ptr(rows), c_int(n), c_int(dim), c_float(eps),
                                   c_int(1 if write_resid else 0), c_int(_dtype_code(weight)), _stream()), "rmsnorm")
    return out


def _check_pages(block_table, k_cache, v_cache, kv_heads: int, head_dim: int, dtype, what: str) -> int:
    """What the kernels that write keys and values into pages assume of the pools and the block table.  -> page size.
    (Positions and request indices inside the batch are the batch builder's: a kernel computes
    ``block_table[token_req[t]][position // page]`` without asking whether the table is that wide.)"""
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelRefused(f"{what}: key pages are [pages, kv_heads, page, head_dim], value pages [pages, kv_heads, head_dim, page]")
    page = k_cache.shape[2]
    if (k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, head_dim, page)
            or k_cache.dtype != dtype or v_cache.dtype != dtype or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
        raise KernelRefused(f"{what}: cache pages do not fit heads, head size or dtype")
    _i32(block_table, "block_table")
    if block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelRefused(f"{what}: block_table is int32 [requests, pages] with unit stride along a row")
    return page


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, token_req: torch.Tensor, block_table: torch.Tensor,
                  inv_freq: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, heads: int, kv_heads: int,
                  head_dim: int, rotary_dim: int, write_kv: bool = True, interleaved: bool = False, factor: float = 1.0) -> None:
    """Rotate q in place inside ``qkv`` [N, (heads + 2 kv_heads) * head_dim]; rotate k and write k and v of
    every token into the pages ``block_table[token_req[t], position // page]``.
    k_cache [pages, kv_heads, page, head_dim]; v_cache [pages, kv_heads, head_dim, page].
    ``interleaved``: pair j of the rotary part is channels (2j, 2j + 1) instead of (j, j + rotary_dim / 2); ``factor``
    multiplies cosine and sine."""
    _gpu(qkv, positions, token_req, block_table, inv_freq, k_cache, v_cache)
    n = positions.numel()
    width = (heads + 2 * kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[0] != n or qkv.shape[1] != width or qkv.stride(1) != 1:
        raise KernelRefused(f"rope_kv_write: qkv must be [{n}, {width}]")
    _i32(positions, "positions"), _i32(token_req, "token_req")
    if token_req.numel() != n:
        raise KernelRefused("rope_kv_write: token_req is per token")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(1, rotary_dim // 2):
        raise KernelRefused("rope_kv_write: inv_freq must hold rotary_dim/2 float32 values")
    page = _check_pages(block_table, k_cache, v_cache, kv_heads, head_dim, qkv.dtype, "rope_kv_write")
    _check(build.core().ns_rope_kv_write(_ptr(qkv), c_int(qkv.stride(0)), _ptr(positions), _ptr(token_req), _ptr(block_table),
                                         c_int(block_table.stride(0)), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), c_int(n),
                                         c_int(heads), c_int(kv_heads), c_int(head_dim), c_int(rotary_dim), c_int(1 if interleaved else 0),
                                         c_float(factor), c_int(page), c_int(1 if write_kv else 0), c_int(_dtype_code(qkv)), _stream()),
           "rope_kv_write")


def silu_mul(gu: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[n, i] = silu(gu[n, i]) * gu[n, I + i] for gu [N, 2 I]."""
    _gpu(gu)
    n, two_i = gu.shape
    inter = two_i // 2
    if two_i % 2 or not gu.is_contiguous():
        raise KernelRefused("silu_mul: gu must be contiguous [N, 2 I]")
    if out is None:
        out = torch.empty((n, inter), dtype=gu.dtype, device=gu.device)
    _check(build.core().ns_silu_mul(_ptr(out), _ptr(gu), c_int(n), c_int(inter), c_int(_dtype_code(gu)), _stream()), "silu_mul")
    return out


def fill_u32(t: torch.Tensor, value: int = 0) -> None:
    """Set every 32-bit word of ``t`` (a kernel, so that it may be part of a captured graph)."""
    _gpu(t)
    nbytes = t.numel() * t.element_size()
    if nbytes % 4 or not t.is_contiguous():
        raise KernelRefused("fill_u32: the tensor must be contiguous and a whole number of 32-bit words")
    _check(build.core().ns_fill_u32(_ptr(t), c_uint32(value), c_size_t(nbytes // 4), _stream()), "fill_u32")


def scatter_i32(dst: torch.Tensor, dst_idx: torch.Tensor, src: torch.Tensor, src_idx: torch.Tensor) -> None:
    """dst[dst_idx[i]] = src[src_idx[i]] for int32 tensors on the GPU (indices are trusted: the caller built them)."""
    _gpu(dst, dst_idx, src, src_idx)
    for name, t in (("dst", dst), ("dst_idx", dst_idx), ("src", src), ("src_idx", src_idx)):
        _i32(t, name)
    if dst_idx.numel() != src_idx.numel():
        raise KernelRefused("scatter_i32: one source index per destination index")
    _check(build.core().ns_scatter_i32(_ptr(dst), _ptr(dst_idx), _ptr(src), _ptr(src_idx), c_int(dst_idx.numel()), _stream()), "scatter_i32")


# ------------------------------------------------------------------------------------------------ matrix products


def _check_linear(x, w, out, out_f32):
    _gpu(x, w, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.stride(1) != 1 or not w.is_contiguous() or x.dtype != w.dtype:
        raise KernelRefused(f"linear: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit (w is [out, in], one dtype)")
    m, n = x.shape[0], w.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    if out is None:
        out = torch.empty((m, n), dtype=want, device=x.device)
    if out.shape != (m, n) or out.dtype != want or out.stride(1) != 1:
        raise KernelRefused("linear: out has the wrong shape or dtype")
    return out


def linear_generic(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None, out_f32: bool = False) -> torch.Tensor:
    """x @ w.T with the plain tiled kernel: any sizes, float32 or bfloat16, 32-bit accumulation in a fixed order."""
    out = _check_linear(x, w, out, out_f32)
    m, k = x.shape
    _check(build.core().ns_gemm_generic(_ptr(out), _ptr(x), _ptr(w), c_int(m), c_int(w.shape[0]), c_int(k), c_int(x.stride(0)),
                                        c_int(out.stride(0)), c_int(1 if out_f32 else 0), c_int(_dtype_code(x)), _stream()), "linear_generic")
    return out


SKINNY_MAX_ROWS = 64
WIDE_TALL_ROWS = 128  # ``linear_wide`` with one matrix and one row tile per wave takes this many rows


class TiledWeight:
    """A bfloat16 weight matrix [N, K] re-laid for the streaming matrix-core kernel:
    wt[rt][kt][i][lane = 16 g + r][e] = w[16 rt + r][128 kt + 32 g + 8 i + e], rows padded to a multiple of 16 and
    k to a multiple of 128 with zeros, so that every load of a wave is one contiguous kilobyte."""

    def __init__(self, w: torch.Tensor, row_order: torch.Tensor | None = None) -> None:
        """``row_order``: the rows of ``w`` in the order in which they are laid out (a permutation), for kernels whose
        epilogue wants particular rows together in a tile."""
        if w.dtype != torch.bfloat16 or w.dim() != 2 or not w.is_cuda:
            raise KernelRefused("TiledWeight takes a bfloat16 matrix on the GPU")
        if row_order is not None:
            w = w[row_order.to(w.device)]
        self.n, self.k = w.shape
        n_pad, k_pad = -(-self.n // 16) * 16, -(-self.k // 128) * 128
        if (n_pad, k_pad) != (self.n, self.k):
            wp = torch.zeros((n_pad, k_pad), dtype=w.dtype, device=w.device)
            wp[: self.n, : self.k] = w
        else:
            wp = w
        # (rt, r, kt, g, i, e) -> (rt, kt, i, g, r, e)
        self.data = wp.view(n_pad // 16, 16, k_pad // 128, 4, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous()

    def rows(self, start: int, stop: int) -> "TiledWeight":
        """The sub-matrix of rows [start, stop); both must be multiples of 16 (or stop the last row)."""
        if start % 16 or (stop % 16 and stop != self.n):
            raise KernelRefused("row slices of a tiled weight start and end at multiples of 16")
        out = object.__new__(TiledWeight)
        out.n, out.k = stop - start, self.k
        out.data = self.data[start // 16 : -(-stop // 16)]
        return out


def untile(w: TiledWeight, out: torch.Tensor, k0: int = 0, k1: int | None = None) -> torch.Tensor:
    """Columns ``k0`` to ``k1`` (all by default; ``k0`` a multiple of 128, ``k1`` one or the last column) of the matrix of
    ``w`` in plain rows, into ``out`` [n, k1 - k0] (bfloat16, unit stride along a row): what a library product over many
    rows reads, made for the one product where only the re-laid copy is kept."""
    _gpu(out)
    k1 = w.k if k1 is None else k1
    if (out.dtype != torch.bfloat16 or out.dim() != 2 or out.shape != (w.n, k1 - k0) or out.stride(1) != 1 or out.stride(0) % 8
            or out.data_ptr() % 16 or w.k % 8):
        raise KernelRefused(f"untile: out must be bfloat16 [{w.n}, {k1 - k0}] with rows a multiple of 8 elements apart, 16-byte "
                            f"aligned, and k a multiple of 8")
    if not 0 <= k0 < k1 <= w.k or k0 % 128 or (k1 % 128 and k1 != w.k):
        raise KernelRefused("untile: the columns start at a multiple of 128 and end at one or at the last column")
    _check(build.core().ns_untile_bf16(_ptr(out), _ptr(w.data), c_int(w.n), c_int(w.k), c_int(k0), c_int(k1), c_int(out.stride(0)),
                                       _stream()), "untile")
    return out


def tiled_takes(x: torch.Tensor, k: int, max_rows: int = SKINNY_MAX_ROWS) -> bool:
    return (x.dtype == torch.bfloat16 and x.shape[0] <= max_rows and k % 8 == 0 and x.stride(0) % 8 == 0
            and x.stride(1) == 1 and x.data_ptr() % 16 == 0)


class PreNormed:
    """The input of an RMS norm's consumer when the norm has no kernel of its own: ``x`` = r * weight [rows, dim] in bfloat16
    (r the rows to normalise), and ``ssq`` [rows, parts], float32, whose sum over parts is each row's sum of r^2.  The
    consumer multiplies its sums by rsqrt(sum / dim + eps): y = w * r / rms(r) is linear in 1/rms(r).  Made by
    ``linear_resid_norm``; taken by ``linear_tiled`` and ``linear_qkv_rope`` for at most 16 rows."""

    def __init__(self, x: torch.Tensor, ssq: torch.Tensor, dim: int, eps: float) -> None:
        self.x, self.ssq, self.dim, self.eps = x, ssq, dim, eps
        self.shape, self.dtype = x.shape, x.dtype


class Added:
    """What a part returns instead of its output when it has already added that output to the residual stream in place
    (a library product with the stream as its addend): nothing is left to add and no statistics come with it."""


def _prenorm_args(pre: "PreNormed | None", m: int, what: str):
    if pre is None:
        return c_void_p(None), c_int(0), c_int(0), c_float(0.0)
    if (pre.ssq.dtype != torch.float32 or pre.ssq.dim() != 2 or pre.ssq.shape[0] != m or not pre.ssq.is_contiguous() or m > 16
            or not pre.ssq.is_cuda):
        raise KernelRefused(f"{what}: the sums of squares must be float32 [rows, parts] for at most 16 rows")
    return _ptr(pre.ssq), c_int(pre.ssq.shape[1]), c_int(pre.dim), c_float(pre.eps)


GATED_HALF_ROWS = 4  # up to this many rows the gated product runs half a row tile of each matrix per workgroup (with more,
#                      reading x in twice as many workgroups costs what the even spread gains)


def linear_tiled(x: "torch.Tensor | PreNormed", w: TiledWeight, w2: TiledWeight | None = None, out: torch.Tensor | None = None,
                 out_f32: bool = False, waves: int = 0, halves: bool | None = None) -> torch.Tensor:
    """bfloat16 x @ w.T for at most 64 rows from a tiled weight; with ``w2``: silu(x @ w.T) * (x @ w2.T).  ``x`` may be a
    ``PreNormed`` (at most 16 rows).  ``halves`` (with ``w2``, at most 16 rows): a workgroup takes 8 rows of each matrix
    instead of 16, which spreads a number of row tiles that is no multiple of the compute units evenly; None: by rows."""
    pre = x if isinstance(x, PreNormed) else None
    if pre is not None:
        x = pre.x
    _gpu(x, out)
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k):
        raise KernelRefused(f"linear_tiled takes bfloat16 x [rows <= {SKINNY_MAX_ROWS}, {w.k}] with an inner size that is a "
                            f"multiple of 8; got {tuple(x.shape)} {x.dtype}")
    m = x.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    if out is None:
        out = torch.empty((m, w.n), dtype=want, device=x.device)
    if out.shape != (m, w.n) or out.dtype != want or out.stride(1) != 1:
        raise KernelRefused("linear_tiled: out has the wrong shape or dtype")
    if w2 is not None and (w2.n != w.n or w2.k != w.k):
        raise KernelRefused("linear_tiled: w2 must match w")
    if waves == 0:  # with more than 8 rows eight waves were never behind four at the shapes measured
        waves = 8 if w.k >= 8192 or ((w.n // 16 < 512 or m > 8) and w.k >= 2048) else 4
    if halves is None:  # (with 3 or 4 rows only where whole row tiles would not spread evenly over 256 compute units)
        halves = m <= 2 or (m <= GATED_HALF_ROWS and -(-w.n // 16) % 256 != 0)
    epi = 0 if w2 is None else (4 if halves and m <= 16 and not out_f32 else 1)
    _check(build.core().ns_gemm_tiled_bf16(_ptr(out), _ptr(x), _ptr(w.data), _ptr(w2.data if w2 is not None else None), c_int(m),
                                           c_int(w.n), c_int(w.k), c_int(x.stride(0)), c_int(out.stride(0)),
                                           c_int(epi), c_int(1 if out_f32 else 0), c_int(waves),
                                           *_prenorm_args(pre, m, "linear_tiled"), _stream()),
           "linear_tiled")
    return out


def linear_resid_norm(x: torch.Tensor, w: TiledWeight, resid: torch.Tensor, next_weight: torch.Tensor, eps: float,
                      x_next: torch.Tensor | None = None, ssq: torch.Tensor | None = None, waves: int = 0) -> PreNormed:
    """A block's contribution to the residual stream, for at most 16 rows: resid += x @ w.T in place (the product and
    the sum rounded to bfloat16 in turn, as separate kernels would), and what the RMS norm that follows needs from it:
    -> PreNormed(resid * next_weight, per-workgroup sums of resid^2)."""
    _gpu(x, resid, next_weight, x_next, ssq)
    m = x.shape[0]
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k) or m > 16:
        raise KernelRefused(f"linear_resid_norm takes at most 16 bfloat16 rows of {w.k} values; got {tuple(x.shape)} {x.dtype}")
    if resid.shape != (m, w.n) or resid.dtype != torch.bfloat16 or resid.stride(1) != 1:
        raise KernelRefused("linear_resid_norm: resid must be bfloat16 [rows, out features]")
    if next_weight.shape != (w.n,) or next_weight.dtype != torch.bfloat16 or not next_weight.is_contiguous():
        raise KernelRefused("linear_resid_norm: the next norm's weight must be bfloat16 [out features]")
    parts = -(-w.n // 16)
    if x_next is None:
        x_next = torch.empty_like(resid)
    if ssq is None:
        ssq = torch.empty((m, parts), dtype=torch.float32, device=x.device)
    if (x_next.shape != resid.shape or x_next.dtype != resid.dtype or x_next.stride() != resid.stride()
            or ssq.shape != (m, parts) or ssq.dtype != torch.float32 or not ssq.is_contiguous()):
        raise KernelRefused("linear_resid_norm: x_next must be laid out like resid, ssq float32 [rows, ceil(out features / 16)]")
    if waves == 0:
        waves = 8 if w.k >= 8192 or (w.n // 16 < 512 and w.k >= 2048) else 4
    _check(build.core().ns_gemm_resid_norm_bf16(_ptr(resid), _ptr(x_next), _ptr(ssq), _ptr(next_weight), _ptr(x), _ptr(w.data),
                                                c_int(m), c_int(w.n), c_int(w.k), c_int(x.stride(0)), c_int(resid.stride(0)),
                                                c_int(waves), _stream()), "linear_resid_norm")
    return PreNormed(x_next, ssq, w.n, eps)


def _wide_cost(tiles: int, per_group: int, ksplit: int, k_tiles: int, units: int) -> int:
    """What the busiest compute unit streams, in row tiles times k tiles: a product of few rows takes as long as that."""
    groups = -(-tiles // per_group)
    return -(-groups * ksplit // units) * per_group * -(-k_tiles // ksplit)


def wide_plan(n: int, k: int, rows: int = SKINNY_MAX_ROWS, units: int | None = None) -> tuple[int, int]:
    """(ranges K is cut into, 16-row tiles per wave) of ``linear_wide``: two tiles per wave when there are rows enough
    (and at most 64 rows of x), then as many ranges as give every compute unit about one workgroup, with at least four k
    tiles of 128 per range (more, shorter ranges were measured slower once the kernel that joins them is counted: 37 against
    31 us for the down-projection of the 8B shape at 64 rows with 10 and with 4 ranges).  With one tile per wave and up to
    64 rows a workgroup may have three waves instead of four (``wide_waves``); the ranges are chosen for whichever of the
    two leaves the busiest compute unit the least to stream.  ``units``: the GPU's compute units (the current device's by
    default)."""
    units = units or compute_units(torch.cuda.current_device())
    nt = 2 if n >= 8192 and rows <= SKINNY_MAX_ROWS else 1
    k_tiles = -(-k // 128)
    most = max(1, min(16, k_tiles // 4))
    ranges = lambda per_group: max(1, min(most, round(units / -(-n // (16 * per_group)))))
    if nt != 1 or rows > SKINNY_MAX_ROWS:
        return ranges(4 * nt), nt
    tiles = -(-n // 16)
    four, three = ranges(4), ranges(3)
    return (three if _wide_cost(tiles, 3, three, k_tiles, units) < _wide_cost(tiles, 4, four, k_tiles, units) else four), nt


def wide_waves(n: int, k: int, rows: int, ksplit: int, nt: int, gated: bool = False, units: int | None = None) -> tuple[int, bool]:
    """(waves per workgroup, by half tiles) of ``linear_wide`` for a product cut as given: what deals the row tiles most
    evenly to the compute units.  One matrix, one tile per wave, up to 64 rows: three waves instead of four where that
    leaves the busiest unit less.  Gate and up in one range: four waves of a whole tile of each (8 half tiles a workgroup),
    seven or four waves of half a tile of each (7 or 4 a workgroup); at the 8B shape 1,792 half tiles are 7 for each of 256
    units instead of 8 for each of 224 (42 against 51 us at 64 rows; the 1B shape's 1,024 as 4 for each: 17 against 25 us)."""
    units = units or compute_units(torch.cuda.current_device())
    if nt != 1 or (rows > SKINNY_MAX_ROWS and not gated):
        return 4, False
    tiles, k_tiles = -(-n // 16), -(-k // 128)
    if gated:
        if rows > SKINNY_MAX_ROWS:  # 65 to 128 rows: only half tiles hold the sums of both matrices
            return (7 if -(-(-(-2 * tiles // 7)) // units) * 7 <= -(-(-(-2 * tiles // 4)) // units) * 4 else 4), ksplit == 1
        if ksplit != 1 or -(-tiles // 4) >= units:  # (whole tiles fill the GPU: measured level or ahead, 163 against 166 us at the 70B shape)
            return 4, False
        options = [(-(-(-(-tiles // 4)) // units) * 8, 4, False), (-(-(-(-2 * tiles // 7)) // units) * 7, 7, True),
                   (-(-(-(-2 * tiles // 4)) // units) * 4, 4, True)]
        _, waves, halves = min(options, key=lambda o: o[0])  # (the first of equals: the fewest workgroups, each reads x)
        return waves, halves
    three = _wide_cost(tiles, 3, ksplit, k_tiles, units) < _wide_cost(tiles, 4, ksplit, k_tiles, units)
    return (3 if three else 4), False


def linear_wide(x: "torch.Tensor | PreNormed", w: TiledWeight, w2: TiledWeight | None = None, out: torch.Tensor | None = None,
                out_f32: bool = False, workspace: torch.Tensor | None = None, ksplit: int = 0, nt: int = 0, defer: bool = False,
                waves: int = 0, halves: bool | None = None):
    """bfloat16 x @ w.T for up to 64 rows from a tiled weight (up to 128 with ``nt=1`` and no ``w2``), with the tile of x
    shared through LDS by the four waves of
    a workgroup and K cut into ``ksplit`` ranges that a second kernel adds up; with ``w2``: silu(x @ w.T) * (x @ w2.T).
    ``workspace``: float32, (2 if w2 else 1) * ksplit * rows * w.n values (none for a single range).  ``defer`` (not with
    ``w2``): with more than one range the second kernel is left out and a ``PartialSums`` over the workspace comes back.
    ``waves``, ``halves``: waves per workgroup and whether gate and up go by half tiles (``wide_waves`` by default).
    ``x`` may be a ``PreNormed`` (at most 16 rows, one range)."""
    pre = x if isinstance(x, PreNormed) else None
    if pre is not None:
        x = pre.x
    _gpu(x, out, workspace)
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k, WIDE_TALL_ROWS):
        raise KernelRefused(f"linear_wide takes bfloat16 x [rows <= {WIDE_TALL_ROWS}, {w.k}] with an inner size that is a "
                            f"multiple of 8; got {tuple(x.shape)} {x.dtype}")
    m = x.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    plan = wide_plan(w.n, w.k, m)
    ksplit, nt = ksplit or plan[0], nt or plan[1]
    if not waves:
        waves, dealt_halves = wide_waves(w.n, w.k, m, ksplit, nt, gated=w2 is not None)
        halves = dealt_halves if halves is None else halves
    halves = bool(halves)
    if m > SKINNY_MAX_ROWS and ((w2 is not None and not halves) or nt != 1):
        raise KernelRefused(f"linear_wide takes more than {SKINNY_MAX_ROWS} rows only with one row tile per wave, and two matrices only by half tiles")
    defer = defer and ksplit > 1 and w2 is None and not out_f32
    if out is None and not defer:
        out = torch.empty((m, w.n), dtype=want, device=x.device)
    if not defer and (out.shape != (m, w.n) or out.dtype != want or out.stride(1) != 1):
        raise KernelRefused("linear_wide: out has the wrong shape or dtype")
    if w2 is not None and (w2.n != w.n or w2.k != w.k or out_f32):
        raise KernelRefused("linear_wide: w2 must match w and the gated result is bfloat16")
    need = (2 if w2 is not None else 1) * ksplit * m * w.n if ksplit > 1 else 0  # a single range writes the result itself
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.float32, device=x.device)
    if need and (workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous()):
        raise KernelRefused("linear_wide: workspace too small")
    if pre is not None and (ksplit != 1 or defer):
        raise KernelRefused("linear_wide: a pre-normed input goes with one range of K")
    if halves and (w2 is None or ksplit != 1 or nt != 1 or waves not in (4, 7)):
        raise KernelRefused("linear_wide: half tiles go with two matrices, one range, one tile per wave, 4 or 7 waves")
    if not halves and waves != 4 and not (waves == 3 and w2 is None and nt == 1 and m <= SKINNY_MAX_ROWS):
        raise KernelRefused("linear_wide: workgroups of 4 waves, or of 3 for one matrix with one tile per wave and up to 64 rows")
    _check(build.core().ns_gemm_wide_dealt_bf16(_ptr(None if defer else out), _ptr(workspace if need else None), _ptr(x), _ptr(w.data),
                                                _ptr(w2.data if w2 is not None else None), c_int(m), c_int(w.n), c_int(w.k), c_int(x.stride(0)),
                                                c_int(w.n if defer else out.stride(0)), c_int(1 if w2 is not None else 0),
                                                c_int(1 if out_f32 else 0), c_int(ksplit), c_int(nt), c_int(1 if defer else 0),
                                                c_int(waves), c_int(1 if halves else 0), *_prenorm_args(pre, m, "linear_wide"), _stream()),
           "linear_wide")
    return PartialSums(workspace, ksplit, m, w.n, x.dtype) if defer else out


def rows_plan(n: int, k: int, rows: int, gated: bool = False, units: int | None = None) -> tuple[int, int]:
    """(ranges K is cut into, 16-row tiles per wave) of ``linear_rows``: the most tiles per wave, then ranges of K until
    the workgroups fill the GPU, with at least eight k tiles of 128 per range."""
    units = units or compute_units(torch.cuda.current_device())
    nt = 2 if gated else 4
    groups = -(-n // (64 * nt)) * -(-rows // 128)
    k_tiles = -(-k // 128)
    return max(1, min(16, k_tiles // 8, units // groups)), nt


def linear_rows(x: torch.Tensor, w: TiledWeight, w2: TiledWeight | None = None, out: torch.Tensor | None = None,
                out_f32: bool = False, workspace: torch.Tensor | None = None, ksplit: int = 0, nt: int = 0):
    """bfloat16 x @ w.T for any number of rows from a tiled weight: the kernel of ``linear_wide`` over blocks of 128 rows,
    with ``nt`` (2 or 4; 1 or 2 with ``w2``) row tiles of the weight per wave.  For models that keep the tiled layout only:
    the platform's library is twice as fast where the plain layout is there for it.  Arguments as ``linear_wide``."""
    _gpu(x, out, workspace)
    if x.dim() != 2 or x.shape[1] != w.k or not tiled_takes(x, w.k, x.shape[0]):
        raise KernelRefused(f"linear_rows takes bfloat16 x [rows, {w.k}] with an inner size that is a multiple of 8; got "
                            f"{tuple(x.shape)} {x.dtype}")
    m = x.shape[0]
    want = torch.float32 if out_f32 else x.dtype
    plan = rows_plan(w.n, w.k, m, w2 is not None)
    ksplit, nt = ksplit or plan[0], nt or plan[1]
    if out is None:
        out = torch.empty((m, w.n), dtype=want, device=x.device)
    if out.shape != (m, w.n) or out.dtype != want or out.stride(1) != 1:
        raise KernelRefused("linear_rows: out has the wrong shape or dtype")
    if w2 is not None and (w2.n != w.n or w2.k != w.k or out_f32):
        raise KernelRefused("linear_rows: w2 must match w and the gated result is bfloat16")
    need = (2 if w2 is not None else 1) * ksplit * m * w.n if ksplit > 1 else 0
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.float32, device=x.device)
    if need and (workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous()):
        raise KernelRefused("linear_rows: workspace too small")
    _check(build.core().ns_gemm_rows_bf16(_ptr(out), _ptr(workspace if need else None), _ptr(x), _ptr(w.data),
                                          _ptr(w2.data if w2 is not None else None), c_int(m), c_int(w.n), c_int(w.k), c_int(x.stride(0)),
                                          c_int(out.stride(0)), c_int(1 if w2 is not None else 0),
                                          c_int(1 if out_f32 else 0), c_int(ksplit), c_int(nt), c_int(0), _stream()),
           "linear_rows")
    return out


def qkv_rope_row_order(heads: int, kv_heads: int, head_dim: int, rotary_dim: int, interleaved: bool = False) -> torch.Tensor:
    """The row order of a stacked [q; k; v] matrix for ``linear_qkv_rope``: per head 16-row tiles; in the rotary part of a
    q or k head a tile holds the first channels of 8 rotary pairs and then their second channels (pair j is channels j and
    j + rotary_dim/2, or 2j and 2j + 1 with ``interleaved``), elsewhere 16 consecutive channels."""
    order = []
    half = rotary_dim // 2
    first, second = ((lambda j: 2 * j), (lambda j: 2 * j + 1)) if interleaved else ((lambda j: j), (lambda j: j + half))
    for g in range(heads + 2 * kv_heads):
        base = g * head_dim
        rot = rotary_dim if g < heads + kv_heads else 0
        for jt in range(rot // 16):
            order += [base + first(jt * 8 + e) for e in range(8)] + [base + second(jt * 8 + e) for e in range(8)]
        for d0 in range(rot, head_dim, 16):
            order += [base + d0 + e for e in range(16)]
    return torch.tensor(order, dtype=torch.int64)


def qkv_rope_takes(x: torch.Tensor, head_dim: int, rotary_dim: int) -> bool:
    return x.dtype == torch.bfloat16 and x.shape[0] <= 16 and head_dim % 16 == 0 and rotary_dim % 16 == 0


def linear_qkv_rope(x: "torch.Tensor | PreNormed", w: TiledWeight, q_out: torch.Tensor, positions, token_req, block_table, inv_freq,
                    k_cache, v_cache, heads: int, kv_heads: int, head_dim: int, rotary_dim: int, write_kv: bool = True,
                    waves: int = 0, interleaved: bool = False, factor: float = 1.0) -> None:
    """The stacked q/k/v product of at most 16 tokens with rotation and cache write fused into its epilogue: q goes rotated
    into ``q_out`` [M, >= heads * head_dim], k rotated into its K page slot, v into the transposed V page.  ``w`` is the
    stacked matrix tiled in ``qkv_rope_row_order`` (of the same ``interleaved``).  ``x`` may be a ``PreNormed``."""
    pre = x if isinstance(x, PreNormed) else None
    if pre is not None:
        x = pre.x
    _gpu(x, q_out, positions, token_req, block_table, inv_freq, k_cache, v_cache)
    m = x.shape[0]
    if not (tiled_takes(x, w.k) and qkv_rope_takes(x, head_dim, rotary_dim)) or x.shape[1] != w.k:
        raise KernelRefused("linear_qkv_rope takes at most 16 bfloat16 rows and head and rotary sizes that are multiples of 16")
    if w.n != (heads + 2 * kv_heads) * head_dim:
        raise KernelRefused("linear_qkv_rope: the weight does not hold heads + 2 kv_heads heads")
    if q_out.dtype != torch.bfloat16 or q_out.shape[0] != m or q_out.shape[1] < heads * head_dim or q_out.stride(1) != 1:
        raise KernelRefused("linear_qkv_rope: q_out must be bfloat16 [rows, >= heads * head_dim]")
    _i32(positions, "positions"), _i32(token_req, "token_req")
    page = _check_pages(block_table, k_cache, v_cache, kv_heads, head_dim, torch.bfloat16, "linear_qkv_rope")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(1, rotary_dim // 2) or positions.numel() != m or token_req.numel() != m:
        raise KernelRefused("linear_qkv_rope: positions, token_req are per row; inv_freq holds rotary_dim / 2 float32 values")
    if waves == 0:
        waves = 8 if w.k >= 2048 else 4
    _check(build.core().ns_gemm_qkv_rope_bf16(_ptr(q_out), _ptr(x), _ptr(w.data), c_int(m), c_int(w.k), c_int(x.stride(0)),
                                              c_int(q_out.stride(0)), _ptr(positions), _ptr(token_req), _ptr(block_table),
                                              c_int(block_table.stride(0)), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), c_int(heads),
                                              c_int(kv_heads), c_int(head_dim), c_int(rotary_dim), c_int(1 if interleaved else 0),
                                              c_float(factor), c_int(page),
                                              c_int(1 if write_kv else 0), c_int(waves), *_prenorm_args(pre, m, "linear_qkv_rope"),
                                              _stream()), "linear_qkv_rope")


def rope_kv_from_partial(p: PartialSums, q_out: torch.Tensor, positions, token_req, block_table, inv_freq, k_cache, v_cache,
                         heads: int, kv_heads: int, head_dim: int, rotary_dim: int, write_kv: bool = True, interleaved: bool = False,
                         factor: float = 1.0) -> None:
    """Rotation and cache write for a stacked q/k/v product whose K ranges are not added up yet (``linear_wide(...,
    defer=True)`` from a weight tiled in ``qkv_rope_row_order`` of the same ``interleaved``): one pass adds the ranges, rotates, and writes q into
    ``q_out`` [rows, >= heads * head_dim], k into its K page slot and v into the transposed V page."""
    _gpu(p.ws, q_out, positions, token_req, block_table, inv_freq, k_cache, v_cache)
    m = p.rows
    if p.dtype != torch.bfloat16 or head_dim % 16 or rotary_dim % 16 or p.n != (heads + 2 * kv_heads) * head_dim:
        raise KernelRefused("rope_kv_from_partial takes a bfloat16 product of heads + 2 kv_heads heads, head and rotary sizes multiples of 16")
    if q_out.dtype != torch.bfloat16 or q_out.shape[0] != m or q_out.shape[1] < heads * head_dim or q_out.stride(1) != 1:
        raise KernelRefused("rope_kv_from_partial: q_out must be bfloat16 [rows, >= heads * head_dim]")
    _i32(positions, "positions"), _i32(token_req, "token_req")
    page = _check_pages(block_table, k_cache, v_cache, kv_heads, head_dim, torch.bfloat16, "rope_kv_from_partial")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(1, rotary_dim // 2) or positions.numel() != m or token_req.numel() != m:
        raise KernelRefused("rope_kv_from_partial: positions, token_req are per row; inv_freq holds rotary_dim / 2 float32 values")
    if p.ws.dtype != torch.float32 or p.ws.numel() < p.ksplit * m * p.n:
        raise KernelRefused("rope_kv_from_partial: the partial sums are too few")
    _check(build.core().ns_rope_kv_partial(_ptr(q_out), c_int(q_out.stride(0)), _ptr(p.ws), c_int(p.ksplit), c_int(m), c_int(p.n),
                                           _ptr(positions), _ptr(token_req), _ptr(block_table), c_int(block_table.stride(0)),
                                           _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), c_int(heads), c_int(kv_heads), c_int(head_dim),
                                           c_int(rotary_dim), c_int(1 if interleaved else 0), c_float(factor), c_int(page),
                                           c_int(1 if write_kv else 0), _stream()), "rope_kv_from_partial")


# ------------------------------------------------------------------------------------------------ attention


def _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim):
    _gpu(q, out, k_cache, v_cache)
    page = k_cache.shape[2] if k_cache.dim() == 4 else 0
    if (k_cache.dim() != 4 or k_cache.shape[1:] != (kv_heads, page, head_dim) or v_cache.shape != (k_cache.shape[0], kv_heads, head_dim, page)
            or not k_cache.is_contiguous() or not v_cache.is_contiguous() or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype):
        raise KernelRefused("attention: cache pages do not fit heads, head size or dtype")
    if q.stride(1) != 1 or q.shape[1] < heads * head_dim:
        raise KernelRefused("attention: q rows must hold heads * head_dim contiguous values")
    if out.shape != (q.shape[0], heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelRefused("attention: out must be contiguous [tokens, heads * head_dim]")
    if heads % kv_heads:
        raise KernelRefused(f"attention: {heads} heads are not a multiple of {kv_heads} key/value heads")
    return page


def attention_generic(q, out, k_cache, v_cache, token_req, positions, block_table, heads: int, kv_heads: int, head_dim: int,
                      scale: float, window: int = 0) -> torch.Tensor:
    """Attention of every token's query over its request's pages; any head size up to 256, either dtype."""
    page = _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim)
    _i32(token_req, "token_req"), _i32(positions, "positions"), _i32(block_table, "block_table")
    if head_dim > 256:
        raise KernelRefused(f"attention_generic takes head sizes up to 256, not {head_dim}")
    n = q.shape[0]
    _check(build.core().ns_attn_generic(_ptr(out), _ptr(q), c_int(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(token_req),
                                        _ptr(positions), _ptr(block_table), c_int(block_table.stride(0)), c_int(n), c_int(heads),
                                        c_int(kv_heads), c_int(head_dim), c_int(page), c_float(scale), c_int(window),
                                        c_int(_dtype_code(q)), _stream()), "attention_generic")
    return out


def mfma_attention_takes(dtype, head_dim: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and page_size >= 4 and page_size & (page_size - 1) == 0


TILE_INTS = 8  # ints per attention tile descriptor: request, first token, first row, tokens, keys, 0, 0, 0


def attention_mfma(q, out, k_cache, v_cache, tiles, block_table, heads: int, kv_heads: int, head_dim: int, scale: float,
                   window: int = 0, hp: int = 1, splits: int = 1,
                   workspace: tuple[torch.Tensor, torch.Tensor] | None = None, qt: int = 1, coop: bool = False,
                   short_offsets: bool = True) -> torch.Tensor:
    """bfloat16 attention on the matrix cores for the tiles described in ``tiles`` (int32 [n_tiles, 8]: request, first
    token of the tile among the request's tokens of this step, row of the request's first token in ``q``, tokens of the
    request in this step, keys after this step, three zeros).  ``hp`` heads of a group times 16/hp tokens make a tile;
    with ``qt`` = 2 (only with hp = 1) a tile is 32 tokens.  ``splits`` > 1 cuts the keys of every tile
    into that many ranges (at most 64) and needs ``workspace`` = (part_o, part_ml) float32 tensors.  With ``coop`` the four
    waves of a workgroup share each tile and range (for decode, where a wave's chain of loads is what takes the time); with
    ``qt`` = 2 it asks for workgroups of one set of four waves instead of two (for long rows of keys).  A pool within
    4 GiB is addressed with 32-bit offsets from its start; ``short_offsets`` = False keeps every address 64 bits wide
    whatever the pool's size (the form that larger pools take)."""
    page = _check_attn(q, out, k_cache, v_cache, heads, kv_heads, head_dim)
    if not mfma_attention_takes(q.dtype, head_dim, page):
        raise KernelRefused(f"attention_mfma takes bfloat16, head sizes that are multiples of 16 up to 256 and page sizes that are "
                            f"powers of two from 4; got {q.dtype}, head size {head_dim}, page {page}")
    _gpu(tiles, block_table)
    _i32(tiles, "tiles"), _i32(block_table, "block_table")
    if tiles.dim() != 2 or tiles.shape[1] != TILE_INTS or tiles.data_ptr() % 16:
        raise KernelRefused(f"attention_mfma: tiles must be int32 [n_tiles, {TILE_INTS}], 16-byte aligned")
    if hp not in (1, 2, 4, 8, 16):
        raise KernelRefused("attention_mfma: hp is a power of two up to 16")
    if qt != 1 and not (qt == 2 and hp == 1):
        raise KernelRefused("attention_mfma: 32-token tiles (qt = 2) go with hp = 1")
    n_tiles = tiles.shape[0]
    po = pm = None
    if splits > 1:
        if workspace is None or splits > 64:
            raise KernelRefused("attention_mfma: 2 to 64 key ranges are taken, with a workspace")
        po, pm = workspace
        cols = n_tiles * (qt * 16 // hp) * heads
        if po.dtype != torch.float32 or pm.dtype != torch.float32 or po.numel() < cols * splits * head_dim or pm.numel() < cols * splits * 2:
            raise KernelRefused("attention_mfma: workspace too small")
    lib = build.attn(head_dim, page)
    _check(lib.ns_attn_mfma(_ptr(out), _ptr(po), _ptr(pm), _ptr(q), c_int(q.stride(0)), _ptr(k_cache), _ptr(v_cache), _ptr(tiles),
                            _ptr(block_table), c_int(block_table.stride(0)), c_int(n_tiles), c_int(heads), c_int(kv_heads),
                            c_int(page), c_int(hp), c_int(splits), c_int(window), c_float(scale), c_int(qt), c_int(1 if coop else 0),
                            ctypes.c_long(k_cache.shape[0] if short_offsets else 0), _stream()),
           "attention_mfma")
    return out


def attention_prompt_form(head_dim: int, page_size: int) -> int:
    """Which kernel of the library for this head and page size takes prompt portions in tiles of 32 tokens: 32 the one
    on the 32x32 matrix instruction with loads straight into LDS, 16 the one on the 16x16 instruction with keys shared
    through LDS, 0 the one without sharing."""
    return int(build.attn(head_dim, page_size).ns_attn_prompt_form())


# ------------------------------------------------------------------------------------------------ sampling


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor, top_k: torch.Tensor | None = None,
           top_p: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """Per row of float32 ``logits``: arg-max when temperature is 0, else a draw by inverse CDF with the row's uniform
    number.  -> int32 [3, rows]: row 0 the tokens, row 1 the bits of the float32 log-probability of the token under the
    raw logits, row 2 the bits of its float32 log-probability under the processed distribution (0 for arg-max rows)."""
    _gpu(logits, temperature, uniform, top_k, top_p, out)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelRefused("sample: logits must be float32 [rows, vocab]")
    rows, vocab = logits.shape
    for name, t, dt in (("temperature", temperature, torch.float32), ("uniform", uniform, torch.float32),
                        ("top_k", top_k, torch.int32), ("top_p", top_p, torch.float32)):
        if t is not None and (t.dtype != dt or t.numel() != rows or not t.is_contiguous()):
            raise KernelRefused(f"sample: {name} must hold one {dt} per row")
    if out is None:
        out = torch.empty((3, rows), dtype=torch.int32, device=logits.device)
    if out.dtype != torch.int32 or out.shape != (3, rows) or not out.is_contiguous():
        raise KernelRefused("sample: out must be a contiguous int32 [3, rows]")
    _check(build.core().ns_sample(_ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _ptr(logits), c_int(logits.stride(0)), _ptr(temperature),
                                  _ptr(top_k), _ptr(top_p), _ptr(uniform), c_int(rows), c_int(vocab), _stream()), "sample")
    return out


def unpack_sample(packed: torch.Tensor):
    """int32 [3, rows] of ``sample`` -> (tokens int32, log-probabilities float32, processed log-probabilities float32)."""
    return packed[0], packed[1].view(torch.float32), packed[2].view(torch.float32)


# ------------------------------------------------------------------------------------------------ graphs


class Graph:
    """A captured stream of launches.  ``with Graph.capture(stream) as g: ...`` then ``g.launch()``."""

    def __init__(self, stream: torch.cuda.Stream) -> None:
        self.stream, self._exec = stream, None

    def __enter__(self):
        self._ctx = torch.cuda.stream(self.stream)
        self._ctx.__enter__()
        _check(build.core().ns_graph_begin(c_void_p(self.stream.cuda_stream)), "graph capture begin")
        return self

    def __exit__(self, et, ev, tb):
        handle = c_void_p()
        code = build.core().ns_graph_end(c_void_p(self.stream.cuda_stream), ctypes.byref(handle))
        self._ctx.__exit__(et, ev, tb)
        if et is None:
            _check(code, "graph capture end")
            self._exec = handle
        return False

    def launch(self) -> None:
        _check(build.core().ns_graph_launch(self._exec, c_void_p(self.stream.cuda_stream)), "graph launch")

    def __del__(self):
        if getattr(self, "_exec", None):
            try:
                build.core().ns_graph_destroy(self._exec)
            except Exception:
                pass
