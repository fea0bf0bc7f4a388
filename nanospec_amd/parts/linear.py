"""x @ W^T for the parts: ``LinearWeight`` holds a weight matrix and chooses the kernel by precision and row count.

float32: always the plain tiled kernel with 32-bit fused multiply-adds in a fixed order (the true 32-bit path; no
matrix-core mode of reduced precision is ever used).

bfloat16: decode and short portions (up to ``STREAM_ROWS`` rows) run the hand-written matrix-core kernel that streams
the weights once; it reads them in a layout re-laid at load time (``kernels.ops.TiledWeight``) in which every load
of a wave is one contiguous kilobyte.  17 to 64 rows run a second hand-written kernel on the same layout (x shared
through LDS, K cut into ranges) where it is ahead of the library, and so do products of up to 128 rows that end in the
residual stream (at 65 to 128 rows the library takes two to three times as long for them).  More rows go to the platform's GEMM library on the
plain layout, as the reference's nn.Linear does (model/llama.py:168-171).  32-bit results (logits) always come from the
hand-written kernels, in slices of 64 rows, so that no logit is rounded to bfloat16.  Both layouts are kept in memory unless
``keep_plain=False``.
"""

from __future__ import annotations

import torch

from ..kernels import ops

# Which copies of a bfloat16 weight matrix a model keeps (``DecoderModel.load(..., layouts=)``; parts that say
# ``takes_layouts`` are told at load time): the re-laid one that the streaming kernels read is always there; the plain one,
# which the library's products for many rows read, only with "both".  With "tiled" many rows run in blocks through the
# hand-written kernels: slower prompts, half the memory.
LAYOUTS = ("both", "tiled")


STREAM_ROWS = 16  # up to here the streaming kernel beats the library at the shapes measured
GATED_WIDE_ROWS = 80  # up to here gate and up with the activation go through the 17-to-128-row kernel where the library's layout is kept too
WIDE_HEAD_ROWS = 12  # above this many rows a wide 32-bit product (the head) is faster through the 17-to-64-row kernel
WIDE_MAX_N = 4096  # 17 to 64 rows: the hand-written kernel is ahead of the library for outputs up to this width (and for
#                    32-bit results, which the library does not give); wider products go to the library
LIBRARY_MAX_K = 14336  # the longest inner size over which the library's product has run here, kernel by kernel and inside
#                        captured steps, with every replay checked.  ``library_product`` refuses a longer one: such a product is cut
#                        into slices of its inner size in steps that are launched kernel by kernel, and runs through the
#                        hand-written kernels in captured steps, whichever layouts are kept.
PLAIN_SLICE_K = 8192  # the slices of a product on its way into the residual stream that is cut along its inner size are no
#                       longer than this (where only the re-laid copy is kept the scratch copy is then a slice, not the
#                       matrix, and products are cut from this size on already)
UNTILE_MIN_ROWS = 768  # where only the re-laid copy is kept: from this many rows on the products whose callers allow it
#                        (``plain_copy``: q/k/v, o, gate/up, down) first write their matrices out in plain rows (scratch) and go to
#                        the library; the copy costs what 300 rows of the product cost, and the library is 1.6 to 2 times as
#                        fast as the many-row kernel (measured at the 70B shape).  Callers allow it in steps that are launched
#                        kernel by kernel only: the scratch is as large as the matrix, and every captured step keeps its own.


def library_product(x: torch.Tensor, w_t: torch.Tensor, out: torch.Tensor | None = None, into: torch.Tensor | None = None) -> torch.Tensor:
    """The one door to the platform's GEMM library: x @ w_t (``w_t`` [in, out], usually the transposed view of a matrix
    in plain rows).  ``into``: the product is added to this tensor in place, summed in 32-bit and rounded once; a 32-bit
    ``into`` beside bfloat16 operands keeps the sum in 32-bit.  An inner size beyond ``LIBRARY_MAX_K`` is refused: the
    library chooses other kernels for it, none of which has run here."""
    if x.shape[1] > LIBRARY_MAX_K:
        raise ops.KernelRefused(f"a library product over an inner size of {x.shape[1]} (more than {LIBRARY_MAX_K}) must be cut into slices")
    if into is not None:
        if into.dtype == torch.float32 and x.dtype != torch.float32:
            return torch.addmm(into, x, w_t, out_dtype=torch.float32, out=into)
        return into.addmm_(x, w_t)
    return torch.matmul(x, w_t) if out is None else torch.matmul(x, w_t, out=out)


class IntoResidual:
    """Asks a part to hand its output to the residual stream and the RMS norm after it in the cheapest form its last
    product has, instead of returning a finished tensor:
      * ``kernels.ops.PreNormed``: ``resid += output`` has been done in place and the norm needs no kernel of its own
        (at most 16 rows: the product's epilogue did the sum and the norm's statistics);
      * ``kernels.ops.PartialSums``: the ranges of a product whose K was cut, which the norm kernel adds up as it reads
        them (17 to 128 rows);
      * ``kernels.ops.Added``: ``resid += output`` has been done in place by the product itself (more rows, through
        the library), the norm still has its kernel;
      * a tensor: the output, still to be added by the norm kernel.
    ``next_weight``, ``eps``: that norm's weight and epsilon.  ``x_next`` (like resid), ``ssq`` (float32 [rows,
    ceil(width / 16)]) and ``carry`` (float32, 16 * rows * width): where the results go if they must outlive the block's
    scratch (``outlives``); otherwise scratch is taken."""

    def __init__(self, resid: torch.Tensor, next_weight: torch.Tensor, eps: float, x_next: torch.Tensor | None = None,
                 ssq: torch.Tensor | None = None, carry: torch.Tensor | None = None, outlives: bool = False) -> None:
        self.resid, self.next_weight, self.eps = resid, next_weight, eps
        self.x_next, self.ssq, self.carry, self.outlives = x_next, ssq, carry, outlives


class LinearWeight:
    def __init__(self, w: torch.Tensor, keep_plain: bool = True, tiled: bool = True) -> None:
        """``w``: [out, in] on the GPU in the compute dtype.  ``tiled=False``: the caller streams this matrix with a
        kernel and a layout of its own for few rows, so only the plain layout is kept here.  ``keep_plain=False``: only the
        re-laid copy is kept (see ``LAYOUTS``)."""
        self.n, self.k = w.shape
        self.dtype = w.dtype
        fast = w.dtype == torch.bfloat16 and self.k % 8 == 0
        # (an inner size that the library does not take in one piece needs the hand-written kernels for many rows too)
        self.tiled = ops.TiledWeight(w) if (fast and (tiled or self.k > LIBRARY_MAX_K)) else None
        self.plain = w if (keep_plain or self.tiled is None) else None
        self._plain_t = self.plain.t() if self.plain is not None else None  # the library product's operand, made once

    def links_norms(self, rows: int) -> bool:
        """Whether a product of ``rows`` rows can take a ``PreNormed`` input and can end in the residual stream."""
        return self.tiled is not None and rows <= STREAM_ROWS

    def into_residual(self, x: torch.Tensor, link: IntoResidual, arena=None, plain_copy: bool = False):
        """x @ W^T on its way into the residual stream, in one of the forms ``IntoResidual`` names.  ``plain_copy``: as for
        ``__call__``."""
        m = x.shape[0]
        take = (lambda shape, dtype: arena.take(shape, dtype)) if arena is not None else (lambda shape, dtype: torch.empty(shape, dtype=dtype, device=x.device))
        if self.links_norms(m) and x.dtype == torch.bfloat16 and ops.tiled_takes(x[:1], self.k):
            x_next = link.x_next if link.x_next is not None else take(tuple(link.resid.shape), link.resid.dtype)
            ssq = link.ssq if link.ssq is not None else take((m, -(-self.n // 16)), torch.float32)
            return ops.linear_resid_norm(x, self.tiled, link.resid, link.next_weight, link.eps, x_next=x_next, ssq=ssq)
        if (self.tiled is not None and STREAM_ROWS < m <= ops.WIDE_TALL_ROWS and (self.plain is None or self.n <= WIDE_MAX_N)
                and x.dtype == torch.bfloat16 and ops.tiled_takes(x[:1], self.k)):
            ksplit, nt = ops.wide_plan(self.n, self.k, m)
            need = ksplit * m * self.n
            ws = None
            if ksplit > 1 and link.carry is not None and link.carry.numel() >= need:
                ws = link.carry
            elif ksplit > 1 and not link.outlives:
                ws = take((need,), torch.float32)
            if ws is not None:
                return ops.linear_wide(x, self.tiled, workspace=ws, ksplit=ksplit, nt=nt, defer=True)
        r = link.resid
        # many rows: the library's product takes the stream as its addend, resid = resid + x @ W^T summed in 32-bit and
        # rounded once, so the norm after it reads one tensor instead of two and writes one instead of two
        library = (m > ops.SKINNY_MAX_ROWS and x.dtype == torch.bfloat16 and r.dtype == torch.bfloat16 and r.shape == (m, self.n)
                   and r.is_contiguous())
        have_plain = self._plain_t is not None
        # only the re-laid copy is kept: many rows of a step that is launched kernel by kernel may copy it into plain rows
        can_copy = (not have_plain and plain_copy and self.tiled is not None and m >= UNTILE_MIN_ROWS and ops.tiled_takes(x[:1], self.k))
        if library and (have_plain or can_copy):
            if self.k > (LIBRARY_MAX_K if have_plain else PLAIN_SLICE_K):
                if plain_copy:
                    # a long inner size in slices: the stream in 32-bit takes every slice's product as the library adds it
                    # (32-bit sums, 32-bit addend and result) and is rounded once at the end, as one product would be
                    slices = -(-self.k // PLAIN_SLICE_K)
                    width = -(-self.k // (128 * slices)) * 128
                    acc = take((m, self.n), torch.float32)
                    acc.copy_(r)
                    scratch = None if have_plain else take((self.n, width), self.dtype)
                    for k0 in range(0, self.k, width):
                        k1 = min(self.k, k0 + width)
                        piece = self.plain[:, k0:k1] if have_plain else ops.untile(self.tiled, scratch[:, : k1 - k0], k0, k1)
                        library_product(x[:, k0:k1], piece.t(), into=acc)
                    r.copy_(acc)
                    return ops.Added()
                # (a captured step: the hand-written kernels below)
            else:
                plain_t = self._plain_t if have_plain else ops.untile(self.tiled, take((self.n, self.k), self.dtype)).t()
                library_product(x, plain_t, into=r)
                return ops.Added()
        out = link.x_next if link.x_next is not None else take((m, self.n), x.dtype)
        return self(x, out=out, arena=arena, plain_copy=plain_copy)

    def __call__(self, x, out: torch.Tensor | None = None, out_f32: bool = False, arena=None, plain_copy: bool = False) -> torch.Tensor:
        """``arena``: where the workspace of the 17-to-64-row kernel comes from (``ctx.arena``); without it it is allocated.
        ``x`` may be a ``PreNormed`` where ``links_norms`` holds.  ``plain_copy``: where only the re-laid copy is kept, many
        rows may go to the library through a plain copy of the matrix in scratch (see ``UNTILE_MIN_ROWS``)."""
        if isinstance(x, ops.PreNormed):
            if not self.links_norms(x.shape[0]):
                raise ops.KernelRefused("this product cannot take a pre-normed input (rows, layout or precision)")
            return ops.linear_tiled(x, self.tiled, out=out, out_f32=out_f32)
        if x.dtype != self.dtype:
            raise ops.KernelRefused(f"linear: input is {x.dtype}, the weight {self.dtype}")
        if self.dtype == torch.float32 or self.k % 8 or not ops.tiled_takes(x[:1], self.k):
            return ops.linear_generic(x, self.plain, out=out, out_f32=out_f32)
        m = x.shape[0]
        if self.tiled is not None and WIDE_HEAD_ROWS < m <= STREAM_ROWS and out_f32 and self.n >= 8192:
            return ops.linear_wide(x, self.tiled, out=out, out_f32=True, ksplit=1, nt=1)
        if self.tiled is not None and m <= STREAM_ROWS:
            return ops.linear_tiled(x, self.tiled, out=out, out_f32=out_f32)
        if self.tiled is not None and m <= ops.SKINNY_MAX_ROWS and (out_f32 or self.plain is None or self.n <= WIDE_MAX_N):
            ksplit, nt = ops.wide_plan(self.n, self.k)
            ws = arena.take((ksplit * m * self.n,), torch.float32) if (arena is not None and ksplit > 1) else None
            return ops.linear_wide(x, self.tiled, out=out, out_f32=out_f32, workspace=ws, ksplit=ksplit, nt=nt)
        if self.tiled is not None and m <= ops.WIDE_TALL_ROWS and self.n <= WIDE_MAX_N:
            # 65 to 128 rows of a narrow product (the last layer's down-projection, which no norm inside the layer loop follows)
            ksplit, nt = ops.wide_plan(self.n, self.k, m)
            ws = arena.take((ksplit * m * self.n,), torch.float32) if (arena is not None and ksplit > 1) else None
            return ops.linear_wide(x, self.tiled, out=out, out_f32=out_f32, workspace=ws, ksplit=ksplit, nt=nt)
        if self.plain is not None and (not out_f32 or self.tiled is None) and (self.k <= LIBRARY_MAX_K or self.tiled is None):
            if out_f32:
                return ops.linear_generic(x, self.plain, out=out, out_f32=True)
            return library_product(x, self._plain_t, out=out)
        if out is None:
            out = torch.empty((m, self.n), dtype=torch.float32 if out_f32 else x.dtype, device=x.device)
        if self.plain is None and m >= UNTILE_MIN_ROWS and not out_f32 and plain_copy and self.k <= PLAIN_SLICE_K:  # only the tiled layout is kept, many rows: a plain copy for this one product
            plain = arena.take((self.n, self.k), self.dtype) if arena is not None else torch.empty((self.n, self.k), dtype=self.dtype, device=x.device)
            return library_product(x, ops.untile(self.tiled, plain).t(), out=out)
        if m > ops.WIDE_TALL_ROWS:  # ... fewer: blocks of 128 rows through the hand-written kernel
            ksplit, nt = ops.rows_plan(self.n, self.k, m)
            ws = arena.take((ksplit * m * self.n,), torch.float32) if (arena is not None and ksplit > 1) else None
            return ops.linear_rows(x, self.tiled, out=out, out_f32=out_f32, workspace=ws, ksplit=ksplit, nt=nt)
        ksplit, nt = ops.wide_plan(self.n, self.k)
        ws = arena.take((ksplit * ops.SKINNY_MAX_ROWS * self.n,), torch.float32) if (arena is not None and ksplit > 1) else None
        for s in range(0, m, ops.SKINNY_MAX_ROWS):
            e = min(m, s + ops.SKINNY_MAX_ROWS)
            if e - s <= STREAM_ROWS:
                ops.linear_tiled(x[s:e], self.tiled, out=out[s:e], out_f32=out_f32)
            else:
                ops.linear_wide(x[s:e], self.tiled, out=out[s:e], out_f32=out_f32, workspace=ws, ksplit=ksplit, nt=nt)
        return out


class GatedWeights:
    """Gate and up matrices of a gated feed-forward: silu(x @ Wg^T) * (x @ Wu^T) in one pass over x."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, keep_plain: bool = True) -> None:
        self.inter, self.k = gate.shape
        self.dtype = gate.dtype
        fast = gate.dtype == torch.bfloat16 and self.k % 8 == 0
        self.tiled = (ops.TiledWeight(gate), ops.TiledWeight(up)) if fast else None
        self.stacked = torch.cat([gate, up]) if (keep_plain or not fast) else None  # [2 I, K] for the two-kernel path
        self._stacked_t = self.stacked.t() if self.stacked is not None else None

    def links_norms(self, rows: int) -> bool:
        return self.tiled is not None and rows <= STREAM_ROWS

    def _few_rows(self, x, m: int, out: torch.Tensor) -> torch.Tensor:
        """Up to 16 rows (plain or pre-normed).  From a few rows on, where the number of row tiles deals unevenly to the
        compute units as whole tiles, the kernel that shares x through LDS and takes half tiles is ahead of the one that
        streams a tile per workgroup (8B shape, 896 tiles on 256 units: 37.6 against 39.7 us at 8 rows, 37.4 against 43.8
        at 16); where the tiles deal evenly it is not (1B shape, 512 tiles: 2% of a decode step behind)."""
        tiles, units = -(-self.inter // 16), ops.compute_units(out.device)
        uneven = -(-tiles // units) * units > 1.05 * tiles  # a tile of each matrix per workgroup leaves some units a round short
        if m > ops.GATED_HALF_ROWS and uneven and ops.wide_waves(self.inter, self.k, m, 1, 1, gated=True, units=units)[1]:
            return ops.linear_wide(x, self.tiled[0], w2=self.tiled[1], out=out, ksplit=1, nt=1)
        return ops.linear_tiled(x, self.tiled[0], w2=self.tiled[1], out=out)

    def __call__(self, ctx, x, out: torch.Tensor) -> torch.Tensor:
        m = x.shape[0]
        if isinstance(x, ops.PreNormed):
            if not self.links_norms(m):
                raise ops.KernelRefused("this product cannot take a pre-normed input (rows, layout or precision)")
            return self._few_rows(x, m, out)
        fast = self.tiled is not None and ops.tiled_takes(x[:1], self.k)
        if fast and m <= STREAM_ROWS:
            return self._few_rows(x, m, out)
        # (an inner size that the library does not take in one piece: the hand-written kernels at every number of rows)
        stacked = self.stacked if (self.k <= LIBRARY_MAX_K or not fast) else None
        if fast and stacked is None and self.k <= LIBRARY_MAX_K and m >= UNTILE_MIN_ROWS and not ctx.captured:
            # only the tiled layout is kept, many rows: both matrices in plain rows into scratch, then as with both layouts
            # (not in a captured step: every captured shape would hold a scratch of its own as large as the two matrices)
            stacked = ctx.arena.take((2 * self.inter, self.k), x.dtype)
            ops.untile(self.tiled[0], stacked[: self.inter])
            ops.untile(self.tiled[1], stacked[self.inter :])
            gu = ctx.arena.take((m, 2 * self.inter), x.dtype)
            library_product(x, stacked.t(), out=gu)
            return ops.silu_mul(gu, out=out)
        if fast and stacked is None and m > ops.WIDE_TALL_ROWS:
            # only the tiled layout is kept: blocks of 128 rows through the hand-written kernel, activation in the same pass
            return ops.linear_rows(x, self.tiled[0], w2=self.tiled[1], out=out, ksplit=1, nt=2)
        if fast and (m <= GATED_WIDE_ROWS or stacked is None):
            # 17 to 80 rows: the second hand-written kernel, one range of K, so that the activation is applied in the same
            # pass (measured ahead of the library's product plus the activation kernel: 50 against 60 us at 72 rows of the
            # 8B shape, level at 96).  Beyond 64 rows it holds the sums of both matrices only by half tiles; where only the
            # tiled layout is kept it takes up to 128 rows a pass that way (70B shape: 243 us where two passes of 64 take 331).
            step = ops.WIDE_TALL_ROWS if ops.wide_waves(self.inter, self.k, ops.WIDE_TALL_ROWS, 1, 1, gated=True)[1] else ops.SKINNY_MAX_ROWS
            for s in range(0, m, step):
                e = min(m, s + step)
                ops.linear_wide(x[s:e], self.tiled[0], w2=self.tiled[1], out=out[s:e], ksplit=1, nt=1)
            return out
        gu = ctx.arena.take((m, 2 * self.inter), x.dtype)
        if self.dtype == torch.float32 or self.k % 8:
            ops.linear_generic(x, self.stacked, out=gu)
        else:
            library_product(x, self._stacked_t, out=gu)
        return ops.silu_mul(gu, out=out)
