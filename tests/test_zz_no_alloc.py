"""The product entry point that allocates nothing (``ns_gemm_wide_bf16_static``, csrc/no_alloc.h), called through ctypes as
a caller outside Python would call it, against ``ns_gemm_wide_bf16`` with a workspace argument: two calls in a row, the
second with a smaller input, so that what the first call left in the library's own array must not show."""

from __future__ import annotations

import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

NS_ERR_SCRATCH_TOO_SMALL = 1003
SCRATCH_FLOATS = 2 * 1024 * 1024


def _lib():
    from nanospec_amd.kernels import build

    lib = build.core()
    lib.ns_gemm_wide_bf16_static.restype = c_int
    lib.ns_gemm_wide_bf16.restype = c_int
    lib.ns_static_scratch_init.restype = c_int
    return lib


def _ptr(t):
    return c_void_p(0 if t is None else t.data_ptr())


def _both(lib, x, w, w2, ksplit, nt, out_f32=False):
    """-> (result of the entry point with a workspace argument, result of the one without), each into a poisoned buffer."""
    m, k = x.shape
    n = w.n
    dtype = torch.float32 if out_f32 else torch.bfloat16
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    gated = w2 is not None
    ws = torch.full(((2 if gated else 1) * ksplit * m * n,), float("nan"), dtype=torch.float32, device=x.device)
    want = torch.full((m, n), 7.0, dtype=dtype, device=x.device)
    got = torch.full((m, n), -7.0, dtype=dtype, device=x.device)
    common = (c_int(m), c_int(n), c_int(k), c_int(x.stride(0)), c_int(n), c_int(1 if gated else 0), c_int(1 if out_f32 else 0),
              c_int(ksplit), c_int(nt))
    rc = lib.ns_gemm_wide_bf16(_ptr(want), _ptr(ws), _ptr(x), _ptr(w.data), _ptr(w2.data if gated else None), *common, c_int(0), stream)
    assert rc == 0
    rc = lib.ns_gemm_wide_bf16_static(_ptr(got), _ptr(x), _ptr(w.data), _ptr(w2.data if gated else None), *common, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return want, got


def test_static_scratch_product_equals_the_workspace_one_on_two_calls_in_a_row():
    from nanospec_amd.kernels import ops

    lib = _lib()
    dev = torch.device("cuda:0")
    assert lib.ns_static_scratch_init() == 0
    gen = torch.Generator(device=dev).manual_seed(5)
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32)
    # first call: 100 rows, 4 ranges of K; second call: fewer rows, a narrower matrix and another number of ranges, so its
    # partial sums lie where the first call's still are
    for m, n, k, ksplit in ((100, 1000, 1024, 4), (37, 328, 640, 5)):
        x = (rnd(m, k) * 0.5).to(torch.bfloat16)
        wp = (rnd(n, k) * 0.05).to(torch.bfloat16)
        w = ops.TiledWeight(wp)
        want, got = _both(lib, x, w, None, ksplit, 1)
        assert torch.equal(want, got)
        ref = x.float() @ wp.float().t()
        assert (got.float() - ref).abs().max() <= 0.02 * ref.abs().max()
    # the gated form (two matrices, 32-bit sums of both in the array) and a 32-bit result, again large then small
    for m, n, k, ksplit in ((64, 704, 512, 4), (17, 176, 384, 3)):
        x = (rnd(m, k) * 0.5).to(torch.bfloat16)
        g, u = (rnd(n, k) * 0.05).to(torch.bfloat16), (rnd(n, k) * 0.05).to(torch.bfloat16)
        want, got = _both(lib, x, ops.TiledWeight(g), ops.TiledWeight(u), ksplit, 1)
        assert torch.equal(want, got)
        want, got = _both(lib, x, ops.TiledWeight(g), None, ksplit, 1, out_f32=True)
        assert torch.equal(want, got)
    # a single range needs no partial sums and is taken at any size
    x = (rnd(20, 256) * 0.5).to(torch.bfloat16)
    want, got = _both(lib, x, ops.TiledWeight((rnd(4096, 256) * 0.05).to(torch.bfloat16)), None, 1, 1)
    assert torch.equal(want, got)


def test_static_scratch_product_refuses_what_its_array_cannot_hold():
    from nanospec_amd.kernels import ops

    lib = _lib()
    dev = torch.device("cuda:0")
    m, n, k, ksplit = 128, 4096, 1024, 8  # 4 Mi partial sums: twice what the array holds
    assert ksplit * m * n > SCRATCH_FLOATS
    x = torch.zeros((m, k), dtype=torch.bfloat16, device=dev)
    w = ops.TiledWeight(torch.zeros((n, k), dtype=torch.bfloat16, device=dev))
    out = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
    rc = lib.ns_gemm_wide_bf16_static(_ptr(out), _ptr(x), _ptr(w.data), _ptr(None), c_int(m), c_int(n), c_int(k), c_int(k), c_int(n),
                                      c_int(0), c_int(0), c_int(ksplit), c_int(1), c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == NS_ERR_SCRATCH_TOO_SMALL
    lib.ns_error_string.restype = ctypes.c_char_p
    assert b"array" in lib.ns_error_string(c_int(rc))
    torch.cuda.synchronize()
