"""The product entry point that allocates nothing (kvcm_gemm_skinny_noalloc), called through ctypes
as a C program would call it, against the package's ordinary split product: the same kernels with
partial sums in a buffer the caller allocated.  Two calls in a row share the library's built-in
array, the second with a smaller input, so stale partial sums of the first would show."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from kvcm_amd import ops as _ops
    _ops.lib()
    return _ops


@pytest.fixture(scope="module")
def clib(ops):
    lib = C.CDLL(ops.library_path())
    vp, i = C.c_void_p, C.c_int
    lib.kvcm_gemm_skinny_noalloc.restype = i
    lib.kvcm_gemm_skinny_noalloc.argtypes = [vp, vp, vp, i, i, i, i, i, i, i, vp]
    lib.kvcm_gemm_skinny_noalloc_capacity.restype = C.c_longlong
    lib.kvcm_gemm_skinny_noalloc_capacity.argtypes = []
    lib.kvcm_hip_last_error.restype = C.c_char_p
    return lib


def _operands(seed, M, N, K):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    return x, w


def _existing(ops, x, w, out_dtype):
    M, K = x.shape
    N = w.shape[0]
    S = ops.skinny_splits(M, N, K)
    assert S > 0
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    scratch = torch.full((max(S, 1) * M * N,), float("nan"), dtype=torch.float32, device=DEV) if S > 1 else None
    keep, ops.LIBRARY_GEMM_MIN_ROWS = ops.LIBRARY_GEMM_MIN_ROWS, 0
    try:
        ops.gemm(x, w, out, scratch=scratch)
    finally:
        ops.LIBRARY_GEMM_MIN_ROWS = keep
    return out, S


def _noalloc(clib, x, w, out_dtype):
    M, K = x.shape
    N = w.shape[0]
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = clib.kvcm_gemm_skinny_noalloc(x.data_ptr(), w.data_ptr(), out.data_ptr(), 1 if out_dtype == torch.bfloat16 else 0,
                                       M, N, K, x.stride(0), w.stride(0), out.stride(0), stream)
    return rc, out


# (M, N, K) pairs: a first call and a smaller second one.  The first of each pair splits K (the
# column tiles alone do not fill the chip); both forms of the kernel: the one whose waves share the
# rows through LDS (widths that are multiples of 64), and the one whose every tile reads them itself.
_PAIRS = [
    ((8, 2048, 2048), (3, 512, 1024)),
    ((64, 2048, 5632), (24, 1024, 512)),
    ((16, 2560, 2048), (1, 2560, 2048)),
    ((8, 2064, 2048), (3, 528, 1024)),
]


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("first,second", _PAIRS)
def test_two_calls_in_a_row_equal_the_ordinary_split_product(ops, clib, first, second, out_dtype):
    splits = []
    for seed, (M, N, K) in enumerate((first, second)):
        x, w = _operands(seed, M, N, K)
        want, S = _existing(ops, x, w, out_dtype)
        splits.append(S)
        rc, got = _noalloc(clib, x, w, out_dtype)
        assert rc == 0, clib.kvcm_hip_last_error().decode()
        torch.cuda.synchronize()
        assert torch.isfinite(want.float()).all()
        # the same kernels add the same numbers in the same order
        assert torch.equal(got, want), (M, N, K, S)
        # and the product is the right one
        ref = x.float().cpu().numpy().astype(np.float64) @ w.float().cpu().numpy().astype(np.float64).T
        tol = 2e-2 * np.abs(ref).max() if out_dtype == torch.bfloat16 else 1e-4 * np.abs(ref).max()
        np.testing.assert_allclose(got.float().cpu().numpy(), ref, atol=tol, rtol=0)
    assert splits[0] > 1, "the first call of a pair is meant to go through the built-in array"


def test_products_beyond_the_built_in_array_are_refused(ops, clib):
    cap = clib.kvcm_gemm_skinny_noalloc_capacity()
    assert cap == 2 << 20
    M, N, K = 512, 2048, 8192
    S = ops.skinny_splits(M, N, K)
    assert S * M * N > cap
    x, w = _operands(5, M, N, K)
    rc, out = _noalloc(clib, x, w, torch.bfloat16)
    torch.cuda.synchronize()
    assert rc != 0
    msg = clib.kvcm_hip_last_error().decode()
    assert "built-in array holds" in msg and str(S * M * N) in msg
    assert torch.isnan(out.float()).all(), "a refused call must launch nothing"
    # shapes the kernel does not take at all are refused the same way
    rc, _ = _noalloc(clib, *_operands(6, 4, 40, 64), torch.bfloat16)
    assert rc != 0 and "unsupported shape" in clib.kvcm_hip_last_error().decode()
