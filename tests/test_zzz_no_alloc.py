"""nmtg_gemm_static — the GEMM entry point that allocates nothing — against nmtg_gemm with a caller-provided
workspace: same kernels, same reduction order, so identical bits. Two calls in a row share the library's scratch
array; the second is smaller, so stale partial sums of the first lie behind it."""
import ctypes

import pytest
import torch

from nmtgminor_amd import _lib as L
from nmtgminor_amd.native.linear_gemm import gemm

pytestmark = pytest.mark.gpu


def gemm_static(a, b, trans_a, trans_b):
    m = a.shape[1] if trans_a else a.shape[0]
    k = a.shape[0] if trans_a else a.shape[1]
    n = b.shape[0] if trans_b else b.shape[1]
    out = torch.empty(m, n, dtype=a.dtype, device=a.device)
    L.call("nmtg_gemm_static", L.i32(int(trans_a)), L.i32(int(trans_b)), L.i64(m), L.i64(n), L.i64(k), L.f32(1.0), L.ptr(a),
           L.i64(a.stride(0)), L.i64(0), L.ptr(b), L.i64(b.stride(0)), L.i64(0), L.ptr(out), L.i64(out.stride(0)), L.i64(0),
           L.i64(1), L.ptr(None), L.i32(L.dtype_code(a)), L.stream_of(a))
    return out


def test_static_scratch_gemm_matches_the_workspace_form(dev):
    lib = L.load()
    lib.nmtg_gemm_static_max_workspace_bytes.restype = ctypes.c_int64
    cap = lib.nmtg_gemm_static_max_workspace_bytes()
    assert cap == 32 << 20
    g = torch.Generator().manual_seed(101)
    for (m, n, k) in [(512, 256, 8192), (256, 128, 4096)]:          # dW-shaped: both split K; the second is smaller
        need = lib.nmtg_gemm_workspace_bytes(L.i64(m), L.i64(n), L.i64(k), L.i64(1))
        assert 0 < need <= cap
        a = torch.randn(k, m, generator=g).to(torch.bfloat16).to(dev)
        b = torch.randn(k, n, generator=g).to(torch.bfloat16).to(dev)
        want = gemm(a, b, True, False)                               # workspace allocated by the caller
        got = gemm_static(a, b, True, False)
        assert torch.equal(got, want)
    # a product that does not split needs no scratch at all
    a = torch.randn(128, 64, generator=g).to(torch.float16).to(dev)
    b = torch.randn(96, 64, generator=g).to(torch.float16).to(dev)
    assert torch.equal(gemm_static(a, b, False, True), gemm(a, b, False, True))
    # beyond the built-in scratch: rejected, nothing launched
    big = (8192, 8192, 65536)
    if lib.nmtg_gemm_workspace_bytes(L.i64(big[0]), L.i64(big[1]), L.i64(big[2]), L.i64(1)) > cap:
        with pytest.raises(RuntimeError, match="built-in scratch"):
            L.call("nmtg_gemm_static", L.i32(1), L.i32(0), L.i64(big[0]), L.i64(big[1]), L.i64(big[2]), L.f32(1.0), L.ptr(a),
                   L.i64(big[0]), L.i64(0), L.ptr(b), L.i64(big[1]), L.i64(0), L.ptr(a), L.i64(big[1]), L.i64(0), L.i64(1),
                   L.ptr(None), L.i32(1), L.stream_of(a))
