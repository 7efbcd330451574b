"""The MFMA GEMM core against a plain PyTorch fp32 product of the same (rounded) operands.

This is a floating-point kernel, so the reference here is torch.matmul in fp32 on the GPU; the
composite ops built on it (MLP, attention) are checked against the CPU oracle in their own tests.
"""
import pytest
import torch

from nmtgminor_amd import _lib
from nmtgminor_amd.native.linear_gemm import gemm
from util import assert_close

pytestmark = pytest.mark.gpu


def _ref(a, b, ta, tb, alpha=1.0, bias=None):
    af = a.float().transpose(-1, -2) if ta else a.float()
    bf = b.float().transpose(-1, -2) if tb else b.float()
    r = alpha * (af @ bf)
    return r + bias.float() if bias is not None else r


def _mk(shape, dev, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype).to(dev)


SHAPES = [(256, 256, 64), (128, 128, 128), (512, 2048, 512), (300, 200, 72), (1, 8, 8), (257, 129, 1000),
          (64, 1504, 64), (1024, 64, 512), (8192, 512, 2048)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
def test_gemm_layouts(dev, dtype, m, n, k, layout):
    ta, tb = layout[0] == "t", layout[1] == "t"
    a = _mk((k, m) if ta else (m, k), dev, dtype, 1)
    b = _mk((n, k) if tb else (k, n), dev, dtype, 2)
    c = gemm(a, b, ta, tb, alpha=0.5)
    assert_close(c, _ref(a, b, ta, tb, 0.5).cpu(), dtype, f"{layout} {m}x{n}x{k}", scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_unaligned_extents(dev, dtype):
    # K = 1500 rows are 8-byte aligned only (3000 B pitch); N = 1500 output likewise; odd sizes fall to scalar access
    for (m, n, k) in [(128, 1500, 64), (128, 64, 1500), (70, 1500, 1500), (33, 77, 55)]:
        a, b = _mk((m, k), dev, dtype, 3), _mk((n, k), dev, dtype, 4)
        assert_close(gemm(a, b, False, True), _ref(a, b, False, True).cpu(), dtype, f"nt {m}x{n}x{k}", scale_atol=True)
        b2 = _mk((k, n), dev, dtype, 5)
        assert_close(gemm(a, b2, False, False), _ref(a, b2, False, False).cpu(), dtype, f"nn {m}x{n}x{k}", scale_atol=True)
        a2 = _mk((k, m), dev, dtype, 6)
        assert_close(gemm(a2, b2, True, False), _ref(a2, b2, True, False).cpu(), dtype, f"tn {m}x{n}x{k}", scale_atol=True)


def test_gemm_bias_and_batched_strided_views(dev):
    dtype = torch.bfloat16
    t, bh, d = 96, 6, 64
    qkv = _mk((t, bh, 3, d), dev, dtype, 7)              # the attention layout: q/k/v interleaved per head
    q, k, v = (qkv[:, :, i, :].transpose(0, 1) for i in range(3))   # [bh, t, d] views, row stride bh*3*d
    s = gemm(q, k, False, True, alpha=d ** -0.5)
    assert_close(s, _ref(q, k, False, True, d ** -0.5).cpu(), dtype, "scores", scale_atol=True)
    p = torch.softmax(s.float(), -1).to(dtype)
    out = torch.empty(t, bh, d, dtype=dtype, device=dev)
    gemm(p, v, False, False, out=out.transpose(0, 1))    # written straight into the [t, bh, d] layout
    assert_close(out.transpose(0, 1), _ref(p, v, False, False).cpu(), dtype, "context", scale_atol=True)
    dv = gemm(p, out.transpose(0, 1), True, False)
    assert_close(dv, _ref(p, out.transpose(0, 1), True, False).cpu(), dtype, "tn batched", scale_atol=True)
    x, w, bias = _mk((200, 128), dev, dtype, 8), _mk((384, 128), dev, dtype, 9), _mk((384,), dev, dtype, 10)
    assert_close(gemm(x, w, False, True, bias=bias), _ref(x, w, False, True, 1.0, bias).cpu(), dtype, "bias", scale_atol=True)


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 200, 72), (1, 8, 8), (257, 129, 1000), (130, 70, 33), (1024, 64, 512)])
@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
def test_gemm_fp32_layouts_against_fp64(dev, m, n, k, layout):
    """The fp32 matrix-core kernel: fp32 products and sums, so the yardstick is the fp64 product of the same operands
    (rtol 1e-5 with an absolute part of 1e-6 times the largest result: the rounding of a sum over k terms)."""
    ta, tb = layout[0] == "t", layout[1] == "t"
    a = _mk((k, m) if ta else (m, k), dev, torch.float32, 21)
    b = _mk((n, k) if tb else (k, n), dev, torch.float32, 22)
    bias = _mk((n,), dev, torch.float32, 23)
    c = gemm(a, b, ta, tb, alpha=0.5, bias=bias)
    ad, bd = a.double().cpu(), b.double().cpu()
    want = 0.5 * ((ad.t() if ta else ad) @ (bd.t() if tb else bd)) + bias.double().cpu()
    assert_close(c, want, torch.float32, f"fp32 {layout} {m}x{n}x{k}", rtol=1e-5, atol=1e-6, scale_atol=True)


def test_gemm_fp32_batched_strided_views(dev):
    t, bh, d = 40, 3, 24
    qkv = _mk((t, bh, 3, d), dev, torch.float32, 24)
    q, k, v = (qkv[:, :, i, :].transpose(0, 1) for i in range(3))      # [bh, t, d] views, row stride bh*3*d
    s = gemm(q, k, False, True, alpha=0.25)
    assert_close(s, 0.25 * (q.double() @ k.double().transpose(1, 2)).cpu(), torch.float32, "scores", rtol=1e-5, atol=1e-6, scale_atol=True)
    out = torch.empty(t, bh, d, dtype=torch.float32, device=dev)
    gemm(s, v, False, False, out=out.transpose(0, 1))
    assert_close(out.transpose(0, 1), (s.double() @ v.double()).cpu(), torch.float32, "context", rtol=1e-5, atol=1e-6, scale_atol=True)
    dv = gemm(s, out.transpose(0, 1), True, False)
    assert_close(dv, (s.double().transpose(1, 2) @ out.transpose(0, 1).double()).cpu(), torch.float32, "tn", rtol=1e-5, atol=1e-6,
                 scale_atol=True)


def test_gemm_split_k_is_deterministic(dev):
    a, b = _mk((8192, 512), dev, torch.float16, 11), _mk((8192, 256), dev, torch.float16, 12)
    c1 = gemm(a, b, True, False)
    c2 = gemm(a, b, True, False)
    assert torch.equal(c1, c2)
    assert_close(c1, _ref(a, b, True, False).cpu(), torch.float16, "split-k", scale_atol=True)
    c3 = gemm(a, b, True, False, split_k=False)
    assert_close(c3, _ref(a, b, True, False).cpu(), torch.float16, "no split", scale_atol=True)


def test_gemm_errors(dev):
    a = torch.randn(8, 8, device=dev)
    with pytest.raises(RuntimeError):
        gemm(a.double(), a.double())                      # there is no fp64 kernel
    h = a.half()
    with pytest.raises(RuntimeError):
        gemm(h, h, True, True)                            # A^T B^T not provided
    with pytest.raises(RuntimeError):
        gemm(h, torch.randn(4, 8, device=dev).half())     # inner dims differ


def _pitched(rows, cols, dev, dtype, seed, pitch_to=64):
    """[rows, cols] view of a buffer whose row pitch is cols rounded up to `pitch_to` elements; the pad columns hold
    NaN so that a kernel that lets them into a sum is caught."""
    pitch = (cols + pitch_to - 1) // pitch_to * pitch_to
    buf = torch.full((rows, pitch), float("nan"), dtype=dtype, device=dev)
    buf[:, :cols] = _mk((rows, cols), dev, dtype, seed)
    return buf[:, :cols]


def _traced(fn):
    _lib.trace_begin()
    out = fn()
    return out, _lib.trace_end()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("v", [250054 % 4096 + 4096, 1030, 70, 6])     # v % 4 == 2: the vocabulary of the loss benchmark is 250 054
def test_ragged_extents_keep_16_byte_accesses(dev, dtype, v):
    """Extents that are not a multiple of the access width on 16-byte aligned, pitched operands (the chunk buffers of
    the projection + cross-entropy module): the three products of that module must run the 16-byte kernels, and the
    slot-ring loop wherever the reduction is a multiple of 64, with a predicated last vector / tile."""
    assert v % 4 == 2
    n, e = 320, 128
    h = _mk((n, e), dev, dtype, 21)
    w = _pitched(v, e, dev, dtype, 22)                       # [V, E], E % 64 == 0
    bias = _mk((v,), dev, dtype, 23)
    z = torch.full((n, (v + 63) // 64 * 64), float("nan"), dtype=dtype, device=dev)[:, :v]
    # logits [N, V] = h W^T + b: ragged N
    _, tr = _traced(lambda: gemm(h, w, trans_b=True, bias=bias, out=z))
    assert_close(z, _ref(h, w, False, True, 1.0, bias).cpu(), dtype, f"nt ragged n={v}", scale_atol=True)
    assert all(k.endswith("_ring") for k in tr), tr
    dz = _pitched(n, v, dev, dtype, 24)
    # dW [V, E] = dz^T h: ragged M, reduction over the 320 rows
    dw, tr = _traced(lambda: gemm(dz, h, trans_a=True, split_k=False))
    assert_close(dw, _ref(dz, h, True, False).cpu(), dtype, f"tn ragged m={v}", scale_atol=True)
    assert all(k.endswith("_ring") for k in tr), tr
    # dh [N, E] = dz W: ragged K (the two-buffer loop zeroes the tail of the last 16-byte vector)
    dh, tr = _traced(lambda: gemm(dz, w))
    assert_close(dh, _ref(dz, w, False, False).cpu(), dtype, f"nn ragged k={v}", scale_atol=True)
    assert not any("_v1" in k or "_v4" in k for k in tr), tr
    # the same with K as the contiguous index of both operands
    a2, b2 = _pitched(96, v, dev, dtype, 25), _pitched(72, v, dev, dtype, 26)
    c2, tr = _traced(lambda: gemm(a2, b2, trans_b=True))
    assert_close(c2, _ref(a2, b2, False, True).cpu(), dtype, f"nt ragged k={v}", scale_atol=True)
    assert not any("_v1" in k or "_v4" in k for k in tr), tr
    # pad columns of the output buffer were not written
    assert torch.isnan(z.as_strided((n, z.stride(0) - v), (z.stride(0), 1), v)).all()


def test_transposed_product_without_workspace_runs_unsplit(dev):
    # a transposed-A product may split K only when it is given a workspace; without one it runs unsplit
    a, b = _mk((4096, 256), dev, torch.float16, 31), _mk((4096, 128), dev, torch.float16, 32)
    c, tr = _traced(lambda: gemm(a, b, True, False, split_k=False))
    assert not any("splitk" in k for k in tr), tr
    assert_close(c, _ref(a, b, True, False).cpu(), torch.float16, "unsplit", scale_atol=True)
