"""The MFMA GEMM core against a plain PyTorch fp32 product of the same (rounded) operands.

This is a floating-point kernel, so the reference here is torch.matmul in fp32 on the GPU; the
composite ops built on it (MLP, attention) are checked against the CPU oracle in their own tests.
"""
import pytest
import torch

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
        gemm(a, a)                                        # fp32 is not an MFMA input type here
    h = a.half()
    with pytest.raises(RuntimeError):
        gemm(h, h, True, True)                            # A^T B^T not provided
    with pytest.raises(RuntimeError):
        gemm(h, torch.randn(4, 8, device=dev).half())     # inner dims differ
