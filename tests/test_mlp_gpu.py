"""Fused MLP parity: HIP (through the C ABI) vs the CPU oracle with the dropout mask replayed.

Follows the reference's MLP tests (onmt/modules/mlp/test_mlp_gelu.py:229-307,
onmt/modules/mlp/test_mlp_relu.py:150-242): the same mask on both sides, outputs and every
gradient compared; sizes include the reference's [1024, 4096, 1024] and the benchmark's
[512, 2048, 512] at 8192 tokens.
"""
import pytest
import torch

from nmtgminor_amd.modules import mlp as mmlp
from nmtgminor_amd.native import fused_mlp_gelu, fused_mlp_relu, mlp_gelu_blaslt
from oracle import inputs, mlp as omlp
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64
NATIVE = {"gelu": fused_mlp_gelu, "relu": fused_mlp_relu}


def _oracle(d, act, p, masks, gate_from=None):
    """Hidden tensors are stored in the working dtype on both sides (round_to).

    gate_from (relu only): the stored dropped output of the run under test. relu' is a step, and a
    pre-activation within accumulation noise of zero can fall on either side of it depending on
    the summation order; the reference's backward takes the gate from the stored output
    (mlp_relu_cuda.cu:1174-1240), so the oracle's backward is handed the same stored tensor."""
    ws, bs = [d["w1"], d["w2"]], [d["b1"], d["b2"]]
    rt = d["x"].dtype
    y, pre, post = omlp.mlp_fwd(d["x"], ws, bs, act, p, masks, D, round_to=rt)
    pre_b, post_b = pre, post
    if gate_from is not None:
        stored = gate_from.detach().cpu().view_as(post[0]).to(D)
        pre_b, post_b = [stored], [stored]
    dx, dws, dbs = omlp.mlp_bwd(d["dy"], d["x"], ws, pre_b, post_b, act, p, masks, D, round_to=rt)
    return y, pre, post, dx, dws, dbs


def _check(dtype, got, want_tuple, tokens):
    y, pre, post, dx, dws, dbs = want_tuple
    gy, gpre, gpost, gdx, gdws, gdbs = got
    assert_close(gy, y, dtype, "y")
    if gpre is not None:
        assert_close(gpre.view_as(pre[0]), pre[0], dtype, "pre-activation")
    assert_close(gpost.view_as(post[0]), post[0], dtype, "post-activation")
    assert_close(gdx, dx, dtype, "dx", scale_atol=True)
    for i in range(2):
        # sums over `tokens` products: scale the absolute tolerance with the result's magnitude
        assert_close(gdws[i], dws[i], dtype, f"dW{i + 1}", scale_atol=True)
        assert_close(gdbs[i], dbs[i], dtype, f"db{i + 1}", scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("act", ["gelu", "relu", "silu", "agelu"])
@pytest.mark.parametrize("tokens,dm,di,p", [(8192, 512, 2048, 0.1), (1000, 1024, 4096, 0.2), (72, 96, 200, 0.5),
                                            (256, 128, 256, 0.0)])
def test_mlp_autograd_function(dev, dtype, act, tokens, dm, di, p):
    d = inputs.mlp_inputs(tokens, dm, di, dtype, p=p, seed=61, zero_bias=False)
    fn = getattr(mmlp, f"mlp_{act}_function")
    leaves = [d[k].to(dev).requires_grad_() for k in ("x", "w1", "w2", "b1", "b2")]
    y = fn(p, False, *leaves, mask=d["mask"].to(dev) if p > 0 else None)
    y.backward(d["dy"].to(dev))
    # intermediates via the native module directly
    native = NATIVE.get(act)
    gpre = gpost = None
    if native is fused_mlp_gelu:
        _, gpost, gpre, _ = native.forward(p, [t.detach() for t in leaves], d["mask"].to(dev) if p > 0 else None)
    elif native is fused_mlp_relu:
        _, gpost, _ = native.forward(p, False, [t.detach() for t in leaves], d["mask"].to(dev) if p > 0 else None)
    want = _oracle(d, act, p, [d["mask"]] if p > 0 else None, gate_from=gpost if act == "relu" else None)
    if gpost is None:
        gpost = want[2][0]
    got = (y, gpre, gpost, leaves[0].grad, [leaves[1].grad, leaves[2].grad], [leaves[3].grad, leaves[4].grad])
    _check(dtype, got, want, tokens)
    if p > 0:
        dropped = (d["mask"] == 0)
        assert (gpost.view(tokens, di).cpu()[dropped] == 0).all()       # dropped units: exact zeros


def test_mlp_benchmark_shape_zero_bias_fp16(dev):
    d = inputs.mlp_inputs(seed=1002)                                      # 8192 x 512 -> 2048 -> 512, fp16, p = 0.1
    want = _oracle(d, "gelu", 0.1, [d["mask"]])
    ins = [d[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
    ins[0].requires_grad_()
    out = fused_mlp_gelu.forward(0.1, ins, d["mask"].to(dev))
    grads = fused_mlp_gelu.backward(0.1, d["dy"].to(dev), out, ins)
    _check(torch.float16, (out[0], out[2], out[1], grads[0], grads[1:3], grads[3:5]), want, 8192)
    assert torch.equal(out[3].cpu(), d["mask"].view(-1))
    again = fused_mlp_gelu.backward(0.1, d["dy"].to(dev), out, ins)
    assert all(torch.equal(a, b) for a, b in zip(grads, again))           # deterministic reductions


def test_mlp_recompute_and_input_only(dev):
    d = inputs.mlp_inputs(512, 256, 1024, torch.bfloat16, p=0.3, seed=62, zero_bias=False)
    want = _oracle(d, "gelu", 0.3, [d["mask"]])
    ins = [d[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
    ins[0].requires_grad_()
    out = mlp_gelu_blaslt.forward(0.3, ins, d["mask"].to(dev))
    g_full = mlp_gelu_blaslt.backward(0.3, False, d["dy"].to(dev), out, ins)
    g_rec = mlp_gelu_blaslt.backward(0.3, True, d["dy"].to(dev), (out[0], out[-1]), ins)
    assert all(torch.equal(a, b) for a, b in zip(g_full, g_rec))
    (dx_only,) = mlp_gelu_blaslt.backward_input_only(0.3, d["dy"].to(dev), out, ins)
    assert torch.equal(dx_only, g_full[0])
    assert_close(dx_only, want[3], torch.bfloat16, "dx", scale_atol=True)
    # relu: backward from the dropped output only, and the recompute entry point
    o = fused_mlp_relu.forward(0.3, True, ins, d["mask"].to(dev))
    wr = _oracle(d, "relu", 0.3, [d["mask"]], gate_from=o[1])
    g1 = fused_mlp_relu.backward(0.3, d["dy"].to(dev), o, ins)
    g2 = fused_mlp_relu.backward_recompute(0.3, d["dy"].to(dev), o[2], ins)
    assert all(torch.equal(a, b) for a, b in zip(g1, g2))
    assert_close(g1[0], wr[3], torch.bfloat16, "relu dx", scale_atol=True)
    assert_close(g1[1], wr[4][0], torch.bfloat16, "relu dW1", scale_atol=True)


def test_mlp_three_layers_and_rng_mask(dev):
    g = torch.Generator().manual_seed(63)
    x = torch.randn(300, 64, generator=g).half()
    ws = [inputs.xavier_uniform(s, g).half() for s in ((128, 64), (192, 128), (32, 192))]
    bs = [(0.1 * torch.randn(s, generator=g)).half() for s in (128, 192, 32)]
    ins = [t.to(dev) for t in [x] + ws + bs]
    ins[0].requires_grad_()
    torch.cuda.manual_seed(5)
    out = fused_mlp_gelu.forward(0.25, ins)                               # mask drawn in the GEMM epilogue
    mask = out[3]
    assert mask.numel() == 300 * (128 + 192) and abs(mask.float().mean().item() - 0.75) < 0.02
    masks = [mask[:300 * 128].view(300, 128).cpu(), mask[300 * 128:].view(300, 192).cpu()]
    y, pre, post = omlp.mlp_fwd(x, ws, bs, "gelu", 0.25, masks, D, round_to=torch.float16)
    assert_close(out[0], y, torch.float16, "3-layer y")
    dy = torch.randn(300, 32, generator=g).half()
    grads = fused_mlp_gelu.backward(0.25, dy.to(dev), out, ins)
    dx, dws, dbs = omlp.mlp_bwd(dy, x, ws, pre, post, "gelu", 0.25, masks, D, round_to=torch.float16)
    assert_close(grads[0], dx, torch.float16, "3-layer dx", scale_atol=True)
    for i in range(3):
        assert_close(grads[1 + i], dws[i], torch.float16, f"3-layer dW{i}", scale_atol=True)
        assert_close(grads[4 + i], dbs[i], torch.float16, f"3-layer db{i}", scale_atol=True)


# fp32: the precision the reference's own MLP tests run in (test_mlp_gelu.py:262-300: sizes [1024, 4096, 1024], a
# token count drawn as a multiple of 8, dropout 0 / 0.2 / 0.5 / 0.7, output atol = rtol = 1e-3, gradients rtol 1e-5 on
# a loss scaled to make them tiny). Here against the fp64 oracle at rtol 1e-4, atol 1e-5 (times the largest expected
# magnitude for the sums over tokens): fp32 products summed over up to 4096 terms, and a gelu whose normal CDF is
# accurate to 1.5e-7.
F32 = dict(rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("act,tokens,dm,di,p", [("gelu", 520, 1024, 4096, 0.0), ("gelu", 520, 1024, 4096, 0.2),
                                                ("gelu", 136, 1024, 4096, 0.7), ("relu", 72, 96, 200, 0.5),
                                                ("silu", 257, 130, 66, 0.2), ("agelu", 64, 33, 129, 0.0)])
def test_mlp_fp32(dev, act, tokens, dm, di, p):
    dtype = torch.float32
    d = inputs.mlp_inputs(tokens, dm, di, dtype, p=p, seed=67, zero_bias=False)
    fn = getattr(mmlp, f"mlp_{act}_function")
    leaves = [d[k].to(dev).requires_grad_() for k in ("x", "w1", "w2", "b1", "b2")]
    y = fn(p, False, *leaves, mask=d["mask"].to(dev) if p > 0 else None)
    y.backward(d["dy"].to(dev))
    gpost = None
    if act == "relu":
        _, gpost, _ = fused_mlp_relu.forward(p, False, [t.detach() for t in leaves], d["mask"].to(dev) if p > 0 else None)
    wy, _, _, wdx, wdws, wdbs = _oracle(d, act, p, [d["mask"]] if p > 0 else None, gate_from=gpost)
    assert_close(y, wy, dtype, "y", **F32)
    assert_close(leaves[0].grad, wdx, dtype, "dx", scale_atol=True, **F32)
    for i in range(2):
        assert_close(leaves[1 + i].grad, wdws[i], dtype, f"dW{i + 1}", scale_atol=True, **F32)
        assert_close(leaves[3 + i].grad, wdbs[i], dtype, f"db{i + 1}", scale_atol=True, **F32)


def test_mlp_fp32_draws_the_same_dropout_stream_as_the_16_bit_kernels(dev):
    d = inputs.mlp_inputs(96, 64, 128, torch.float32, p=0.3, seed=68, zero_bias=False)
    ins = [d[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
    torch.cuda.manual_seed(77)
    _, post, _, mask32 = fused_mlp_gelu.forward(0.3, ins)
    torch.cuda.manual_seed(77)
    _, _, _, mask16 = fused_mlp_gelu.forward(0.3, [t.half() for t in ins])
    assert torch.equal(mask32, mask16)
    assert 0.6 < float(mask32.float().mean()) < 0.8
    assert bool((post.view(96, 128)[mask32.view(96, 128) == 0] == 0).all())


def test_mlp_errors(dev):
    x = torch.randn(8, 16, device=dev)
    w1, w2 = torch.randn(32, 16, device=dev), torch.randn(16, 32, device=dev)
    b1, b2 = torch.zeros(32, device=dev), torch.zeros(16, device=dev)
    with pytest.raises(RuntimeError):
        fused_mlp_gelu.forward(0.0, [t.double() for t in (x, w1, w2, b1, b2)])   # there is no fp64 kernel
    h = [t.half() for t in (x, w1, w2, b1, b2)]
    with pytest.raises(RuntimeError):
        fused_mlp_gelu.forward(0.0, [h[0], h[2], h[1], h[3], h[4]])        # weight shapes do not chain
    with pytest.raises(RuntimeError):
        fused_mlp_gelu.forward(0.0, [t.cpu() for t in h])
