"""The HIP path (through the C ABI) against the golden fixtures tests/golden/*.npz.

The fixtures hold small seeded inputs and the values PyTorch's own library routines and autograd
give for them in fp64 (tests/golden/make_fixtures.py); they are independent of oracle/. The
bandwidth-bound ops run in fp32 (tolerance 1e-5 relative), the GEMM-based ops in bf16 (2e-2
relative, 1e-3 absolute; the fixtures carry the fallback's bf16 rounding points).
Collected last on purpose: every other parity test has run when this file starts.
"""
import pytest
import torch

from nmtgminor_amd.modules import mlp as mmlp
from nmtgminor_amd.modules.encdec_attention_func_bias import encdec_attn_bias_func
from nmtgminor_amd.modules.self_attention_func import self_attn_func
from nmtgminor_amd.native import (fast_layer_norm_cuda, fused_dropout_add_cuda, fused_mlp_gelu, mask_softmax_dropout_cuda,
                                  self_multihead_attn_blaslt as sa_native, xentropy_cuda)
from util import assert_close, load_golden

pytestmark = pytest.mark.gpu
F32 = torch.float32
BF = torch.bfloat16


load = load_golden


def test_layer_norm_fixture(dev):
    f = load("layer_norm")
    x, g, b, dy = (f[k].to(F32).to(dev) for k in ("x", "gamma", "beta", "dy"))
    z, mu, rs = fast_layer_norm_cuda.ln_fwd(x, g, b, float(f["eps"]))
    assert_close(z, f["y"], F32, "y", atol=1e-5)
    assert_close(mu, f["mu"], F32, "mu", atol=1e-6)
    assert_close(rs, f["rsigma"], F32, "rsigma")
    dx, dg, db, _, _ = fast_layer_norm_cuda.ln_bwd(dy, x, mu, rs, g, None, False)
    assert_close(dx, f["dx"], F32, "dx", atol=1e-5)
    assert_close(dg, f["dgamma"], F32, "dgamma", atol=1e-5, scale_atol=True)
    assert_close(db, f["dbeta"], F32, "dbeta", atol=1e-5, scale_atol=True)


def test_dropout_add_fixture(dev):
    f = load("dropout_add")
    p = float(f["p"])
    x = f["x"].to(F32).to(dev)
    mask, out = fused_dropout_add_cuda.forward(True, x, f["residual"].to(F32).to(dev), p, f["mask"].to(dev))
    assert_close(out, f["out"], F32, "out")
    dx = fused_dropout_add_cuda.backward(f["dout"].to(F32).to(dev), mask, p)
    assert_close(dx, f["dx"], F32, "dx")
    assert (dx.cpu()[f["mask"] == 0] == 0).all()


def test_softmax_dropout_fixture(dev):
    f = load("softmax_dropout")
    p, heads = float(f["p"]), int(f["heads"])
    s = f["scores"].to(F32).to(dev)
    pad = f["pad_mask"].bool().to(dev)
    dm = f["dropout_mask"].to(dev)
    _, sm, dr = mask_softmax_dropout_cuda.forward(True, heads, s, p, pad_mask=pad, dropout_mask=dm)
    assert_close(sm, f["softmax"], F32, "softmax")
    assert_close(dr, f["dropped"], F32, "dropped")
    assert (sm.cpu()[f["softmax"] == 0] == 0).all()                      # masked keys: exact zeros
    ds = mask_softmax_dropout_cuda.backward_recompute(heads, f["dout"].to(F32).to(dev), None, s, dm, p, pad_mask=pad)
    assert_close(ds, f["dscores"], F32, "dscores", atol=1e-5)


def test_xentropy_fixture(dev):
    f = load("xentropy")
    eps, pad = float(f["smoothing"]), int(f["padding_idx"])
    logits = f["logits"].to(F32).to(dev)
    labels = f["labels"].to(dev)
    losses, lse = xentropy_cuda.forward(logits, labels, eps, False, padding_idx=pad)
    assert_close(losses, f["losses"], F32, "losses", rtol=2e-5, atol=2e-5)
    assert_close(lse, f["lse"], F32, "lse", rtol=2e-6, atol=2e-5)
    dx = xentropy_cuda.backward(f["grad_loss"].to(F32).to(dev), logits, lse, labels, eps, padding_idx=pad)
    assert_close(dx, f["dlogits"], F32, "dlogits", atol=1e-6)
    padrows = f["labels"] == pad
    assert (losses.cpu()[padrows] == 0).all() and (dx.cpu()[padrows] == 0).all()


@pytest.mark.parametrize("act", ["gelu", "relu", "silu", "agelu"])
def test_mlp_fixture(dev, act):
    f = load("mlp")
    p = float(f["p"])
    leaves = [f[k].to(BF).to(dev).requires_grad_() for k in ("x", "w1", "w2", "b1", "b2")]
    mask = f["mask"].to(dev)
    y = getattr(mmlp, f"mlp_{act}_function")(p, False, *leaves, mask=mask)
    y.backward(f["dy"].to(BF).to(dev))
    assert_close(y, f[f"{act}_y"], BF, "y")
    assert_close(leaves[0].grad, f[f"{act}_dx"], BF, "dx", scale_atol=True)
    assert_close(leaves[1].grad, f[f"{act}_dw1"], BF, "dW1", scale_atol=True)
    assert_close(leaves[2].grad, f[f"{act}_dw2"], BF, "dW2", scale_atol=True)
    assert_close(leaves[3].grad, f[f"{act}_db1"], BF, "db1", scale_atol=True)
    assert_close(leaves[4].grad, f[f"{act}_db2"], BF, "db2", scale_atol=True)
    if act == "gelu":
        _, post, pre, _ = fused_mlp_gelu.forward(p, [t.detach() for t in leaves], mask)
        assert_close(pre.view_as(f["gelu_pre"]), f["gelu_pre"], BF, "pre-activation")
        assert_close(post.view_as(f["gelu_post"]), f["gelu_post"], BF, "activation")
        assert (post.view_as(f["gelu_post"]).cpu()[f["mask"] == 0] == 0).all()


def test_self_attention_fixture(dev):
    f = load("self_attention")
    p, h = float(f["p"]), int(f["heads"])
    leaves = [f[k].to(BF).to(dev).requires_grad_() for k in ("x", "w_in", "w_out", "b_in", "b_out")]
    pad = f["pad_mask"].bool().to(dev)
    dm = f["dropout_mask"].to(dev)
    out, cov = self_attn_func(False, True, h, leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], pad, p, False, None,
                              False, None, True, True, False, dm)
    out.backward(f["dout"].to(BF).to(dev))
    assert_close(out, f["outputs"], BF, "outputs")
    assert_close(cov, f["dropout_results"], BF, "dropout_results")
    for i, k in enumerate(("dx", "dw_in", "dw_out", "db_in", "db_out")):
        assert_close(leaves[i].grad, f[k], BF, k, scale_atol=True)
    lin, _, _, _, ctx, _ = sa_native.forward(False, True, h, *[t.detach() for t in leaves], pad, p, dropout_mask=dm)
    assert_close(lin, f["input_lin_results"], BF, "input_lin_results")
    assert_close(ctx, f["matmul2_results"], BF, "matmul2_results")


def test_encdec_attention_fixture(dev):
    f = load("encdec_attention")
    h = int(f["heads"])
    g = lambda k: f[k].to(BF).to(dev)
    out, cov = encdec_attn_bias_func(False, True, h, g("x_q"), g("x_kv"), g("w_q"), g("w_kv"), g("w_out"), g("b_q"), g("b_kv"),
                                     g("b_out"), f["pad_mask"].bool().to(dev), 0.0, False, None, False, None, None, True, True,
                                     None)
    assert_close(out, f["outputs"], BF, "outputs")
    assert_close(cov, f["softmax_results"], BF, "softmax_results")
