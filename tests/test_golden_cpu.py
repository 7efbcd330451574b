"""The CPU oracle against the golden fixtures (tests/golden/*.npz, written by
tests/golden/make_fixtures.py from PyTorch's library routines and autograd in fp64).

The fixtures are independent of oracle/: a change in the arithmetic of either side shows up here.
The 16-bit cases carry the fallback's rounding points (bf16), which the oracle reproduces with
round_to=torch.bfloat16."""
import os

import numpy as np
import torch

from oracle import attention, dropout_add, fused_optim, layer_norm, mlp, relative_attention, softmax_dropout, xentropy

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
D = torch.float64
BF = torch.bfloat16


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: torch.from_numpy(np.array(z[k])) for k in z.files}


F32 = dict(rtol=2e-6, atol=1e-6)   # fixtures of the 16-bit cases are stored as float32


def close(got, want, what, rtol=1e-9, atol=1e-11):
    torch.testing.assert_close(got.to(D), want.to(D), rtol=rtol, atol=atol, msg=lambda m: f"{what}: {m}")


def test_layer_norm_fixture():
    f = load("layer_norm")
    y, mu, rs = layer_norm.ln_fwd(f["x"], f["gamma"], f["beta"], float(f["eps"]), D)
    close(y, f["y"], "y")
    close(mu, f["mu"], "mu")
    close(rs, f["rsigma"], "rsigma")
    dx, dg, db = layer_norm.ln_bwd(f["dy"], f["x"], mu, rs, f["gamma"], D)
    close(dx, f["dx"], "dx")
    close(dg, f["dgamma"], "dgamma")
    close(db, f["dbeta"], "dbeta")
    dx2, dg2, db2 = layer_norm.ln_bwd_memory_efficient(f["dy"], y, rs, f["gamma"], f["beta"], D)
    close(dx2, f["dx"], "dx (from the output)", rtol=1e-7, atol=1e-9)
    close(dg2, f["dgamma"], "dgamma (from the output)", rtol=1e-7, atol=1e-9)


def test_dropout_add_fixture():
    f = load("dropout_add")
    p = float(f["p"])
    close(dropout_add.dropout_add_fwd(f["x"], f["residual"], f["mask"], p, D), f["out"], "out")
    close(dropout_add.dropout_add_bwd(f["dout"], f["mask"], p, D)[0], f["dx"], "dx")


def test_softmax_dropout_fixture():
    f = load("softmax_dropout")
    p, heads = float(f["p"]), int(f["heads"])
    masked = softmax_dropout.masked_scores(f["scores"].to(D), pad_mask=f["pad_mask"].bool(), heads=heads)
    sm, dr = softmax_dropout.softmax_dropout_fwd(masked, f["dropout_mask"], p, D)
    close(sm, f["softmax"], "softmax")
    close(dr, f["dropped"], "dropped")
    close(softmax_dropout.softmax_dropout_bwd(f["dout"], sm, f["dropout_mask"], p, D), f["dscores"], "dscores")


def test_xentropy_fixture():
    f = load("xentropy")
    eps, pad = float(f["smoothing"]), int(f["padding_idx"])
    losses, lse = xentropy.xentropy_fwd(f["logits"], f["labels"], eps, pad, D)
    close(losses, f["losses"], "losses")
    close(lse, f["lse"], "lse")
    close(xentropy.xentropy_bwd(f["grad_loss"], f["logits"], lse, f["labels"], eps, pad, D), f["dlogits"], "dlogits")
    assert (losses[f["labels"] == pad] == 0).all()


def test_mlp_fixture():
    f = load("mlp")
    p = float(f["p"])
    ws, bs = [f["w1"], f["w2"]], [f["b1"], f["b2"]]
    for act in ("gelu", "relu", "silu", "agelu"):
        y, pre, post = mlp.mlp_fwd(f["x"], ws, bs, act, p, [f["mask"]], D, round_to=BF)
        close(pre[0], f[f"{act}_pre"], f"{act} pre-activation", **F32)
        close(post[0], f[f"{act}_post"], f"{act} activation", **F32)
        close(y, f[f"{act}_y"], f"{act} y", **F32)
        dx, dws, dbs = mlp.mlp_bwd(f["dy"], f["x"], ws, pre, post, act, p, [f["mask"]], D, round_to=BF)
        close(dx, f[f"{act}_dx"], f"{act} dx", **F32)
        for i in (0, 1):
            close(dws[i], f[f"{act}_dw{i + 1}"], f"{act} dW{i + 1}", **F32)
            close(dbs[i], f[f"{act}_db{i + 1}"], f"{act} db{i + 1}", **F32)


def test_self_attention_fixture():
    f = load("self_attention")
    p, h = float(f["p"]), int(f["heads"])
    fwd = attention.self_attn_fwd(f["x"], f["w_in"], f["w_out"], f["b_in"], f["b_out"], h, f["pad_mask"].bool(), None, p,
                                  f["dropout_mask"], D, round_to=BF)
    for k in ("input_lin_results", "softmax_results", "dropout_results", "matmul2_results", "outputs"):
        close(fwd[k], f[k], k, **F32)
    bwd = attention.self_attn_bwd(f["dout"], f["x"], f["w_in"], f["w_out"], h, fwd, p, f["dropout_mask"], D, round_to=BF)
    for k in ("dx", "dw_in", "dw_out", "db_in", "db_out"):
        close(bwd[k], f[k], k, **F32)


def test_encdec_attention_fixture():
    f = load("encdec_attention")
    h = int(f["heads"])
    fwd = attention.encdec_attn_fwd(f["x_q"], f["x_kv"], f["w_q"], f["w_kv"], f["w_out"], f["b_q"], f["b_kv"], f["b_out"], h,
                                    f["pad_mask"].bool(), 0.0, None, D, round_to=BF)
    for k in ("softmax_results", "matmul2_results", "outputs"):
        close(fwd[k], f[k], k, **F32)


def test_relative_attention_fixture():
    f = load("relative_attention")
    p, h = float(f["p"]), int(f["heads"])
    names = ("x", "pos", "w_in", "w_out", "w_pos", "b_in", "b_out", "b_pos", "r_w_bias", "r_r_bias")
    fwd = relative_attention.rel_self_attn_fwd(*(f[k] for k in names), h, f["pad_mask"].bool(), None, p, f["dropout_mask"], D,
                                               round_to=BF)
    for k in ("softmax_results", "dropout_results", "matmul2_results", "outputs"):
        close(fwd[k], f[k], k, **F32)
    bwd = relative_attention.rel_self_attn_bwd(f["dout"], f["x"], f["pos"], f["w_in"], f["w_out"], f["w_pos"], h, fwd, p,
                                               f["dropout_mask"], D, round_to=BF)
    for k in ("dx", "dw_in", "dw_out", "dw_pos", "db_in", "db_out", "db_pos", "dr_w_bias", "dr_r_bias"):
        close(bwd[k], f[k], k, **F32)


def test_fused_optim_fixture():
    f = load("fused_optim")
    hp = [float(f[k]) for k in ("lr", "beta1", "beta2", "eps")]
    wd = float(f["weight_decay"])
    for name, mode in (("adamw", 1), ("adam", 0)):
        for i in range(3):
            p, m, v = f[f"p{i}"], torch.zeros_like(f[f"p{i}"]), torch.zeros_like(f[f"p{i}"])
            for step in range(4):
                p, m, v = fused_optim.adam_step(f[f"g{step}_{i}"], p, m, v, *hp, step + 1, mode, True, wd, D)
            close(p, f[f"{name}_p{i}"], f"{name} p{i}", rtol=1e-12, atol=1e-14)
            close(m, f[f"{name}_m{i}"], f"{name} m{i}", rtol=1e-12, atol=1e-14)
            close(v, f[f"{name}_v{i}"], f"{name} v{i}", rtol=1e-12, atol=1e-14)
    total, _ = fused_optim.l2norm([f[f"g3_{i}"] for i in range(3)], D)
    close(total, f["norm"], "norm", rtol=1e-12)
    factor = min(1.0, float(f["max_norm"]) / (float(total) + 1e-6))
    for i in range(3):
        close(fused_optim.scale(f[f"g3_{i}"], factor, D)[0], f[f"clipped{i}"], f"clipped gradient {i}", rtol=1e-12)
