"""Randomly drawn shapes (seeded): every operator against the CPU oracle at sizes nobody picked by hand — odd row
counts, row pitches with padding, head sizes 32 / 64 / 128, key lengths from 1 to 2048, vocabularies that are not
multiples of anything. One case per seed; the drawn case is part of the failure message."""
import random

import pytest
import torch

from nmtgminor_amd.native import (encdec_multihead_attn_bias_blaslt as ed, fast_layer_norm_cuda as ln, fused_mlp_gelu, fused_mlp_silu,
                                  mask_softmax_dropout_cuda as sm, self_multihead_attn_blaslt as sa, xentropy_cuda as xe)
from nmtgminor_amd.native.linear_gemm import gemm
from oracle import attention as oat, inputs, layer_norm as oln, mlp as omlp, softmax_dropout as osd, xentropy as oxe
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64
F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16
SEEDS = list(range(1000, 1048))


def _gemm(rnd, seed, dev):
    m, n = (rnd.choice([1, 2, 7, 8, 33, 64, 100, 128, 129, 200, 256, 300]) for _ in range(2))
    k = rnd.choice([8, 24, 64, 72, 128, 192, 200, 1000])
    batch, d = rnd.choice([1, 1, 3]), rnd.choice([F16, BF16])
    layout, pad = rnd.choice(["nt", "nn", "tn"]), rnd.choice([0, 0, 8, 3])
    rnd.case = f"gemm {layout} {m}x{n}x{k} batch {batch} pad {pad} {d}"
    ta, tb = layout[0] == "t", layout[1] == "t"
    sa_, sb_ = ((k, m) if ta else (m, k)), ((n, k) if tb else (k, n))
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(batch, sa_[0], sa_[1] + pad, generator=g).to(d).to(dev)[:, :, :sa_[1]]       # rows with a padded pitch
    b = torch.randn(batch, sb_[0], sb_[1] + pad, generator=g).to(d).to(dev)[:, :, :sb_[1]]
    c = gemm(a, b, ta, tb, alpha=0.5)
    af = a.double().cpu().transpose(1, 2) if ta else a.double().cpu()
    bf = b.double().cpu().transpose(1, 2) if tb else b.double().cpu()
    assert_close(c, 0.5 * (af @ bf), d, "gemm", scale_atol=True)


def _self(rnd, seed, dev):
    t, b, h, dh = rnd.choice([1, 2, 9, 33, 64, 100, 130]), rnd.choice([1, 2, 3]), rnd.choice([1, 2, 4]), rnd.choice([32, 64, 128])
    e, p, causal, d = h * dh, rnd.choice([0.0, 0.1]), rnd.random() < 0.4, rnd.choice([F16, BF16])
    rnd.case = f"self-attention T {t} B {b} E {e} H {h} p {p} causal {causal} {d}"
    x = inputs.self_attn_inputs(t, b, e, h, d, p=p, seed=seed, causal=causal, zero_bias=False)
    g = lambda k: x[k].to(dev) if x[k] is not None else None
    dm = x["dropout_mask"] if p > 0 else None
    r = sa.forward(causal, True, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("time_mask") if causal else g("pad_mask"), p,
                   dropout_mask=dm.to(dev) if dm is not None else None)
    fw = oat.self_attn_fwd(x["x"], x["w_in"], x["w_out"], x["b_in"], x["b_out"], h, x["pad_mask"], x["time_mask"], p, dm, D, round_to=d)
    assert_close(r[5], fw["outputs"], d, "outputs")
    gr = sa.backward(causal, h, g("dout"), r[4], r[2], r[1], r[0], g("x"), g("w_in"), g("w_out"), r[3], p)
    bw = oat.self_attn_bwd(x["dout"], x["x"], x["w_in"], x["w_out"], h, fw, p, dm, D, round_to=d)
    for name, a_, o_ in (("dx", gr[0], bw["dx"]), ("dw_in", gr[1], bw["dw_in"]), ("dw_out", gr[2], bw["dw_out"]), ("db_in", gr[3], bw["db_in"])):
        assert_close(a_, o_, d, name, scale_atol=True)


def _encdec(rnd, seed, dev):
    tq, tk, b, h = rnd.choice([1, 5, 17, 64]), rnd.choice([1, 3, 40, 100, 257]), rnd.choice([1, 2]), rnd.choice([2, 4])
    e, d, p = h * rnd.choice([32, 64]), rnd.choice([F16, BF16]), rnd.choice([0.0, 0.2])
    rnd.case = f"cross-attention Tq {tq} Tk {tk} B {b} E {e} H {h} p {p} {d}"
    x = inputs.encdec_attn_inputs(tq, tk, b, e, h, d, p=p, seed=seed, zero_bias=False)
    g = lambda k: x[k].to(dev) if x[k] is not None else None
    dm = x["dropout_mask"] if p > 0 else None
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out", "b_q", "b_kv", "b_out")
    r = ed.forward(True, h, *[g(k) for k in names], g("pad_mask"), p, dropout_mask=dm.to(dev) if dm is not None else None)
    fw = oat.encdec_attn_fwd(*[x[k] for k in names], h, x["pad_mask"], p, dm, D, round_to=d)
    assert_close(r[6], fw["outputs"], d, "outputs")
    gr = ed.backward(h, g("dout"), r[5], r[3], r[2], r[0], r[1], g("x_q"), g("x_kv"), g("w_q"), g("w_kv"), g("w_out"), r[4], p)
    bw = oat.encdec_attn_bwd(x["dout"], x["x_q"], x["x_kv"], x["w_q"], x["w_kv"], x["w_out"], h, fw, p, dm, D, round_to=d)
    for name, a_, o_ in (("dx_q", gr[0], bw["dx_q"]), ("dx_kv", gr[1], bw["dx_kv"]), ("dw_q", gr[2], bw["dw_q"]), ("dw_kv", gr[3], bw["dw_kv"])):
        assert_close(a_, o_, d, name, scale_atol=True)


def _mlp(rnd, seed, dev):
    n, dm_, di = rnd.choice([1, 3, 64, 100, 257, 1000]), rnd.choice([8, 64, 96, 128, 200]), rnd.choice([8, 64, 200, 256, 512])
    d, p = rnd.choice([F16, BF16]), rnd.choice([0.0, 0.1, 0.5])
    act, mod = rnd.choice([("gelu", fused_mlp_gelu), ("silu", fused_mlp_silu)])
    rnd.case = f"mlp {act} tokens {n} {dm_}->{di} p {p} {d}"
    x = inputs.mlp_inputs(n, dm_, di, d, p=p, seed=seed, zero_bias=False)
    ins = [x[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
    ins[0].requires_grad_()
    out = mod.forward(p, ins, x["mask"].to(dev) if p > 0 else None)
    gr = mod.backward(p, x["dy"].to(dev), out, ins)
    ws, bs, masks = [x["w1"], x["w2"]], [x["b1"], x["b2"]], ([x["mask"]] if p > 0 else None)
    y, pre, post = omlp.mlp_fwd(x["x"], ws, bs, act, p, masks, D, round_to=d)
    gx, gws, gbs = omlp.mlp_bwd(x["dy"], x["x"], ws, pre, post, act, p, masks, D, round_to=d)
    for name, a_, o_ in (("y", out[0], y), ("dx", gr[0], gx), ("dw1", gr[1], gws[0]), ("dw2", gr[2], gws[1]), ("db1", gr[3], gbs[0]),
                         ("db2", gr[4], gbs[1])):
        assert_close(a_, o_, d, name, scale_atol=True)


def _softmax(rnd, seed, dev):
    bh, tq, tk = rnd.choice([2, 4, 6]), rnd.choice([1, 5, 33]), rnd.choice([1, 2, 7, 64, 100, 333, 512, 1000, 1500, 2048])
    d = rnd.choice([F32, F16, BF16])
    rnd.case = f"softmax BH {bh} Tq {tq} Tk {tk} {d}"
    g = torch.Generator().manual_seed(seed)
    s = (torch.randn(bh, tq, tk, generator=g) * 3).to(d)
    pad, _ = inputs.lengths_mask(bh // 2, tk, max(1, tk // 2), tk, g)
    dmk = inputs.bernoulli_mask((bh, tq, tk), 0.9, g)
    go = torch.randn(bh, tq, tk, generator=g).to(d)
    sm_o, dr_o = osd.softmax_dropout_fwd(osd.masked_scores(s.to(D), pad_mask=pad, heads=2), dmk, 0.1, D)
    _, _, dr = sm.forward(True, 2, s.to(dev), 0.1, pad_mask=pad.to(dev), dropout_mask=dmk.to(dev))
    assert_close(dr, dr_o, d, "dropped")
    ds = sm.backward_recompute(2, go.to(dev), None, s.to(dev), dmk.to(dev), 0.1, pad_mask=pad.to(dev))
    assert_close(ds, osd.softmax_dropout_bwd(go, sm_o, dmk, 0.1, D), d, "dscores")


def _layer_norm(rnd, seed, dev):
    rows, hid = rnd.choice([1, 2, 7, 64, 257]), rnd.choice([8, 24, 64, 100, 512, 768, 1000, 1024, 4096, 5000])
    d, wd = rnd.choice([(F32, F32), (BF16, BF16), (F16, F32)])
    rnd.case = f"layer norm rows {rows} hidden {hid} {d}/{wd}"
    x = inputs.layer_norm_inputs(rows, hid, d, wd, seed=seed)
    g = lambda k: x[k].to(dev)
    z, mu, rs = ln.ln_fwd(g("x"), g("gamma"), g("beta"), 1e-5)
    zo, muo, rso = oln.ln_fwd(x["x"], x["gamma"], x["beta"], 1e-5, D)
    assert_close(z, zo, wd, "z")
    dx, dg, db, _, _ = ln.ln_bwd(g("dy"), g("x"), mu, rs, g("gamma"), None, False)
    dxo, dgo, dbo = oln.ln_bwd(x["dy"], x["x"], muo, rso, x["gamma"], D)
    assert_close(dx, dxo, d, "dx", atol=1e-5 if d == F32 else None)
    assert_close(dg, dgo, wd, "dgamma", scale_atol=True, atol=1e-5 if wd == F32 else None)
    assert_close(db, dbo, wd, "dbeta", scale_atol=True, atol=1e-5 if wd == F32 else None)


def _xentropy(rnd, seed, dev):
    n, v = rnd.choice([1, 3, 17, 64]), rnd.choice([1, 2, 7, 100, 1000, 4099, 32001])
    d, eps = rnd.choice([F32, F16, BF16]), rnd.choice([0.0, 0.1])
    rnd.case = f"cross-entropy N {n} V {v} {d} eps {eps}"
    x = inputs.xentropy_inputs(n, v, d, eps, padding_idx=0, pad_fraction=0.2, seed=seed)
    lo, lse = xe.forward(x["logits"].to(dev), x["labels"].to(dev), eps, d != F32, padding_idx=0)
    loo, lseo = oxe.xentropy_fwd(x["logits"], x["labels"], eps, 0, D)
    assert_close(lo, loo, F32, "losses", rtol=2e-5, atol=2e-5)
    gl = xe.backward(x["grad_loss"].to(dev), x["logits"].to(dev), lse, x["labels"].to(dev), eps, padding_idx=0)
    assert_close(gl, oxe.xentropy_bwd(x["grad_loss"], x["logits"], lseo, x["labels"], eps, 0, D), d, "dlogits", atol=1e-6 if d == F32 else None)
    pad_rows = x["labels"] == 0
    assert (lo.cpu()[pad_rows] == 0).all() and (gl.cpu()[pad_rows] == 0).all()


KINDS = [_gemm, _gemm, _self, _encdec, _mlp, _softmax, _layer_norm, _xentropy]


@pytest.mark.parametrize("seed", SEEDS)
def test_random_shape(dev, seed):
    rnd = random.Random(seed)
    kind = rnd.choice(KINDS)
    try:
        kind(rnd, seed, dev)
    except AssertionError as e:
        raise AssertionError(f"seed {seed}, {getattr(rnd, 'case', kind.__name__)}: {e}") from None
