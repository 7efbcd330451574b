"""Pins the CPU oracle (oracle/) against PyTorch library routines, closed forms, invariants,
brute-force loops and fp64 finite differences. All CPU; nothing here touches the HIP library.

The reference tree stores no golden vectors for these ops (its tests draw random inputs and
compare with PyTorch at run time), so the pins are the routines its fallback reduces to.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import (attention, dropout_add, fused_optim as ofo, generator_loss, inputs, layer_norm, mlp, relative_attention, softmax_dropout,
                    transformer_layers, xentropy)

D = torch.float64


# ------------------------------------------------------------------ LayerNorm
@pytest.mark.parametrize("rows,hidden", [(7, 12), (33, 512), (5, 1000)])
def test_ln_matches_library_and_autograd(rows, hidden):
    d = inputs.layer_norm_inputs(rows, hidden, torch.float64, seed=3)
    x = d["x"].clone().requires_grad_()
    g = d["gamma"].clone().requires_grad_()
    b = d["beta"].clone().requires_grad_()
    z_lib = F.layer_norm(x, (hidden,), g, b, d["eps"])
    z_lib.backward(d["dy"])
    z, mu, rs = layer_norm.ln_fwd(d["x"], d["gamma"], d["beta"], d["eps"], D)
    torch.testing.assert_close(z, z_lib.detach(), rtol=1e-12, atol=1e-12)
    dx, dg, db = layer_norm.ln_bwd(d["dy"], d["x"], mu, rs, d["gamma"], D)
    torch.testing.assert_close(dx, x.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dg, g.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(db, b.grad, rtol=1e-10, atol=1e-12)
    # memory-efficient backward (from z) equals the backward from x
    dx2, dg2, db2 = layer_norm.ln_bwd_memory_efficient(d["dy"], z, rs, d["gamma"], d["beta"], D)
    torch.testing.assert_close(dx2, dx, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(dg2, dg, rtol=1e-9, atol=1e-11)


def test_ln_invariants():
    d = inputs.layer_norm_inputs(16, 64, torch.float64, seed=4)
    ones, zeros = torch.ones(64, dtype=D), torch.zeros(64, dtype=D)
    z, mu, rs = layer_norm.ln_fwd(d["x"], ones, zeros, 0.0, D)
    assert z.mean(1).abs().max() < 1e-12                      # normalised rows have zero mean
    torch.testing.assert_close((z * z).mean(1), torch.ones(16, dtype=D))  # ... and unit variance
    torch.testing.assert_close(mu, d["x"].mean(1))
    torch.testing.assert_close(rs, 1.0 / d["x"].var(1, unbiased=False).sqrt())
    dx, _, _ = layer_norm.ln_bwd(d["dy"], d["x"], mu, rs, ones, D)
    assert dx.sum(1).abs().max() < 1e-10                      # constant gamma: row sums of dx vanish
    # shifting x by a row constant changes nothing
    z2, _, _ = layer_norm.ln_fwd(d["x"] + 3.5, ones, zeros, 0.0, D)
    torch.testing.assert_close(z2, z, rtol=1e-9, atol=1e-10)


# ------------------------------------------------------------------ dropout-add
def test_dropout_add_matches_autograd():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 10, generator=g, dtype=D, requires_grad=True)
    r = torch.randn(6, 10, generator=g, dtype=D, requires_grad=True)
    m = inputs.bernoulli_mask((6, 10), 0.7, g)
    go = torch.randn(6, 10, generator=g, dtype=D)
    out = dropout_add.dropout_add_fwd(x.detach(), r.detach(), m, 0.3, D)
    ref = r + x * m.to(D) / 0.7
    torch.testing.assert_close(out, ref.detach())
    ref.backward(go)
    dx, dr = dropout_add.dropout_add_bwd(go, m, 0.3, D)
    torch.testing.assert_close(dx, x.grad)
    torch.testing.assert_close(dr, r.grad)
    torch.testing.assert_close(dropout_add.dropout_add_fwd(x.detach(), r.detach(), None, 0.0, D), (x + r).detach())
    # all-ones mask at p -> 0 is the plain sum; all-zero mask leaves the residual
    torch.testing.assert_close(dropout_add.dropout_add_fwd(x.detach(), r.detach(), torch.zeros_like(m), 0.3, D), r.detach())


# ------------------------------------------------------------------ masked softmax + dropout
def test_softmax_dropout_matches_library():
    g = torch.Generator().manual_seed(6)
    bh, tq, tk, heads = 6, 5, 9, 3
    s = torch.randn(bh, tq, tk, generator=g, dtype=D)
    pad = torch.zeros(2, tk, dtype=torch.bool)
    pad[0, 6:] = True
    pad[1, 3:] = True
    sm_in = softmax_dropout.masked_scores(s, pad_mask=pad, heads=heads).requires_grad_()
    m = inputs.bernoulli_mask((bh, tq, tk), 0.8, g)
    lib = F.softmax(sm_in, dim=-1)
    lib_dr = lib * m.to(D) / 0.8
    sm, dr = softmax_dropout.softmax_dropout_fwd(sm_in.detach(), m, 0.2, D)
    torch.testing.assert_close(sm, lib.detach())
    torch.testing.assert_close(dr, lib_dr.detach())
    go = torch.randn(bh, tq, tk, generator=g, dtype=D)
    lib_dr.backward(go)
    ds = softmax_dropout.softmax_dropout_bwd(go, sm, m, 0.2, D)
    torch.testing.assert_close(ds, sm_in.grad)
    # masked keys: exactly zero probability and gradient; rows sum to one
    assert (sm.view(2, heads, tq, tk)[0, :, :, 6:] == 0).all() and (ds.view(2, heads, tq, tk)[1, :, :, 3:] == 0).all()
    torch.testing.assert_close(sm.sum(-1), torch.ones(bh, tq, dtype=D))
    assert ds.sum(-1).abs().max() < 1e-12


def test_softmax_fully_masked_row_is_zero_and_time_mask():
    s = torch.randn(2, 4, 4, dtype=D)
    tm = torch.triu(torch.ones(4, 4), 1).bool()
    sm, _ = softmax_dropout.softmax_dropout_fwd(softmax_dropout.masked_scores(s, time_mask=tm), None, 0.0, D)
    assert (sm[:, 0, 1:] == 0).all() and torch.allclose(sm[:, 0, 0], torch.ones(2, dtype=D))
    lib = F.softmax(s.masked_fill(tm, float("-inf")), -1)
    torch.testing.assert_close(sm, lib)
    allmask = torch.full((1, 2, 3), float("-inf"), dtype=D)
    sm0, dr0 = softmax_dropout.softmax_dropout_fwd(allmask, None, 0.0, D)
    assert (sm0 == 0).all() and (dr0 == 0).all()   # the library gives NaN here; the reference zeroes it


# ------------------------------------------------------------------ xentropy
@pytest.mark.parametrize("n,v,eps", [(9, 17, 0.1), (64, 1000, 0.0), (16, 4099, 0.3)])
def test_xentropy_matches_library(n, v, eps):
    d = inputs.xentropy_inputs(n, v, torch.float64, eps, padding_idx=1, pad_fraction=0.25, seed=7)
    x = d["logits"].clone().requires_grad_()
    lib = F.cross_entropy(x, d["labels"], ignore_index=1, reduction="none", label_smoothing=eps)
    loss, lse = xentropy.xentropy_fwd(d["logits"], d["labels"], eps, 1, D)
    torch.testing.assert_close(loss, lib.detach(), rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(lse, torch.logsumexp(d["logits"], 1))
    gl = torch.rand(n, dtype=D) + 0.5
    lib.backward(gl)
    dx = xentropy.xentropy_bwd(gl, d["logits"], lse, d["labels"], eps, 1, D)
    torch.testing.assert_close(dx, x.grad, rtol=1e-10, atol=1e-13)
    pad = d["labels"] == 1
    assert pad.any() and (loss[pad] == 0).all() and (dx[pad] == 0).all()      # exact zeros on padding
    assert dx[~pad].sum(1).abs().max() < 1e-12                                # gradient rows sum to 0


def test_xentropy_closed_forms():
    # the two closed forms the reference's test states (extensions/xentropy/test_xentropy.py:44-62)
    d = inputs.xentropy_inputs(12, 50, torch.float64, 0.1, padding_idx=0, pad_fraction=0.2, seed=8)
    lp = F.log_softmax(d["logits"], -1)
    ll = lp.gather(1, d["labels"].unsqueeze(1)).squeeze(1)
    form = ((0.1 - 1.0) * ll - 0.1 * lp.mean(-1)).masked_fill(d["labels"] == 0, 0)
    loss, _ = xentropy.xentropy_fwd(d["logits"], d["labels"], 0.1, 0, D)
    torch.testing.assert_close(loss, form)
    # eps = 0 reduces to lse - x_y; uniform logits give log V
    loss0, lse0 = xentropy.xentropy_fwd(d["logits"], d["labels"], 0.0, -100, D)
    torch.testing.assert_close(loss0, lse0 - d["logits"].gather(1, d["labels"].unsqueeze(1)).squeeze(1))
    lu, _ = xentropy.xentropy_fwd(torch.zeros(3, 50, dtype=D), torch.tensor([4, 5, 6]), 0.1, -100, D)
    torch.testing.assert_close(lu, torch.full((3,), math.log(50.0), dtype=D))


@pytest.mark.parametrize("bias", [True, False])
def test_generator_loss_matches_library_and_autograd(bias):
    # projection + loss against F.linear -> F.cross_entropy and autograd through both
    g = torch.Generator().manual_seed(77)
    n, e, v, eps, pad = 23, 12, 41, 0.1, 3
    h = torch.randn(n, e, dtype=D, generator=g).requires_grad_()
    w = (torch.randn(v, e, dtype=D, generator=g) * 0.3).requires_grad_()
    b = (torch.randn(v, dtype=D, generator=g) * 0.1).requires_grad_() if bias else None
    y = torch.randint(0, v, (n,), generator=g)
    y[::5] = pad
    gl = torch.rand(n, dtype=D, generator=g) + 0.5
    z = F.linear(h, w, b)
    lib = F.cross_entropy(z, y, ignore_index=pad, reduction="none", label_smoothing=eps)
    lib.backward(gl)
    loss, lse, am = generator_loss.generator_loss_fwd(h.detach(), w.detach(), None if b is None else b.detach(), y, eps, pad, D, D)
    torch.testing.assert_close(loss, lib.detach(), rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(lse, torch.logsumexp(z.detach(), 1))
    assert torch.equal(am, z.detach().argmax(1))
    dh, dw, db = generator_loss.generator_loss_bwd(gl, h.detach(), w.detach(), None if b is None else b.detach(), y, eps, pad, D, D)
    torch.testing.assert_close(dh, h.grad, rtol=1e-10, atol=1e-13)
    torch.testing.assert_close(dw, w.grad, rtol=1e-10, atol=1e-13)
    if bias:
        torch.testing.assert_close(db, b.grad, rtol=1e-10, atol=1e-13)
        assert abs(float(db.sum())) < 1e-12                   # every gradient row of the logits sums to zero
    else:
        assert db is None
    assert (loss[y == pad] == 0).all() and (dh[y == pad] == 0).all()


def test_generator_loss_rounds_the_logits_where_the_reference_stores_them():
    g = torch.Generator().manual_seed(78)
    h, w = torch.randn(8, 16, generator=g).bfloat16(), torch.randn(30, 16, generator=g).bfloat16()
    y = torch.randint(0, 30, (8,), generator=g)
    loss, _, _ = generator_loss.generator_loss_fwd(h, w, None, y, 0.0, -100, torch.bfloat16)
    z = (h.float() @ w.float().t()).bfloat16()
    torch.testing.assert_close(loss, F.cross_entropy(z.float(), y, reduction="none"))


# ------------------------------------------------------------------ MLP
@pytest.mark.parametrize("act", ["relu", "gelu", "silu", "agelu", "none"])
def test_mlp_matches_library_and_autograd(act):
    d = inputs.mlp_inputs(24, 16, 40, torch.float64, p=0.2, seed=9, zero_bias=False)
    x = d["x"].clone().requires_grad_()
    ws = [d["w1"].clone().requires_grad_(), d["w2"].clone().requires_grad_()]
    bs = [d["b1"].clone().requires_grad_(), d["b2"].clone().requires_grad_()]
    h = F.linear(x, ws[0], bs[0])
    lib_act = {"relu": F.relu, "gelu": F.gelu, "silu": F.silu, "none": lambda t: t,
               "agelu": lambda t: F.gelu(t, approximate="tanh")}[act]
    a = lib_act(h) * d["mask"].to(D) / 0.8
    y_lib = F.linear(a, ws[1], bs[1])
    y_lib.backward(d["dy"])
    y, pre, post = mlp.mlp_fwd(d["x"], [d["w1"], d["w2"]], [d["b1"], d["b2"]], act, 0.2, [d["mask"]], D)
    torch.testing.assert_close(y, y_lib.detach(), rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(pre[0], h.detach(), rtol=1e-12, atol=1e-12)
    dx, dws, dbs = mlp.mlp_bwd(d["dy"], d["x"], [d["w1"], d["w2"]], pre, post, act, 0.2, [d["mask"]], D)
    torch.testing.assert_close(dx, x.grad, rtol=1e-9, atol=1e-11)
    for i in range(2):
        torch.testing.assert_close(dws[i], ws[i].grad, rtol=1e-9, atol=1e-11)
        torch.testing.assert_close(dbs[i], bs[i].grad, rtol=1e-9, atol=1e-11)


def test_mlp_three_layers_and_activation_values():
    g = torch.Generator().manual_seed(10)
    x = torch.randn(5, 6, generator=g, dtype=D, requires_grad=True)
    ws = [torch.randn(7, 6, generator=g, dtype=D), torch.randn(4, 7, generator=g, dtype=D), torch.randn(3, 4, generator=g, dtype=D)]
    y_lib = F.linear(F.gelu(F.linear(F.gelu(F.linear(x, ws[0])), ws[1])), ws[2])
    y, pre, post = mlp.mlp_fwd(x.detach(), ws, None, "gelu", 0.0, None, D)
    torch.testing.assert_close(y, y_lib.detach())
    dy = torch.randn(5, 3, generator=g, dtype=D)
    y_lib.backward(dy)
    dx, _, _ = mlp.mlp_bwd(dy, x.detach(), ws, pre, post, "gelu", 0.0, None, D)
    torch.testing.assert_close(dx, x.grad)
    # textbook values
    t = torch.tensor([0.0, 1.0, -1.0], dtype=D)
    torch.testing.assert_close(mlp.act_fwd(t, "gelu"), torch.tensor([0.0, 0.8413447460685429, -0.15865525393145707], dtype=D))
    torch.testing.assert_close(mlp.act_fwd(t, "silu"), torch.tensor([0.0, 0.7310585786300049, -0.2689414213699951], dtype=D))


# ------------------------------------------------------------------ attention
def _deinterleave(w, heads, parts):
    e3 = w.shape[0]
    d = e3 // (heads * parts)
    rest = w.shape[1:]
    v = w.reshape(heads, parts, d, *rest)
    return [v[:, i].reshape(heads * d, *rest) for i in range(parts)]


def test_self_attention_matches_library_mha():
    t, b, e, h = 7, 3, 16, 4
    d = inputs.self_attn_inputs(t, b, e, h, torch.float64, p=0.0, seed=11, min_len=3, zero_bias=False)
    out = attention.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, pad_mask=d["pad_mask"], ctype=D)
    wq, wk, wv = _deinterleave(d["w_in"], h, 3)
    bq, bk, bv = _deinterleave(d["b_in"], h, 3)
    mha = torch.nn.MultiheadAttention(e, h, bias=True, dtype=D)
    with torch.no_grad():
        mha.in_proj_weight.copy_(torch.cat([wq, wk, wv]))
        mha.in_proj_bias.copy_(torch.cat([bq, bk, bv]))
        mha.out_proj.weight.copy_(d["w_out"])
        mha.out_proj.bias.copy_(d["b_out"])
    ref, attn = mha(d["x"], d["x"], d["x"], key_padding_mask=d["pad_mask"], need_weights=True, average_attn_weights=False)
    torch.testing.assert_close(out["outputs"], ref.detach(), rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(out["softmax_results"].view(b, h, t, t), attn.detach(), rtol=1e-10, atol=1e-12)
    # round trip of the weight interleave helper
    torch.testing.assert_close(attention.interleave_qkv(wq, wk, wv, h), d["w_in"])


def test_self_attention_causal_matches_sdpa_and_bruteforce():
    t, b, e, h = 6, 2, 8, 2
    d = inputs.self_attn_inputs(t, b, e, h, torch.float64, p=0.0, seed=12, causal=True, zero_bias=False)
    out = attention.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, time_mask=d["time_mask"], ctype=D)
    lin = out["input_lin_results"].view(t, b, h, 3, e // h)
    q, k, v = [lin[:, :, :, i].permute(1, 2, 0, 3) for i in range(3)]   # [B,H,T,D]
    sd = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    torch.testing.assert_close(out["matmul2_results"], sd.permute(2, 0, 1, 3).reshape(t, b, e), rtol=1e-10, atol=1e-12)
    # brute force one (batch, head, query)
    bi, hi, qi = 1, 1, 3
    dd = e // h
    acc = torch.zeros(dd, dtype=D)
    ws = torch.tensor([math.exp(float(q[bi, hi, qi] @ k[bi, hi, j]) / math.sqrt(dd)) for j in range(qi + 1)], dtype=D)
    for j in range(qi + 1):
        acc += ws[j] / ws.sum() * v[bi, hi, j]
    torch.testing.assert_close(out["matmul2_results"][qi, bi, hi * dd:(hi + 1) * dd], acc, rtol=1e-10, atol=1e-12)


def _self_attn_autograd(d, h, pad=None, tm=None, p=0.0, dm=None):
    """Independent autograd graph built from library ops on de-interleaved weights."""
    t, b, e = d["x"].shape
    dd = e // h
    x = d["x"].clone().requires_grad_()
    ps = [d[k].clone().requires_grad_() for k in ("w_in", "w_out", "b_in", "b_out")]
    lin = F.linear(x, ps[0], ps[2]).view(t, b, h, 3, dd)
    q, k, v = [lin[:, :, :, i].permute(1, 2, 0, 3) for i in range(3)]
    s = q @ k.transpose(-1, -2) / math.sqrt(dd)
    if pad is not None:
        s = s.masked_fill(pad.view(b, 1, 1, t), float("-inf"))
    if tm is not None:
        s = s.masked_fill(tm.view(1, 1, t, t), float("-inf"))
    pr = F.softmax(s, -1)
    if dm is not None:
        pr = pr * dm.view(b, h, t, t).to(D) / (1 - p)
    ctx = (pr @ v).permute(2, 0, 1, 3).reshape(t, b, e)
    out = F.linear(ctx, ps[1], ps[3])
    out.backward(d["dout"])
    return out.detach(), x.grad, [q_.grad for q_ in ps]


@pytest.mark.parametrize("causal,p", [(False, 0.0), (False, 0.25), (True, 0.25)])
def test_self_attention_backward_matches_autograd(causal, p):
    t, b, e, h = 9, 3, 12, 3
    d = inputs.self_attn_inputs(t, b, e, h, torch.float64, p=p, seed=13, min_len=4, causal=causal, zero_bias=False)
    fwd = attention.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"],
                                  p, d["dropout_mask"], D)
    bwd = attention.self_attn_bwd(d["dout"], d["x"], d["w_in"], d["w_out"], h, fwd, p, d["dropout_mask"], D)
    out, dx, (dwi, dwo, dbi, dbo) = _self_attn_autograd(d, h, d["pad_mask"], d["time_mask"], p, d["dropout_mask"])
    torch.testing.assert_close(fwd["outputs"], out, rtol=1e-10, atol=1e-11)
    for name, got, want in (("dx", bwd["dx"], dx), ("dw_in", bwd["dw_in"], dwi), ("dw_out", bwd["dw_out"], dwo),
                            ("db_in", bwd["db_in"], dbi), ("db_out", bwd["db_out"], dbo)):
        torch.testing.assert_close(got, want, rtol=1e-8, atol=1e-10, msg=lambda m, n=name: f"{n}: {m}")


def test_encdec_attention_matches_library_and_autograd():
    tq, tk, b, e, h = 5, 11, 2, 12, 3
    dd = e // h
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, torch.float64, p=0.2, seed=14, zero_bias=False)
    fwd = attention.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], d["b_q"], d["b_kv"], d["b_out"],
                                    h, d["pad_mask"], 0.2, d["dropout_mask"], D)
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out", "b_q", "b_kv", "b_out")
    leaf = {k: d[k].clone().requires_grad_() for k in names}
    q = F.linear(leaf["x_q"], leaf["w_q"], leaf["b_q"]).view(tq, b, h, dd).permute(1, 2, 0, 3)
    kv = F.linear(leaf["x_kv"], leaf["w_kv"], leaf["b_kv"]).view(tk, b, h, 2, dd)
    k, v = kv[:, :, :, 0].permute(1, 2, 0, 3), kv[:, :, :, 1].permute(1, 2, 0, 3)
    s = (q @ k.transpose(-1, -2) / math.sqrt(dd)).masked_fill(d["pad_mask"].view(b, 1, 1, tk), float("-inf"))
    pr = F.softmax(s, -1) * d["dropout_mask"].view(b, h, tq, tk).to(D) / 0.8
    out = F.linear((pr @ v).permute(2, 0, 1, 3).reshape(tq, b, e), leaf["w_out"], leaf["b_out"])
    out.backward(d["dout"])
    torch.testing.assert_close(fwd["outputs"], out.detach(), rtol=1e-10, atol=1e-11)
    bwd = attention.encdec_attn_bwd(d["dout"], d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], h, fwd, 0.2,
                                    d["dropout_mask"], D)
    for k_, n in (("dx_q", "x_q"), ("dx_kv", "x_kv"), ("dw_q", "w_q"), ("dw_kv", "w_kv"), ("dw_out", "w_out"),
                  ("db_q", "b_q"), ("db_kv", "b_kv"), ("db_out", "b_out")):
        torch.testing.assert_close(bwd[k_], leaf[n].grad, rtol=1e-8, atol=1e-10, msg=lambda m, n=k_: f"{n}: {m}")
    # p = 0 cross-check with the library's MultiheadAttention on de-interleaved weights
    fwd0 = attention.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], d["b_q"], d["b_kv"], d["b_out"],
                                     h, d["pad_mask"], 0.0, None, D)
    wk, wv = _deinterleave(d["w_kv"], h, 2)
    bk, bv = _deinterleave(d["b_kv"], h, 2)
    mha = torch.nn.MultiheadAttention(e, h, bias=True, dtype=D)
    with torch.no_grad():
        mha.in_proj_weight.copy_(torch.cat([d["w_q"], wk, wv]))
        mha.in_proj_bias.copy_(torch.cat([d["b_q"], bk, bv]))
        mha.out_proj.weight.copy_(d["w_out"])
        mha.out_proj.bias.copy_(d["b_out"])
    ref, _ = mha(d["x_q"], d["x_kv"], d["x_kv"], key_padding_mask=d["pad_mask"])
    torch.testing.assert_close(fwd0["outputs"], ref.detach(), rtol=1e-10, atol=1e-11)


@pytest.mark.parametrize("causal,p", [(False, 0.0), (False, 0.25), (True, 0.25)])
def test_tiled_core_restatement_matches_autograd_when_nothing_is_rounded(causal, p):
    """core="tiled" regroups the same mathematics (unnormalised exponentials times V, divided by the row sum afterwards;
    dS from D = rowsum(dctx * ctx)): with round_to=None it has to equal autograd through the library's ops, for self- and
    encoder-decoder attention, with a fully masked row among the cases (encoder-decoder inputs mask whole tails)."""
    t, b, e, h = 9, 3, 12, 3
    d = inputs.self_attn_inputs(t, b, e, h, torch.float64, p=p, seed=13, min_len=4, causal=causal, zero_bias=False)
    fwd = attention.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"],
                                  p, d["dropout_mask"], D, core="tiled")
    bwd = attention.self_attn_bwd(d["dout"], d["x"], d["w_in"], d["w_out"], h, fwd, p, d["dropout_mask"], D, core="tiled")
    out, dx, (dwi, dwo, dbi, dbo) = _self_attn_autograd(d, h, d["pad_mask"], d["time_mask"], p, d["dropout_mask"])
    torch.testing.assert_close(fwd["outputs"], out, rtol=1e-10, atol=1e-11)
    for name, got, want in (("dx", bwd["dx"], dx), ("dw_in", bwd["dw_in"], dwi), ("dw_out", bwd["dw_out"], dwo),
                            ("db_in", bwd["db_in"], dbi), ("db_out", bwd["db_out"], dbo)):
        torch.testing.assert_close(got, want, rtol=1e-8, atol=1e-10, msg=lambda m, n=name: f"{n}: {m}")
    tq, tk = 5, 11
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, torch.float64, p=p, seed=14, zero_bias=False)
    args = (d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"])
    res = {}
    for core in ("stored", "tiled"):
        f = attention.encdec_attn_fwd(*args, d["b_q"], d["b_kv"], d["b_out"], h, d["pad_mask"], p, d["dropout_mask"], D, core=core)
        res[core] = (f, attention.encdec_attn_bwd(d["dout"], *args, h, f, p, d["dropout_mask"], D, core=core))
    torch.testing.assert_close(res["tiled"][0]["outputs"], res["stored"][0]["outputs"], rtol=1e-10, atol=1e-11)
    for key, want in res["stored"][1].items():
        torch.testing.assert_close(res["tiled"][1][key], want, rtol=1e-8, atol=1e-10, msg=lambda m, n=key: f"{n}: {m}")


def test_tiled_core_restatement_rounds_only_operands_and_results():
    """With round_to=bf16 the two restatements differ by roundings only: the tiled one keeps scores and statistics exact,
    so its context is the closer of the two to the unrounded one, and a single key (probability exactly 1, dropout scale
    1 / (1 - p) applied in full precision at the end) gives round(v / (1 - p)) rather than round(round(1 / (1 - p)) v)."""
    t, b, e, h, p = 40, 2, 64, 2, 0.25
    d = inputs.self_attn_inputs(t, b, e, h, torch.bfloat16, p=p, seed=21, zero_bias=False)
    kw = dict(pad_mask=d["pad_mask"], p=p, dropout_mask=d["dropout_mask"], ctype=D)
    a = (d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h)
    exact = attention.self_attn_fwd(*a, **kw)["matmul2_results"]
    err = {c: (attention.self_attn_fwd(*a, **kw, round_to=torch.bfloat16, core=c)["matmul2_results"] - exact).abs().mean()
           for c in ("stored", "tiled")}
    assert err["tiled"] < err["stored"]
    q = torch.randn(1, 1, 8, dtype=D)
    v = torch.randn(1, 1, 8, dtype=D).to(torch.bfloat16).to(D)
    keep = torch.ones(1, 1, 1, dtype=torch.bool)
    _, prob, _, ctx = attention._core_fwd_tiled(q, q, v, 1, None, None, p, keep, D, torch.bfloat16)
    assert prob.item() == 1.0
    assert torch.equal(ctx, (v / (1 - p)).to(torch.bfloat16).to(D))


def test_attention_finite_differences():
    # the reference validates its hand-written backward with fp64 gradcheck on tiny shapes
    t, b, e, h = 4, 2, 8, 2
    d = inputs.self_attn_inputs(t, b, e, h, torch.float64, p=0.0, seed=15, min_len=2, zero_bias=False)
    fwd = attention.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], ctype=D)
    bwd = attention.self_attn_bwd(d["dout"], d["x"], d["w_in"], d["w_out"], h, fwd, ctype=D)
    f = lambda x_: (attention.self_attn_fwd(x_, d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], ctype=D)["outputs"] * d["dout"]).sum()
    eps = 1e-6
    for idx in [(0, 0, 0), (2, 1, 5), (3, 0, 7)]:
        xp, xm = d["x"].clone(), d["x"].clone()
        xp[idx] += eps
        xm[idx] -= eps
        fd = (f(xp) - f(xm)) / (2 * eps)
        assert abs(float(fd) - float(bwd["dx"][idx])) < 1e-6 * max(1.0, abs(float(fd)))


# ------------------------------------------------------------------ relative-position self-attention
@pytest.mark.parametrize("b,tq,r", [(2, 5, 5), (1, 4, 9), (3, 7, 8), (1, 1, 1)])
def test_relative_shift_index_arithmetic_and_adjoint(b, tq, r):
    g = torch.Generator().manual_seed(tq * 31 + r)
    x = torch.randn(b, tq, r, generator=g, dtype=D)
    got = relative_attention.relative_shift(x)
    want = torch.zeros_like(x)
    for n in range(b):                       # the closed form of the pad / view / drop / view sequence, element by element
        for i in range(tq):
            for j in range(r):
                p = i * r + j + tq
                i2, c = divmod(p, r + 1)
                want[n, i, j] = 0.0 if c == 0 else x[n, i2, c - 1]
    assert torch.equal(got, want)
    # the adjoint: <shift(x), y> == <x, shift_bwd(y)>, and autograd of the forward agrees
    y = torch.randn(b, tq, r, generator=g, dtype=D)
    back = relative_attention.relative_shift_bwd(y)
    torch.testing.assert_close((got * y).sum(), (x * back).sum(), rtol=1e-12, atol=1e-12)
    xa = x.clone().requires_grad_()
    relative_attention.relative_shift(xa).backward(y)
    assert torch.equal(back, xa.grad)


def test_relative_shift_aligns_distances_on_and_below_the_diagonal():
    # what the shift is for (Transformer-XL): with R = T positions ordered from distance T-1 down to 0, the score of
    # query i against key j <= i is the one computed against the position of distance i - j
    t = 6
    x = torch.arange(2 * t * t, dtype=D).view(2, t, t)
    got = relative_attention.relative_shift(x)
    for i in range(t):
        for j in range(i + 1):
            assert torch.equal(got[:, i, j], x[:, i, t - 1 - (i - j)])
        if i + 1 < t:
            assert (got[:, i, i + 1] == 0).all()          # the padded zero lands just above the diagonal


def _rel_direct(d, h):
    """Per-element Transformer-XL definition under a causal mask (only j <= i is looked at)."""
    x, pos = d["x"].to(D), d["pos"].to(D)
    t, b, e = x.shape
    dh = e // h
    lin = (x.reshape(t * b, e) @ d["w_in"].to(D).t() + d["b_in"].to(D)).view(t, b, h, 3, dh)
    rk = (pos[:, 0] @ d["w_pos"].to(D).t() + d["b_pos"].to(D)).view(-1, h, dh)        # [R, H, D], R == T
    u, vb = d["r_w_bias"].to(D), d["r_r_bias"].to(D)
    out = torch.zeros(t, b, e, dtype=D)
    for n in range(b):
        for hh in range(h):
            q, k, v = lin[:, n, hh, 0], lin[:, n, hh, 1], lin[:, n, hh, 2]
            for i in range(t):
                s = torch.stack([((q[i] + u[hh]) @ k[j] + (q[i] + vb[hh]) @ rk[t - 1 - (i - j), hh]) * dh ** -0.5
                                 for j in range(i + 1)])
                out[i, n, hh * dh:(hh + 1) * dh] = torch.softmax(s, 0) @ v[:i + 1]
    return (out.reshape(t * b, e) @ d["w_out"].to(D).t() + d["b_out"].to(D)).view(t, b, e)


def test_relative_attention_forward_matches_the_per_element_definition():
    d = inputs.rel_self_attn_inputs(7, 2, 24, 3, torch.float64, p=0.0, seed=5, causal=True)
    f = relative_attention.rel_self_attn_fwd(d["x"], d["pos"], d["w_in"], d["w_out"], d["w_pos"], d["b_in"], d["b_out"],
                                             d["b_pos"], d["r_w_bias"], d["r_r_bias"], 3, None, d["time_mask"], 0.0, None, D)
    torch.testing.assert_close(f["outputs"], _rel_direct(d, 3), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("causal,p,len_r,pos_batch", [(False, 0.0, None, 1), (False, 0.25, 13, 1), (True, 0.25, None, 2)])
def test_relative_attention_backward_matches_autograd(causal, p, len_r, pos_batch):
    h = 2
    d = inputs.rel_self_attn_inputs(9, 2, 16, h, torch.float64, p=p, seed=6, len_r=len_r, pos_batch=pos_batch, causal=causal)
    names = ("x", "pos", "w_in", "w_out", "w_pos", "b_in", "b_out", "b_pos", "r_w_bias", "r_r_bias")
    leaves = {k: d[k].clone().requires_grad_() for k in names}
    fa = relative_attention.rel_self_attn_fwd(*(leaves[k] for k in names), h, d["pad_mask"], d["time_mask"], p,
                                              d["dropout_mask"], D)
    fa["outputs"].backward(d["dout"])
    f = relative_attention.rel_self_attn_fwd(*(d[k] for k in names), h, d["pad_mask"], d["time_mask"], p, d["dropout_mask"], D)
    g = relative_attention.rel_self_attn_bwd(d["dout"], d["x"], d["pos"], d["w_in"], d["w_out"], d["w_pos"], h, f, p,
                                             d["dropout_mask"], D)
    for k, gk in (("x", "dx"), ("w_in", "dw_in"), ("w_out", "dw_out"), ("w_pos", "dw_pos"), ("b_in", "db_in"),
                  ("b_out", "db_out"), ("b_pos", "db_pos"), ("r_w_bias", "dr_w_bias"), ("r_r_bias", "dr_r_bias")):
        torch.testing.assert_close(g[gk], leaves[k].grad, rtol=1e-9, atol=1e-10, msg=lambda m, k=k: f"{k}: {m}")
    if pos_batch == 1:            # the position states are shared over the batch: their gradient sums over it
        assert leaves["pos"].grad.shape == d["pos"].shape


def test_learnable_position_attention_matches_the_per_element_definition_and_autograd():
    h, t, b, e = 2, 6, 2, 16
    dh = e // h
    d = inputs.self_attn_inputs(t, b, e, h, torch.float64, p=0.25, seed=11, zero_bias=False)
    g = torch.Generator().manual_seed(12)
    pos = torch.randn(t, t, dh, generator=g, dtype=D)
    # forward, no dropout, no mask: out[i] = softmax_j((q_i . k_j + q_i . pos[i][j]) / sqrt(D)) v_j per (batch, head)
    f0 = relative_attention.rel_learnable_attn_fwd(d["x"], pos, d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, None, None, 0.0,
                                                   None, D)
    lin = (d["x"].reshape(t * b, e) @ d["w_in"].t() + d["b_in"]).view(t, b, h, 3, dh)
    want = torch.zeros(t, b, e, dtype=D)
    for n in range(b):
        for hh in range(h):
            q, k, v = lin[:, n, hh, 0], lin[:, n, hh, 1], lin[:, n, hh, 2]
            for i in range(t):
                s = torch.stack([(q[i] @ k[j] + q[i] @ pos[i, j]) * dh ** -0.5 for j in range(t)])
                want[i, n, hh * dh:(hh + 1) * dh] = torch.softmax(s, 0) @ v
    want = (want.reshape(t * b, e) @ d["w_out"].t() + d["b_out"]).view(t, b, e)
    torch.testing.assert_close(f0["outputs"], want, rtol=1e-10, atol=1e-10)
    # backward with key padding and dropout against autograd
    names = ("x", "w_in", "w_out", "b_in", "b_out")
    leaves = {k: d[k].clone().requires_grad_() for k in names}
    pl = pos.clone().requires_grad_()
    fa = relative_attention.rel_learnable_attn_fwd(leaves["x"], pl, leaves["w_in"], leaves["w_out"], leaves["b_in"],
                                                   leaves["b_out"], h, d["pad_mask"], None, 0.25, d["dropout_mask"], D)
    fa["outputs"].backward(d["dout"])
    f = relative_attention.rel_learnable_attn_fwd(d["x"], pos, d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"],
                                                  None, 0.25, d["dropout_mask"], D)
    gr = relative_attention.rel_learnable_attn_bwd(d["dout"], d["x"], pos, d["w_in"], d["w_out"], h, f, 0.25, d["dropout_mask"], D)
    for k, gk in (("x", "dx"), ("w_in", "dw_in"), ("w_out", "dw_out"), ("b_in", "db_in"), ("b_out", "db_out")):
        torch.testing.assert_close(gr[gk], leaves[k].grad, rtol=1e-9, atol=1e-10, msg=lambda m, k=k: f"{k}: {m}")
    torch.testing.assert_close(gr["dpos"], pl.grad, rtol=1e-9, atol=1e-10)


# ------------------------------------------------------------------ multi-tensor optimizer passes
@pytest.mark.parametrize("adamw,wd,bias_correction", [(True, 0.01, True), (False, 0.01, True), (True, 0.0, True)])
def test_adam_step_matches_torch_optimizers(adamw, wd, bias_correction):
    g = torch.Generator().manual_seed(17)
    p0 = torch.randn(37, 5, generator=g, dtype=D)
    ref = p0.clone().requires_grad_()
    opt = (torch.optim.AdamW if adamw else torch.optim.Adam)([ref], lr=3e-3, betas=(0.9, 0.98), eps=1e-8, weight_decay=wd)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step in range(1, 5):
        grad = torch.randn(37, 5, generator=g, dtype=D)
        ref.grad = grad.clone()
        opt.step()
        p, m, v = ofo.adam_step(grad, p, m, v, 3e-3, 0.9, 0.98, 1e-8, step, 1 if adamw else 0, bias_correction, wd, D)
        # torch applies eps after dividing sqrt(v) by sqrt(c2), the same quantity; AdamW decays p by (1 - lr wd) first,
        # which equals subtracting lr wd p computed from the old p
        torch.testing.assert_close(p, ref.detach(), rtol=1e-12, atol=1e-14)
    # without bias correction the first step divides by 1: update = (1 - beta1) g / (sqrt((1 - beta2) g^2) + eps)
    gr = torch.tensor([2.0, -3.0], dtype=D)
    pn, _, _ = ofo.adam_step(gr, torch.zeros(2, dtype=D), torch.zeros(2, dtype=D), torch.zeros(2, dtype=D), 0.1, 0.9, 0.99, 0.0, 1,
                             1, False, 0.0, D)
    torch.testing.assert_close(pn, -0.1 * 0.1 * gr / (0.1 * gr.abs()), rtol=1e-12, atol=0)


def test_scale_and_l2norm_match_library_routines():
    g = torch.Generator().manual_seed(18)
    xs = [torch.randn(n, generator=g, dtype=D) for n in (1, 77, 4096, 0, 300)]
    total, each = ofo.l2norm(xs, D)
    torch.testing.assert_close(total, torch.linalg.vector_norm(torch.cat(xs)), rtol=1e-12, atol=0)
    torch.testing.assert_close(each, torch.stack([torch.linalg.vector_norm(x) for x in xs]), rtol=1e-12, atol=0)
    y, bad = ofo.scale(xs[1], 0.25, D)
    assert torch.equal(y, xs[1] * 0.25) and not bad
    for poison in (float("inf"), float("-inf"), float("nan")):
        x = xs[1].clone()
        x[5] = poison
        assert ofo.scale(x, 0.25, D)[1]


def _layer_params_from_torch(layer, heads, decoder):
    """nn.Transformer{En,De}coderLayer weights under the reference's key names and layouts."""
    sd = {k: v.detach() for k, v in layer.state_dict().items()}
    e = sd["norm1.weight"].numel()
    p = {}

    def ln(dst, src):
        p[dst + ".layer_norm.function.weight"], p[dst + ".layer_norm.function.bias"] = sd[src + ".weight"], sd[src + ".bias"]

    def self_attn(dst, src):
        w, b = sd[src + ".in_proj_weight"], sd[src + ".in_proj_bias"]
        p[dst + ".in_proj_weight"] = attention.interleave_qkv(w[:e], w[e:2 * e], w[2 * e:], heads)
        p[dst + ".in_proj_bias"] = attention.interleave_qkv(b[:e], b[e:2 * e], b[2 * e:], heads)
        p[dst + ".out_proj_weight"], p[dst + ".out_proj_bias"] = sd[src + ".out_proj.weight"], sd[src + ".out_proj.bias"]

    ln("preprocess_attn", "norm1")
    self_attn("multihead_tgt" if decoder else "multihead", "self_attn")
    if decoder:
        ln("preprocess_src_attn", "norm2")
        w, b = sd["multihead_attn.in_proj_weight"], sd["multihead_attn.in_proj_bias"]
        p["multihead_src.in_proj_weight_q"], p["multihead_src.in_proj_bias_q"] = w[:e], b[:e]
        p["multihead_src.in_proj_weight_kv"] = attention.interleave_kv(w[e:2 * e], w[2 * e:], heads)
        p["multihead_src.in_proj_bias_kv"] = attention.interleave_kv(b[e:2 * e], b[2 * e:], heads)
        p["multihead_src.out_proj_weight"], p["multihead_src.out_proj_bias"] = sd["multihead_attn.out_proj.weight"], sd["multihead_attn.out_proj.bias"]
    ln("preprocess_ffn", "norm3" if decoder else "norm2")
    p["feedforward.in_proj_weight"], p["feedforward.in_proj_bias"] = sd["linear1.weight"], sd["linear1.bias"]
    p["feedforward.out_proj_weight"], p["feedforward.out_proj_bias"] = sd["linear2.weight"], sd["linear2.bias"]
    return p


def test_layer_oracle_matches_torch_modules():
    # pre-norm residual blocks: the composition is PyTorch's own norm_first Transformer layer
    t, tk, b, e, h, inner = 9, 11, 3, 16, 4, 40
    g = torch.Generator().manual_seed(71)
    x = torch.randn(t, b, e, generator=g, dtype=D)
    ctxt = torch.randn(tk, b, e, generator=g, dtype=D)
    pad, _ = inputs.lengths_mask(b, t, 4, t, g)
    src_pad, _ = inputs.lengths_mask(b, tk, 5, tk, g)
    causal = torch.triu(torch.ones(t, t), 1).bool()
    torch.manual_seed(72)
    enc = torch.nn.TransformerEncoderLayer(e, h, inner, dropout=0.0, activation="gelu", norm_first=True, dtype=D)
    dec = torch.nn.TransformerDecoderLayer(e, h, inner, dropout=0.0, activation="gelu", norm_first=True, dtype=D)
    for m in list(enc.modules()) + list(dec.modules()):          # biases and LayerNorm affines away from 0 / 1
        for name, prm in m.named_parameters(recurse=False):
            if prm.dim() == 1:
                prm.data.add_(0.1 * torch.randn(prm.shape, generator=g, dtype=D))
    want = enc(x, src_key_padding_mask=pad)
    got = transformer_layers.encoder_layer(x, _layer_params_from_torch(enc, h, False), h, pad, act="gelu")
    torch.testing.assert_close(got, want.detach(), rtol=1e-10, atol=1e-10)
    want = dec(x, ctxt, tgt_mask=causal, memory_key_padding_mask=src_pad)
    got, cov = transformer_layers.decoder_layer(x, ctxt, _layer_params_from_torch(dec, h, True), h, causal, src_pad, act="gelu")
    torch.testing.assert_close(got, want.detach(), rtol=1e-10, atol=1e-10)
    assert cov.shape == (b * h, t, tk) and torch.allclose(cov.sum(-1), torch.ones(b * h, t, dtype=D))
    # the scale factors: macaron halves both feed-forward blocks, a surviving layer is scaled by 1 / (1 - death_rate)
    p = _layer_params_from_torch(enc, h, False)
    base = transformer_layers.encoder_layer(x, p, h, pad, act="gelu")
    scaled = transformer_layers.encoder_layer(x, p, h, pad, act="gelu", death_rate=0.5, training=True)
    assert not torch.allclose(base, scaled)
    assert torch.allclose(transformer_layers.encoder_layer(x, p, h, pad, act="gelu", death_rate=0.5, training=False), base)
    # death_rate = 0.5 doubles each residual branch: check against the hand composition on the first branch only
    zero_ffn = dict(p)
    zero_ffn["feedforward.out_proj_weight"] = torch.zeros_like(p["feedforward.out_proj_weight"])
    zero_ffn["feedforward.out_proj_bias"] = torch.zeros_like(p["feedforward.out_proj_bias"])
    a1 = transformer_layers.encoder_layer(x, zero_ffn, h, pad, act="gelu") - x
    a2 = transformer_layers.encoder_layer(x, zero_ffn, h, pad, act="gelu", death_rate=0.5, training=True) - x
    torch.testing.assert_close(a2, 2 * a1, rtol=1e-10, atol=1e-12)
    # macaron: with the macaron block a copy of the feed-forward block and the attention silenced,
    # y = x + 0.5 F(x) followed by + 0.5 F(.) again
    mac = dict(zero_ffn)
    for k in list(p):
        if k.startswith("feedforward."):
            mac[k] = p[k]
            mac[k.replace("feedforward.", "mcr_feedforward.")] = p[k]
        if k.startswith("preprocess_ffn."):
            mac[k.replace("preprocess_ffn.", "preprocess_mcr_ffn.")] = p[k]
    mac["multihead.out_proj_weight"] = torch.zeros_like(p["multihead.out_proj_weight"])
    mac["multihead.out_proj_bias"] = torch.zeros_like(p["multihead.out_proj_bias"])
    half = lambda z: z + 0.5 * (transformer_layers.encoder_layer(z, dict(mac, **{"multihead.out_proj_weight": mac["multihead.out_proj_weight"]}), h, pad, act="gelu", macaron=False) - z)
    got = transformer_layers.encoder_layer(x, mac, h, pad, act="gelu", macaron=True)
    torch.testing.assert_close(got, half(half(x)), rtol=1e-10, atol=1e-12)


def test_layer_oracle_with_the_tiled_core_differentiates_to_the_same_gradients():
    """attn_core="tiled" routes the self-attention through an autograd node whose backward is written out (the kernels'
    formulation); nothing rounded, a whole layer's gradients have to equal those of plain autograd."""
    t, b, e, h, inner = 9, 3, 16, 4, 40
    g = torch.Generator().manual_seed(73)
    torch.manual_seed(74)
    dec = torch.nn.TransformerDecoderLayer(e, h, inner, dropout=0.0, activation="gelu", norm_first=True, dtype=D)
    params = _layer_params_from_torch(dec, h, True)
    x0 = torch.randn(t, b, e, generator=g, dtype=D)
    c0 = torch.randn(11, b, e, generator=g, dtype=D)
    dy = torch.randn(t, b, e, generator=g, dtype=D)
    causal = torch.triu(torch.ones(t, t), 1).bool()
    src_pad, _ = inputs.lengths_mask(b, 11, 5, 11, g)
    grads = {}
    for core in ("stored", "tiled"):
        x, c = x0.clone().requires_grad_(), c0.clone().requires_grad_()
        prm = {k: v.detach().clone().requires_grad_() for k, v in params.items()}
        y, _ = transformer_layers.decoder_layer(x, c, prm, h, causal, src_pad, act="gelu", attn_core=core)
        y.backward(dy)
        grads[core] = [y.detach(), x.grad, c.grad] + [prm[k].grad for k in sorted(prm)]
    for a, bb in zip(grads["stored"], grads["tiled"]):
        torch.testing.assert_close(a, bb, rtol=1e-9, atol=1e-11)


def test_zipf_targets_and_masks_are_seeded():
    a = inputs.xentropy_inputs(2000, 1000, with_logits=False, seed=1)
    b = inputs.xentropy_inputs(2000, 1000, with_logits=False, seed=1)
    assert torch.equal(a["labels"], b["labels"])
    assert int((a["labels"] == 1).sum()) >= 200
    assert a["labels"].min() >= 0 and a["labels"].max() < 1000
    # heavy head: rank-0 id is the most frequent non-pad target
    counts = torch.bincount(a["labels"], minlength=1000)
    counts[1] = 0
    assert int(counts.argmax()) == 0


# ----------------------------------------------------------------------------- rotary position encoding
def test_rotary_rotation_is_orthogonal_relative_and_its_backward_is_the_transpose():
    from oracle import rotary as orot
    g = torch.Generator().manual_seed(401)
    t, n, d = 9, 3, 16
    cos, sin = orot.tables(torch.arange(t), d)
    x = torch.randn(t, n, d, generator=g, dtype=D)
    y = orot.apply_rotary(x, cos, sin)
    h = d // 2
    # a plane rotation of every pair (j, j + D/2): the pair's norm is kept, and by hand for one element
    assert torch.allclose(x[..., :h] ** 2 + x[..., h:] ** 2, y[..., :h] ** 2 + y[..., h:] ** 2, atol=1e-12)
    i, j = 4, 3
    want = x[i, 1, j] * cos[i, 0, j] - x[i, 1, j + h] * sin[i, 0, j]
    assert abs(y[i, 1, j] - want) < 1e-12
    want = x[i, 1, j + h] * cos[i, 0, j + h] + x[i, 1, j] * sin[i, 0, j + h]
    assert abs(y[i, 1, j + h] - want) < 1e-12
    # the property rotary encodings exist for: <rot(q, m), rot(k, n)> depends on m - n only
    q, k = torch.randn(d, generator=g, dtype=D), torch.randn(d, generator=g, dtype=D)
    rq = orot.apply_rotary(q.expand(t, 1, d), cos, sin)[:, 0]
    rk = orot.apply_rotary(k.expand(t, 1, d), cos, sin)[:, 0]
    s = rq @ rk.t()
    for delta in (0, 1, 3):
        diag = torch.diagonal(s, -delta)
        assert torch.allclose(diag, diag[0].expand_as(diag), atol=1e-10)
    assert not torch.allclose(torch.diagonal(s, 0)[0], torch.diagonal(s, -1)[0])
    # the gradient rule of the reference is the transpose of the forward map: <A x, g> == <x, A^T g>, and autograd agrees
    gr = torch.randn(t, n, d, generator=g, dtype=D)
    assert abs((y * gr).sum() - (x * orot.apply_rotary_transposed(gr, cos, sin)).sum()) < 1e-10
    xr = x.clone().requires_grad_()
    orot.apply_rotary(xr, cos, sin).backward(gr)
    assert torch.allclose(xr.grad, orot.apply_rotary_transposed(gr, cos, sin), atol=1e-12)


def test_rotary_attention_reduces_to_plain_attention_at_angle_zero_and_to_a_per_head_loop():
    from oracle import rotary as orot
    d_in = inputs.self_attn_inputs(12, 2, 32, 2, torch.float32, p=0.0, seed=402, zero_bias=False)
    x, w_in, w_out, b_in, b_out = (d_in[k].to(D) for k in ("x", "w_in", "w_out", "b_in", "b_out"))
    one, zero = torch.ones(12, 1, 16, dtype=D), torch.zeros(12, 1, 16, dtype=D)
    # angle zero: the plain attention oracle (itself pinned against nn.MultiheadAttention above)
    out, cov = orot.self_attn_rotary(x, w_in, w_out, b_in, b_out, 2, d_in["pad_mask"], None, one, zero)
    plain = attention.self_attn_fwd(x, w_in, w_out, b_in, b_out, 2, d_in["pad_mask"], None, 0.0, None, D)
    assert torch.allclose(out, plain["outputs"], atol=1e-12) and torch.allclose(cov, plain["dropout_results"], atol=1e-12)
    # one (batch, head) by hand: rotate its queries and keys, softmax(q k^T / sqrt(D)) v, against the batched form
    cos, sin = orot.tables(torch.arange(12), 16)
    out2, cov2 = orot.self_attn_rotary(x, w_in, w_out, b_in, b_out, 2, None, None, cos, sin)
    lin = (x.reshape(24, 32) @ w_in.t() + b_in).view(12, 2, 2, 3, 16)        # [T, B, H, {q,k,v}, D]
    b_i, h_i = 1, 0
    q = orot.apply_rotary(lin[:, b_i, h_i, 0][:, None], cos, sin)[:, 0]
    k = orot.apply_rotary(lin[:, b_i, h_i, 1][:, None], cos, sin)[:, 0]
    probs = torch.softmax(q @ k.t() / 4.0, -1)
    assert torch.allclose(cov2[b_i * 2 + h_i], probs, atol=1e-12)
    ctx = (out2 - b_out).reshape(24, 32) @ torch.linalg.inv(w_out.t())         # undo the output projection
    assert torch.allclose(ctx.view(12, 2, 2, 16)[:, b_i, h_i], probs @ lin[:, b_i, h_i, 2], atol=1e-9)
    # the cross-attention form rotates queries and keys with their own tables
    de = inputs.encdec_attn_inputs(5, 9, 2, 32, 2, torch.float32, p=0.0, seed=403, zero_bias=False)
    cq, sq = orot.tables(torch.arange(5), 16)
    ck, sk = orot.tables(torch.arange(9), 16)
    oe, ce = orot.encdec_attn_rotary(de["x_q"], de["x_kv"], de["w_q"], de["w_kv"], de["w_out"], 2, None, cq, sq, ck, sk)
    ql = (de["x_q"].to(D).reshape(10, 32) @ de["w_q"].to(D).t()).view(5, 2, 2, 16)
    kl = (de["x_kv"].to(D).reshape(18, 32) @ de["w_kv"].to(D).t()).view(9, 2, 2, 2, 16)
    q = orot.apply_rotary(ql[:, 0, 1][:, None], cq, sq)[:, 0]
    k = orot.apply_rotary(kl[:, 0, 1, 0][:, None], ck, sk)[:, 0]
    assert torch.allclose(ce[1], torch.softmax(q @ k.t() / 4.0, -1), atol=1e-12)


# ----------------------------------------------------------------------------- attention over packed sequences
def _packed_case(seed, lq, lk, heads=2, d=8):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(sum(lq), heads, d, generator=g, dtype=D)
    k = torch.randn(sum(lk), heads, d, generator=g, dtype=D)
    v = torch.randn(sum(lk), heads, d, generator=g, dtype=D)
    do = torch.randn(sum(lq), heads, d, generator=g, dtype=D)
    cu = lambda n: torch.tensor([0] + list(torch.cumsum(torch.tensor(n), 0)), dtype=torch.int32)
    return q, k, v, do, cu(lq), cu(lk)


@pytest.mark.parametrize("causal", [False, True])
def test_packed_attention_is_library_attention_on_every_sequence_by_itself(causal):
    from oracle import flash_attention as ofa
    lq = lk = [5, 1, 9]                                     # causal in the library aligns the first tokens too
    q, k, v, do, cu_q, cu_k = _packed_case(501, lq, lk)
    scale = 0.37
    out, lse = ofa.flash_attn_fwd(q, k, v, cu_q, cu_k, max(lq), scale, causal)
    dq, dk, dv, delta = ofa.flash_attn_bwd(do, q, k, v, cu_q, cu_k, max(lq), scale, causal)
    for b in range(3):
        sq, sk = slice(int(cu_q[b]), int(cu_q[b + 1])), slice(int(cu_k[b]), int(cu_k[b + 1]))
        qb, kb, vb = (t.transpose(0, 1).clone().requires_grad_() for t in (q[sq], k[sk], v[sk]))       # [H, L, D]
        lib = F.scaled_dot_product_attention(qb, kb, vb, is_causal=causal, scale=scale)
        lib.backward(do[sq].transpose(0, 1))
        assert torch.allclose(out[sq].transpose(0, 1), lib.detach(), atol=1e-12)
        assert torch.allclose(dq[sq].transpose(0, 1), qb.grad, atol=1e-12)
        assert torch.allclose(dk[sk].transpose(0, 1), kb.grad, atol=1e-12)
        assert torch.allclose(dv[sk].transpose(0, 1), vb.grad, atol=1e-12)
        s = torch.einsum("hid,hjd->hij", qb.detach(), kb.detach()) * scale
        if causal:
            s = s.masked_fill(torch.ones(lq[b], lk[b], dtype=torch.bool).triu(1), -math.inf)
        assert torch.allclose(lse[b, :, :lq[b]], torch.logsumexp(s, -1), atol=1e-12)
        assert bool((lse[b, :, lq[b]:] == 0).all())
        # D = rowsum(dO * O) = rowsum(P * dP): the identity the backward kernels rest on
        dp = torch.einsum("hid,hjd->hij", do[sq].transpose(0, 1), vb.detach())
        assert torch.allclose(delta[b, :, :lq[b]], (torch.softmax(s, -1) * dp).sum(-1), atol=1e-12)


@pytest.mark.parametrize("causal,p", [(False, 0.0), (True, 0.25)])
def test_packed_attention_written_out_backward_equals_autograd(causal, p):
    """The backward as the kernels compute it (dS = P (keep dP / (1 - p) - D) with D = rowsum(dO O)) against autograd of
    the forward, nothing rounded; an empty sequence and unequal lengths among the cases."""
    from oracle import flash_attention as ofa
    lq, lk = ([3, 6, 4], [5, 0, 7]) if not causal else ([3, 6, 4], [3, 6, 4])
    q, k, v, do, cu_q, cu_k = _packed_case(503, lq, lk)
    keep = (torch.rand(3, 2, max(lq), max(lk), generator=torch.Generator().manual_seed(8)) < 0.75).to(torch.uint8)
    a = ofa.flash_attn_bwd(do, q, k, v, cu_q, cu_k, max(lq), 0.3, causal, p, keep, explicit=False)
    b = ofa.flash_attn_bwd(do, q, k, v, cu_q, cu_k, max(lq), 0.3, causal, p, keep, explicit=True)
    for x, y in zip(a, b):
        assert torch.allclose(x, y, atol=1e-12)


def test_tiled_operand_is_the_softmax_numerator_under_a_moving_reference_point():
    """Unrounded, operand / l is the softmax whatever the reference points were (rows whose maximum sits in a late tile
    and exceeds the first tile's by more than 2^8, rows that start with masked tiles, a row without a live key); rounded,
    every entry is a 16-bit value times the reference shift, i.e. the rounding was applied to exp2(s2 - m_tile): dividing
    the shift back out leaves exactly representable numbers."""
    g = torch.Generator().manual_seed(9)
    s = torch.randn(2, 5, 200, generator=g, dtype=D)
    s[0, 0, 150] += 12.0                    # a late maximum beyond the lazy threshold: the reference point moves at tile 2
    s[0, 1, 70] += 3.0                      # a late maximum below it: the reference point stays
    s[1, 2, :130] = -math.inf               # the first two tiles masked: the reference point is set in the third
    s[1, 3, :] = -math.inf                  # no live key at all
    keep = torch.ones_like(s)
    op, l = attention.tiled_operand(s, keep, None)
    want = torch.softmax(s, -1)
    want[1, 3] = 0
    got = torch.where(l > 0, op / l, torch.zeros_like(op))
    assert torch.allclose(got, want, atol=1e-14)
    assert l[1, 3].item() == 0 and bool((op[1, 3] == 0).all())
    opr, lr = attention.tiled_operand(s, keep, torch.bfloat16)
    assert torch.equal(lr, l)                                                  # the row sum is formed before the rounding
    rel = ((opr - op).abs() / op.clamp_min(1e-300))[op > 0]
    assert rel.max() <= 2.0 ** -8 + 1e-12 and rel.mean() > 2.0 ** -12           # half a unit of an 8-bit significand at most, and really rounded
    # row (0, 0): keys of tiles 0 and 1 were rounded against the first tile's maximum, then rescaled by 2^(m0 - m2)
    s2 = s[0, 0] * 1.4426950408889634
    m0, m2 = s2[:64].max(), s2[128:192].max()
    first = opr[0, 0, :128] * torch.exp2(m2 - m0)
    assert torch.allclose(first, first.to(torch.bfloat16).to(D), rtol=1e-12, atol=0)
    assert torch.allclose(opr[0, 0, 128:], opr[0, 0, 128:].to(torch.bfloat16).to(D), rtol=1e-12, atol=0)


def test_packed_attention_with_unequal_lengths_dropout_and_an_empty_sequence_by_loops():
    from oracle import flash_attention as ofa
    lq, lk = [3, 2, 4], [5, 0, 2]
    q, k, v, do, cu_q, cu_k = _packed_case(502, lq, lk, heads=1, d=4)
    p = 0.25
    keep = (torch.rand(3, 1, max(lq), max(lk), generator=torch.Generator().manual_seed(7)) < 0.75).to(torch.uint8)
    out, lse = ofa.flash_attn_fwd(q, k, v, cu_q, cu_k, max(lq), None, True, p, keep)
    for b in range(3):
        for i in range(lq[b]):
            row = torch.zeros(4, dtype=D)
            visible = [j for j in range(lk[b]) if j <= i]                        # causal: aligned at the first tokens
            z = sum(math.exp(float(q[cu_q[b] + i, 0] @ k[cu_k[b] + j, 0]) * 0.5) for j in visible)     # scale 1 / sqrt(4)
            for j in visible:
                pr = math.exp(float(q[cu_q[b] + i, 0] @ k[cu_k[b] + j, 0]) * 0.5) / z
                row += pr * float(keep[b, 0, i, j]) / (1 - p) * v[cu_k[b] + j, 0]      # dropout after the normalisation
            assert torch.allclose(out[cu_q[b] + i, 0], row, atol=1e-12), (b, i)
            assert (math.isinf(float(lse[b, 0, i])) and lse[b, 0, i] < 0) if not visible else abs(float(lse[b, 0, i]) - math.log(z)) < 1e-12
    # the gradient of that loop, by finite differences on one element of each input
    dq, dk, dv, _ = ofa.flash_attn_bwd(do, q, k, v, cu_q, cu_k, max(lq), None, True, p, keep)
    f = lambda q_, k_, v_: float((ofa.flash_attn_fwd(q_, k_, v_, cu_q, cu_k, max(lq), None, True, p, keep)[0] * do).sum())
    for t, gr, idx in ((q, dq, (1, 0, 2)), (k, dk, (0, 0, 1)), (v, dv, (6, 0, 3)), (q, dq, (4, 0, 0))):
        e = torch.zeros_like(t)
        e[idx] = 1e-6
        args = lambda s: [x + s * e if x is t else x for x in (q, k, v)]
        assert abs((f(*args(1)) - f(*args(-1))) / 2e-6 - float(gr[idx])) < 1e-7, idx


# ----------------------------------------------------------------------------- gated / variational feed-forward
@pytest.mark.parametrize("act", ["relu", "gelu", "silu", "agelu", "sigmoid"])
def test_gated_feed_forward_is_the_chain_of_library_ops(act):
    from oracle import feed_forward as off
    g = torch.Generator().manual_seed(601)
    t, b, dm, di = 5, 3, 8, 6
    x = torch.randn(t, b, dm, generator=g, dtype=D)
    w_in, b_in = torch.randn(2 * di, dm, generator=g, dtype=D), torch.randn(2 * di, generator=g, dtype=D)
    w_out, b_out = torch.randn(dm, di, generator=g, dtype=D), torch.randn(dm, generator=g, dtype=D)
    got = off.feed_forward(x, w_in, b_in, w_out, b_out, act, glu=True)
    lin = F.linear(x, w_in, b_in)
    if act == "sigmoid":
        hidden = F.glu(lin)                                   # the reference's act for 'sigmoid' (feed_forward.py:57-58)
    else:
        a, gate = lin.chunk(2, dim=-1)
        fn = {"relu": F.relu, "gelu": F.gelu, "silu": F.silu, "agelu": lambda v: F.gelu(v, approximate="tanh")}[act]
        hidden = fn(a) * gate
    assert torch.allclose(got, F.linear(hidden, w_out, b_out), atol=1e-12)


def test_variational_dropout_shares_one_mask_row_over_time_and_the_residual_form_adds_the_input():
    from oracle import feed_forward as off
    g = torch.Generator().manual_seed(602)
    t, b, dm, di, p = 4, 3, 6, 10, 0.25
    x = torch.randn(t, b, dm, generator=g, dtype=D)
    w_in, b_in = torch.randn(di, dm, generator=g, dtype=D), torch.randn(di, generator=g, dtype=D)
    w_out, b_out = torch.randn(dm, di, generator=g, dtype=D), torch.randn(dm, generator=g, dtype=D)
    keep = (torch.rand(1, b, di, generator=g) < 0.75).to(D)
    res_keep = (torch.rand(1, b, dm, generator=g) < 0.75).to(D)
    got = off.feed_forward(x, w_in, b_in, w_out, b_out, "relu", False, p, keep, True, p, res_keep)
    for ti in range(t):                                       # time step by time step, the same mask row each time
        h = F.relu(F.linear(x[ti], w_in, b_in)) * keep[0] / (1 - p)
        o = F.linear(h, w_out, b_out) * res_keep[0] / (1 - p) + x[ti]
        assert torch.allclose(got[ti], o, atol=1e-12)
    # and what variational_dropout is for: E[mask / (1 - p)] = 1, so the expectation over masks is the undropped layer
    plain = off.feed_forward(x, w_in, b_in, w_out, b_out, "relu")
    acc = torch.zeros_like(plain)
    n = 4000
    for _ in range(n):
        acc += off.feed_forward(x, w_in, b_in, w_out, b_out, "relu", False, p, (torch.rand(1, b, di, generator=g) < 0.75).to(D))
    assert float((acc / n - plain).abs().max()) < 0.25
