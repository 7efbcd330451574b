"""Self / encoder-decoder attention parity: HIP (through the C ABI) vs the CPU oracle on identical
seeded inputs, dropout via a replayed mask or p = 0.

Follows the reference's attention tests: the same function evaluated on the fused path and on
the PyTorch path with random key-padding or triu time masks, outputs and every gradient compared
(onmt/modules/optimized/test_encdec_attention_func.py:93-181 — Tq=64, Tk=512, B=64, E=1024, H=16;
test_self_attention_func.py:38-68 — T=512, B=64), tolerance 1e-2 / 1e-3 there, 2e-2 / 1e-3 here.
"""
import pytest
import torch

from nmtgminor_amd.modules.encdec_attention import EncdecMultiheadAttn
from nmtgminor_amd.modules.encdec_attention_func_bias import encdec_attn_bias_compact_func, encdec_attn_bias_func
from nmtgminor_amd.modules.self_attention import SelfMultiheadAttn
from nmtgminor_amd.modules.self_attention_func import self_attn_compact_func, self_attn_func
from nmtgminor_amd.native import encdec_multihead_attn_bias_blaslt as ed_native, self_multihead_attn_blaslt as sa_native
from oracle import attention as oat, inputs
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64


def _self_case(dev, t, b, e, h, dtype, p, causal=False, zero_bias=False, seed=71, recompute=False):
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=p, seed=seed, causal=causal, zero_bias=zero_bias)
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"], p,
                            d["dropout_mask"], D, round_to=dtype)
    bwd = oat.self_attn_bwd(d["dout"], d["x"], d["w_in"], d["w_out"], h, fwd, p, d["dropout_mask"], D, round_to=dtype)
    leaves = [d[k].to(dev).requires_grad_() for k in ("x", "w_in", "w_out", "b_in", "b_out")]
    mask = (d["time_mask"] if causal else d["pad_mask"]).to(dev)
    dm = d["dropout_mask"].to(dev) if p > 0 else None
    out, cov = self_attn_func(causal, True, h, leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], mask, p, False, None,
                              False, None, True, True, recompute, dm)
    out.backward(d["dout"].to(dev))
    assert_close(out, fwd["outputs"], dtype, "outputs")
    assert_close(cov, fwd["dropout_results"], dtype, "dropout_results")
    # masked keys carry exactly zero probability
    covc = cov.float().cpu().view(b, h, t, t)
    if causal:
        assert (covc[:, :, torch.triu(torch.ones(t, t), 1).bool()] == 0).all()
    else:
        assert (covc.permute(0, 3, 1, 2)[d["pad_mask"]] == 0).all()
    assert_close(leaves[0].grad, bwd["dx"], dtype, "dx", scale_atol=True)
    assert_close(leaves[1].grad, bwd["dw_in"], dtype, "dW_in", scale_atol=True)
    assert_close(leaves[2].grad, bwd["dw_out"], dtype, "dW_out", scale_atol=True)
    assert_close(leaves[3].grad, bwd["db_in"], dtype, "db_in", scale_atol=True)
    assert_close(leaves[4].grad, bwd["db_out"], dtype, "db_out", scale_atol=True)
    return d, fwd, bwd


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t,b,e,h,p", [(64, 4, 256, 4, 0.0), (128, 3, 512, 8, 0.1), (200, 2, 256, 4, 0.25), (33, 2, 128, 2, 0.1)])
def test_self_attention_key_padding(dev, dtype, t, b, e, h, p):
    _self_case(dev, t, b, e, h, dtype, p)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_self_attention_causal_and_recompute(dev, dtype):
    _self_case(dev, 128, 4, 512, 8, dtype, 0.1, causal=True)
    _self_case(dev, 96, 2, 256, 4, dtype, 0.2, recompute=True)


def test_self_attention_intermediates_and_native_contract(dev):
    dtype = torch.bfloat16
    t, b, e, h = 64, 2, 256, 4
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.1, seed=72, zero_bias=False)
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], None, 0.1,
                            d["dropout_mask"], D, round_to=dtype)
    g = lambda k: d[k].to(dev)
    lin, scores, dropped, dmask, ctx, out = sa_native.forward(False, True, h, g("x"), g("w_in"), g("w_out"), g("b_in"),
                                                              g("b_out"), g("pad_mask"), 0.1, dropout_mask=g("dropout_mask"))
    assert lin.shape == (t, b, 3 * e) and scores.shape == (b * h, t, t) and ctx.shape == (t, b, e)
    assert_close(lin, fwd["input_lin_results"], dtype, "input_lin_results")
    sc, so = scores.float().cpu(), fwd["attn_scores"].float()
    assert torch.equal(torch.isinf(sc), torch.isinf(so))                       # -inf exactly on the masked keys
    fin = ~torch.isinf(so)
    assert_close(sc[fin], so[fin], dtype, "attn_scores")
    assert_close(ctx, fwd["matmul2_results"], dtype, "matmul2_results")
    assert torch.equal(dmask.cpu(), d["dropout_mask"])
    # compact form: projections outside
    scores2, dropped2, _, ctx2 = sa_native.forward_compact(False, True, h, lin, g("pad_mask"), 0.1, dropout_mask=g("dropout_mask"))
    assert torch.equal(ctx2, ctx) and torch.equal(dropped2, dropped)
    dctx = torch.randn(t, b, e, generator=torch.Generator().manual_seed(1)).to(dtype)
    (dlin,) = sa_native.backward_compact(False, h, dctx.to(dev), dropped, scores, lin, dmask, 0.1)
    q, k, v = [fwd["input_lin_results"].to(D).view(t, b * h, 3, e // h)[:, :, i] for i in range(3)]
    dq, dk, dv = oat._core_bwd(dctx.to(D).view(t, b * h, e // h), q, k, v, fwd["softmax_results"], fwd["dropout_results"],
                               0.1, d["dropout_mask"], D, round_to=dtype)
    assert_close(dlin, torch.stack([dq, dk, dv], 2).reshape(t, b, 3 * e), dtype, "compact dlin", scale_atol=True)


def test_self_attention_rng_dropout_eval_and_no_bias(dev):
    dtype = torch.float16
    t, b, e, h = 64, 2, 128, 4
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=73, zero_bias=False)
    g = lambda k: d[k].to(dev)
    # biases None (Whisper-style projections without bias)
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], None, None, h, d["pad_mask"], None, 0.0, None, D, round_to=dtype)
    out, cov = self_attn_func(False, False, h, g("x"), g("w_in"), g("w_out"), None, None, g("pad_mask"), 0.3, False, None,
                              False, None, True, True, False)
    assert_close(out, fwd["outputs"], dtype, "eval, no bias")              # eval: dropout not applied
    torch.cuda.manual_seed(11)
    r = sa_native.forward(False, True, h, g("x"), g("w_in"), g("w_out"), None, None, g("pad_mask"), 0.3)
    dmask = r[3]
    assert dmask.shape == (b * h, t, t) and abs(dmask.float().mean().item() - 0.7) < 0.02
    fwd2 = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], None, None, h, d["pad_mask"], None, 0.3, dmask.cpu(), D, round_to=dtype)
    assert_close(r[5], fwd2["outputs"], dtype, "rng dropout outputs")
    with pytest.raises(RuntimeError):            # rotary encodings without their (cos, sin) tables
        self_attn_func(False, False, h, g("x"), g("w_in"), g("w_out"), None, None, None, 0.0, True, None, False, None, True, True, False)
    with pytest.raises(RuntimeError):
        sa_native.forward(False, False, h, g("x").float(), g("w_in").float(), g("w_out").float(), None, None, None, 0.0)


@pytest.mark.parametrize("mode", ["eval", "eval_no_coverage", "recompute_p0"])
def test_self_attention_backward_without_dropout_state(dev, mode):
    # A backward through a call that is not in training mode (grad mode on, is_training False), and through a
    # recomputing call with p = 0: inside an autograd function the grad mode is off, so the decision to keep the
    # scores for the backward must come from the inputs' requires_grad (head dimension 64 and a key count that is a
    # multiple of 4: the shape the score-free inference kernel would otherwise take).
    dtype = torch.bfloat16
    t, b, e, h = 64, 2, 256, 4
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=75, zero_bias=False)
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], None, 0.0, None, D,
                            round_to=dtype)
    bwd = oat.self_attn_bwd(d["dout"], d["x"], d["w_in"], d["w_out"], h, fwd, 0.0, None, D, round_to=dtype)
    leaves = [d[k].to(dev).requires_grad_() for k in ("x", "w_in", "w_out", "b_in", "b_out")]
    training, p, cover, recompute = {"eval": (False, 0.3, True, False), "eval_no_coverage": (False, 0.3, False, False),
                                     "recompute_p0": (True, 0.0, True, True)}[mode]
    out, cov = self_attn_func(False, training, h, *leaves, d["pad_mask"].to(dev), p, False, None, False, None, True, cover,
                              recompute)
    out.backward(d["dout"].to(dev))
    assert_close(out, fwd["outputs"], dtype, "outputs")
    if cover:
        assert_close(cov, fwd["dropout_results"], dtype, "coverage")
    for leaf, key in zip(leaves, ("dx", "dw_in", "dw_out", "db_in", "db_out")):
        assert_close(leaf.grad, bwd[key], dtype, key, scale_atol=True)
    # the same call under no_grad still leaves the score tensor out
    with torch.no_grad():
        r = sa_native.forward(False, False, h, *[z.detach() for z in leaves], d["pad_mask"].to(dev), 0.0)
    assert r[1].numel() == 0


@pytest.mark.parametrize("mode", ["eval", "eval_compact", "recompute_p0"])
def test_encdec_attention_backward_without_dropout_state(dev, mode):
    dtype = torch.bfloat16
    tq, tk, b, e, h = 32, 128, 2, 256, 4
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=0.0, seed=76, zero_bias=False)
    fwd = oat.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], d["b_q"], d["b_kv"], d["b_out"], h,
                              d["pad_mask"], 0.0, None, D, round_to=dtype)
    bwd = oat.encdec_attn_bwd(d["dout"], d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], h, fwd, 0.0, None, D,
                              round_to=dtype)
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out", "b_q", "b_kv", "b_out")
    leaf = {k: d[k].to(dev).requires_grad_() for k in names}
    pad = d["pad_mask"].to(dev)
    if mode == "eval_compact":
        q_lin = fwd["input_lin_q_results"].to(dtype).to(dev).requires_grad_()
        kv_lin = fwd["input_lin_kv_results"].to(dtype).to(dev).requires_grad_()
        (ctx_t,) = encdec_attn_bias_compact_func(False, False, h, q_lin, kv_lin, pad, 0.3, False, None, False, None, None, True,
                                                 False)
        dctx = torch.randn(tq, b, e, generator=torch.Generator().manual_seed(2)).to(dtype)
        ctx_t.backward(dctx.to(dev))
        assert_close(ctx_t, fwd["matmul2_results"], dtype, "context")
        k, v = [fwd["input_lin_kv_results"].to(D).view(tk, b * h, 2, e // h)[:, :, i] for i in range(2)]
        q = fwd["input_lin_q_results"].to(D).view(tq, b * h, e // h)
        dq, dk, dv = oat._core_bwd(dctx.to(D).view(tq, b * h, e // h), q, k, v, fwd["softmax_results"], fwd["dropout_results"],
                                   0.0, None, D, round_to=dtype)
        assert_close(q_lin.grad, dq.reshape(tq, b, e), dtype, "dq", scale_atol=True)
        assert_close(kv_lin.grad, torch.stack([dk, dv], 2).reshape(tk, b, 2 * e), dtype, "dkv", scale_atol=True)
        return
    recompute, training, p = (True, True, 0.0) if mode == "recompute_p0" else (False, False, 0.3)
    out, cov = encdec_attn_bias_func(recompute, training, h, leaf["x_q"], leaf["x_kv"], leaf["w_q"], leaf["w_kv"], leaf["w_out"],
                                     leaf["b_q"], leaf["b_kv"], leaf["b_out"], pad, p, False, None, False, None, None, True, True)
    out.backward(d["dout"].to(dev))
    assert_close(out, fwd["outputs"], dtype, "outputs")
    assert_close(cov, fwd["dropout_results"], dtype, "coverage")
    for key, n in (("dx_q", "x_q"), ("dx_kv", "x_kv"), ("dw_q", "w_q"), ("dw_kv", "w_kv"), ("dw_out", "w_out"),
                   ("db_q", "b_q"), ("db_kv", "b_kv"), ("db_out", "b_out")):
        assert_close(leaf[n].grad, bwd[key], dtype, key, scale_atol=True)


def _encdec_case(dev, tq, tk, b, e, h, dtype, p, zero_bias=False, biases=True, seed=74):
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=p, seed=seed, zero_bias=zero_bias)
    if not biases:
        d["b_q"] = d["b_kv"] = d["b_out"] = None
    fwd = oat.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], d["b_q"], d["b_kv"], d["b_out"], h,
                              d["pad_mask"], p, d["dropout_mask"], D, round_to=dtype)
    bwd = oat.encdec_attn_bwd(d["dout"], d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], h, fwd, p, d["dropout_mask"],
                              D, round_to=dtype)
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out", "b_q", "b_kv", "b_out")
    leaf = {k: (d[k].to(dev).requires_grad_() if d[k] is not None else None) for k in names}
    dm = d["dropout_mask"].to(dev) if p > 0 else None
    out, cov = encdec_attn_bias_func(False, True, h, leaf["x_q"], leaf["x_kv"], leaf["w_q"], leaf["w_kv"], leaf["w_out"],
                                     leaf["b_q"], leaf["b_kv"], leaf["b_out"], d["pad_mask"].to(dev), p, False, None, False,
                                     None, None, True, True, dm)
    out.backward(d["dout"].to(dev))
    assert_close(out, fwd["outputs"], dtype, "outputs")
    assert_close(cov, fwd["dropout_results"], dtype, "dropout_results")
    assert (cov.float().cpu().view(b, h, tq, tk).permute(0, 3, 1, 2)[d["pad_mask"]] == 0).all()
    for key, n in (("dx_q", "x_q"), ("dx_kv", "x_kv"), ("dw_q", "w_q"), ("dw_kv", "w_kv"), ("dw_out", "w_out"),
                   ("db_q", "b_q"), ("db_kv", "b_kv"), ("db_out", "b_out")):
        if leaf[n] is not None:
            assert_close(leaf[n].grad, bwd[key], dtype, key, scale_atol=True)
    return d, fwd, leaf


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tq,tk,b,e,h,p", [(64, 512, 4, 256, 4, 0.0), (32, 1500, 2, 256, 4, 0.1), (17, 100, 3, 128, 2, 0.2)])
def test_encdec_attention(dev, dtype, tq, tk, b, e, h, p):
    _encdec_case(dev, tq, tk, b, e, h, dtype, p)


def test_encdec_attention_without_biases_and_compact(dev):
    dtype = torch.bfloat16
    d, fwd, leaf = _encdec_case(dev, 48, 300, 2, 256, 4, dtype, 0.1, biases=False)
    r = ed_native.forward(True, 4, leaf["x_q"].detach(), leaf["x_kv"].detach(), leaf["w_q"].detach(), leaf["w_kv"].detach(),
                          leaf["w_out"].detach(), None, None, None, d["pad_mask"].to(dev), 0.1,
                          dropout_mask=d["dropout_mask"].to(dev))
    q_lin, kv_lin, scores, dropped, dmask, ctx, out = r
    assert q_lin.shape == (48, 2, 256) and kv_lin.shape == (300, 2, 512) and scores.shape == (8, 48, 300)
    assert_close(kv_lin, fwd["input_lin_kv_results"], dtype, "kv_lin")
    ctx2, cov2 = encdec_attn_bias_compact_func(False, True, 4, q_lin, kv_lin, d["pad_mask"].to(dev), 0.1, False, None, False,
                                               None, None, True, True, d["dropout_mask"].to(dev))
    assert torch.equal(ctx2, ctx) and torch.equal(cov2, dropped)
    dq, dkv = ed_native.backward_compact(4, d["dout"].to(dev), dropped, scores, q_lin, kv_lin, dmask, 0.1)
    assert dq.shape == q_lin.shape and dkv.shape == kv_lin.shape and torch.isfinite(dq.float()).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tq,tk,b,e,h,p,recompute", [(48, 300, 2, 256, 4, 0.1, False), (33, 512, 3, 128, 2, 0.25, True),
                                                     (16, 70, 2, 128, 2, 0.0, False)])
def test_bias_free_encdec_function_returns_the_pre_dropout_probabilities(dev, dtype, tq, tk, b, e, h, p, recompute):
    # EncdecAttnFunc (onmt/modules/optimized/encdec_attention_func.py:36-568): 17 arguments, no biases; its fused branch
    # hands back softmax_results as coverage (:123-124) and its backward starts from them (:322-345)
    from nmtgminor_amd.modules.encdec_attention_func import encdec_attn_func
    from nmtgminor_amd.native import encdec_multihead_attn_cuda as free_native
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=p, seed=75, zero_bias=False)
    fwd = oat.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], None, None, None, h, d["pad_mask"], p,
                              d["dropout_mask"], D, round_to=dtype)
    # this backward starts from the probabilities as stored (rounded to 16 bits), not from the scores
    saved = dict(fwd, softmax_results=fwd["softmax_results"].to(dtype).to(D))
    bwd = oat.encdec_attn_bwd(d["dout"], d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], h, saved, p, d["dropout_mask"], D,
                              round_to=dtype)
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out")
    leaf = {k: d[k].to(dev).requires_grad_() for k in names}
    dm = d["dropout_mask"].to(dev) if p > 0 else None
    mask3 = d["pad_mask"].to(dev).unsqueeze(1)                     # the broadcast form the reference's callers pass
    out, cov = encdec_attn_func(recompute, True, h, leaf["x_q"], leaf["x_kv"], leaf["w_q"], leaf["w_kv"], leaf["w_out"], mask3, p,
                                False, None, False, None, None, False, True, dm)
    out.backward(d["dout"].to(dev))
    assert_close(out, fwd["outputs"], dtype, "outputs")
    assert_close(cov, fwd["softmax_results"], dtype, "coverage = probabilities before dropout")
    if p > 0:
        assert not torch.equal(cov.cpu() == 0, fwd["dropout_results"].to(dtype) == 0)      # no dropped units in it
    assert_close(cov.float().sum(-1), torch.ones(b * h, tq), dtype, "rows sum to one", atol=2e-2)
    for key, n in (("dx_q", "x_q"), ("dx_kv", "x_kv"), ("dw_q", "w_q"), ("dw_kv", "w_kv"), ("dw_out", "w_out")):
        assert_close(leaf[n].grad, bwd[key], dtype, key, scale_atol=True)
    # the extension's own lists
    r = free_native.forward(True, h, d["x_q"].to(dev), d["x_kv"].to(dev), d["w_q"].to(dev), d["w_kv"].to(dev), d["w_out"].to(dev),
                            d["pad_mask"].to(dev), p, dropout_mask=dm)
    assert len(r) == 7 and r[2].shape == (b * h, tq, tk) and torch.equal(r[2], cov)
    g = free_native.backward(h, d["dout"].to(dev), r[5], r[3], r[2], r[0], r[1], d["x_q"].to(dev), d["x_kv"].to(dev),
                             d["w_q"].to(dev), d["w_kv"].to(dev), d["w_out"].to(dev), r[4], p)
    assert len(g) == 5
    assert_close(g[3], bwd["dw_kv"], dtype, "dw_kv from the extension's backward", scale_atol=True)
    out1 = encdec_attn_func(False, False, h, d["x_q"].to(dev), d["x_kv"].to(dev), d["w_q"].to(dev), d["w_kv"].to(dev),
                            d["w_out"].to(dev), None, p, False, None, False, None, None, False, False)
    assert isinstance(out1, tuple) and len(out1) == 1


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t,b,e,h,causal", [(40, 2, 128, 2, False), (64, 3, 256, 4, True)])
def test_self_attention_with_rotary_position_encodings(dev, dtype, t, b, e, h, causal):
    # self_attn_func with rotary_pos_enc = True and pos_emb = (cos, sin) [T, 1, D] (self_attention_func.py:178-184, :467-469)
    from oracle import rotary as orot
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=76, causal=causal, zero_bias=False)
    cos, sin = orot.tables(torch.arange(t), e // h)
    cos, sin = cos.to(dtype), sin.to(dtype)
    names = ("x", "w_in", "w_out", "b_in", "b_out")
    leaf = {k: d[k].to(dev).requires_grad_() for k in names}
    mask = d["time_mask"] if causal else d["pad_mask"]
    out, cov = self_attn_func(causal, True, h, leaf["x"], leaf["w_in"], leaf["w_out"], leaf["b_in"], leaf["b_out"], mask.to(dev), 0.0,
                              True, (cos.to(dev), sin.to(dev)), False, None, True, True, False)
    out.backward(d["dout"].to(dev))
    ref = {k: d[k].to(D).requires_grad_() for k in names}
    want, wcov = orot.self_attn_rotary(ref["x"], ref["w_in"], ref["w_out"], ref["b_in"], ref["b_out"], h,
                                       None if causal else d["pad_mask"], d["time_mask"] if causal else None, cos.to(D), sin.to(D),
                                       round_to=dtype)
    want.backward(d["dout"].to(D))
    assert_close(out, want.detach(), dtype, "outputs")
    assert_close(cov, wcov.detach(), dtype, "coverage")
    for k in names:
        assert_close(leaf[k].grad, ref[k].grad, dtype, "d " + k, scale_atol=True)
    # the rotation kernel alone, forward then transposed, on the strided head slots
    from nmtgminor_amd.native import rotary_position as rot
    lin = torch.randn(t, b, 3 * e, generator=torch.Generator().manual_seed(77)).to(dtype)
    got = rot.rotate_qk_(lin.clone().to(dev), cos.to(dev), sin.to(dev), b * h, e // h)
    v4 = lin.to(D).view(t, b * h, 3, e // h)
    assert_close(got.view(t, b * h, 3, -1)[:, :, 0], orot.apply_rotary(v4[:, :, 0], cos.to(D), sin.to(D)), dtype, "rotated q")
    assert_close(got.view(t, b * h, 3, -1)[:, :, 1], orot.apply_rotary(v4[:, :, 1], cos.to(D), sin.to(D)), dtype, "rotated k")
    assert torch.equal(got.view(t, b * h, 3, -1)[:, :, 2].cpu(), lin.view(t, b * h, 3, -1)[:, :, 2])      # values untouched
    back = rot.rotate_qk_(lin.clone().to(dev), cos.to(dev), sin.to(dev), b * h, e // h, inverse=True)
    assert_close(back.view(t, b * h, 3, -1)[:, :, 1], orot.apply_rotary_transposed(v4[:, :, 1], cos.to(D), sin.to(D)), dtype,
                 "transposed rotation")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_encdec_attention_with_rotary_position_encodings(dev, dtype):
    from nmtgminor_amd.modules.encdec_attention_func import encdec_attn_func
    from oracle import rotary as orot
    tq, tk, b, e, h = 24, 70, 2, 128, 2
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=0.0, seed=78, zero_bias=False)
    cq, sq = (z.to(dtype) for z in orot.tables(torch.arange(tq), e // h))
    ck, sk = (z.to(dtype) for z in orot.tables(torch.arange(tk), e // h))
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out")
    leaf = {k: d[k].to(dev).requires_grad_() for k in names}
    out, cov = encdec_attn_func(False, True, h, leaf["x_q"], leaf["x_kv"], leaf["w_q"], leaf["w_kv"], leaf["w_out"],
                                d["pad_mask"].to(dev), 0.0, False, None, True, (cq.to(dev), sq.to(dev)), (ck.to(dev), sk.to(dev)),
                                False, True)
    out.backward(d["dout"].to(dev))
    ref = {k: d[k].to(D).requires_grad_() for k in names}
    want, wcov = orot.encdec_attn_rotary(ref["x_q"], ref["x_kv"], ref["w_q"], ref["w_kv"], ref["w_out"], h, d["pad_mask"],
                                         cq.to(D), sq.to(D), ck.to(D), sk.to(D), round_to=dtype)
    want.backward(d["dout"].to(D))
    assert_close(out, want.detach(), dtype, "outputs")
    assert_close(cov, wcov.detach(), dtype, "coverage")
    for k in names:
        assert_close(leaf[k].grad, ref[k].grad, dtype, "d " + k, scale_atol=True)


def test_modules_state_dict_names_and_forward(dev):
    sa = SelfMultiheadAttn(256, 4, dropout=0.0).to(dev).half()
    assert sorted(sa.state_dict()) == ["in_proj_bias", "in_proj_weight", "out_proj_bias", "out_proj_weight"]
    x = torch.randn(40, 3, 256, device=dev).half()
    pad = torch.zeros(3, 40, dtype=torch.bool, device=dev)
    pad[1, 30:] = True
    y, cov = sa(x, None, key_padding_mask=pad)
    ref = oat.self_attn_fwd(x.cpu(), sa.in_proj_weight.detach().cpu(), sa.out_proj_weight.detach().cpu(),
                            sa.in_proj_bias.detach().cpu(), sa.out_proj_bias.detach().cpu(), 4, pad.cpu(), None, 0.0, None, D,
                            round_to=torch.float16)
    assert_close(y, ref["outputs"], torch.float16, "module outputs")
    y2, _ = sa(x, None, attn_mask=torch.triu(torch.ones(40, 40, device=dev), 1).bool())
    assert y2.shape == x.shape
    ed = EncdecMultiheadAttn(4, 256).to(dev).half()
    assert sorted(ed.state_dict()) == ["in_proj_weight_kv", "in_proj_weight_q", "out_proj_weight"]
    mem = torch.randn(70, 3, 256, device=dev).half()
    o, c = ed(x, mem, mem, attn_mask=torch.zeros(3, 70, dtype=torch.bool, device=dev))
    assert o.shape == x.shape and c.shape == (12, 40, 70)


def test_feed_forward_module(dev):
    from nmtgminor_amd.modules.feed_forward import PositionWiseFeedForward
    from oracle import mlp as omlp
    ff = PositionWiseFeedForward(128, 512, dropout=0.1, activation="gelu").to(dev).half().eval()
    assert sorted(ff.state_dict()) == ["in_proj_bias", "in_proj_weight", "out_proj_bias", "out_proj_weight"]
    x = torch.randn(20, 4, 128, device=dev).half()
    y = ff(x)
    w = [ff.in_proj_weight.detach().cpu(), ff.out_proj_weight.detach().cpu()]
    bb = [ff.in_proj_bias.detach().cpu(), ff.out_proj_bias.detach().cpu()]
    yo, _, _ = omlp.mlp_fwd(x.cpu().view(80, 128), w, bb, "gelu", 0.0, None, D, round_to=torch.float16)
    assert_close(y.view(80, 128), yo, torch.float16, "feed-forward eval")
    ffr = PositionWiseFeedForward(128, 512, dropout=0.0, activation="relu", dropout_residual=True, res_dropout=0.0).to(dev).half()
    yr = ffr(x.clone())
    w = [ffr.in_proj_weight.detach().cpu(), ffr.out_proj_weight.detach().cpu()]
    bb = [ffr.in_proj_bias.detach().cpu(), ffr.out_proj_bias.detach().cpu()]
    yo, _, _ = omlp.mlp_fwd(x.cpu().view(80, 128), w, bb, "relu", 0.0, None, D, round_to=torch.float16)
    assert_close(yr.view(80, 128), yo.to(torch.float16).to(D) + x.cpu().view(80, 128).to(D), torch.float16, "residual")
    with pytest.raises(NotImplementedError):
        PositionWiseFeedForward(128, 512, activation="tanh")


# ----------------------------------------------------------------------------- inference without a score tensor
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("t,b,e,h,causal", [(100, 3, 256, 4, False), (72, 2, 256, 2, True), (200, 2, 128, 2, False), (36, 2, 256, 4, True)])
def test_self_attention_inference_without_the_score_tensor(dev, monkeypatch, dtype, t, b, e, h, causal, split):
    """Under torch.no_grad() an inference call returns no scores and runs the one-kernel path (probabilities and context
    from two passes over the keys). Held against the oracle and against the score-keeping path of the same library
    (the same rounding points: scores rounded to the 16-bit type, probabilities rounded before they multiply v). `split`
    forces one of the kernel's two forms: blocks of 128 queries, or blocks of 32 queries whose wavefronts share the keys."""
    monkeypatch.setenv("NMTG_ATTN_PROBS_SPLIT", split)
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=300 + t, causal=causal)
    if not causal:
        d["pad_mask"][-1, :] = True                                        # a sentence without any live key: zeros, not NaN
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"], 0.0, None, D,
                            round_to=dtype)
    g = lambda k: d[k].to(dev)
    mask = g("time_mask") if causal else g("pad_mask")
    args = (causal, False, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), mask, 0.1)
    with torch.no_grad():
        lin, scores, dropped, dmask, ctx, out = sa_native.forward(*args)
    assert scores.numel() == 0 and dmask.numel() == 0 and dropped.shape == (b * h, t, t)
    lin2, scores2, dropped2, _, ctx2, out2 = sa_native.forward(*args)     # recorded by autograd: keeps the scores
    assert scores2.shape == (b * h, t, t)
    assert_close(out, fwd["outputs"], dtype, "outputs")
    assert_close(dropped, fwd["dropout_results"], dtype, "probabilities")
    assert_close(dropped, dropped2.cpu(), dtype, "probabilities, against the score-keeping path")
    assert_close(ctx, ctx2.cpu(), dtype, "context, against the score-keeping path")
    assert not torch.isnan(dropped.float()).any()
    cov = dropped.float().cpu().view(b, h, t, t)
    if causal:
        assert (cov[:, :, torch.triu(torch.ones(t, t), 1).bool()] == 0).all()
    else:
        assert (cov.permute(0, 3, 1, 2)[d["pad_mask"]] == 0).all() and (cov[-1] == 0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tq,tk,b,e,h,masked", [(32, 1500, 2, 256, 4, True), (17, 100, 3, 128, 2, True), (130, 64, 2, 512, 4, False),
                                                (5, 260, 1, 128, 1, True)])
@pytest.mark.parametrize("split", ["0", "1"])
def test_encdec_attention_inference_without_the_score_tensor(dev, monkeypatch, dtype, tq, tk, b, e, h, masked, split):
    monkeypatch.setenv("NMTG_ATTN_PROBS_SPLIT", split)
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=0.0, seed=400 + tq)
    pad = d["pad_mask"] if masked else None
    fwd = oat.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], d["b_q"], d["b_kv"], d["b_out"], h, pad, 0.0,
                              None, D, round_to=dtype)
    g = lambda k: d[k].to(dev)
    args = (False, h, g("x_q"), g("x_kv"), g("w_q"), g("w_kv"), g("w_out"), g("b_q"), g("b_kv"), g("b_out"),
            None if pad is None else pad.to(dev), 0.0)
    with torch.no_grad():
        q_lin, kv_lin, scores, dropped, dmask, ctx, out = ed_native.forward(*args)
    assert scores.numel() == 0 and dropped.shape == (b * h, tq, tk) and kv_lin.shape == (tk, b, 2 * e)
    r2 = ed_native.forward(*args)
    assert r2[2].shape == (b * h, tq, tk)
    assert_close(out, fwd["outputs"], dtype, "outputs")
    assert_close(dropped, fwd["dropout_results"], dtype, "probabilities")
    assert_close(dropped, r2[3].cpu(), dtype, "probabilities, against the score-keeping path")
    assert_close(ctx, r2[5].cpu(), dtype, "context, against the score-keeping path")
    if masked:
        assert (dropped.float().cpu().view(b, h, tq, tk).permute(0, 3, 1, 2)[d["pad_mask"]] == 0).all()
    assert (dropped.float().sum(-1) - 1).abs().max() < 2e-2


def test_inference_keeps_the_score_tensor_where_the_one_kernel_path_does_not_apply(dev, monkeypatch):
    d = inputs.self_attn_inputs(30, 2, 64, 2, torch.bfloat16, p=0.0, seed=9)        # head dimension 32, 30 keys
    g = lambda k: d[k].to(dev)
    with torch.no_grad():
        r = sa_native.forward(False, False, 2, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.0)
    assert r[1].shape == (4, 30, 30)
    d = inputs.self_attn_inputs(64, 2, 128, 2, torch.bfloat16, p=0.0, seed=9)
    g = lambda k: d[k].to(dev)
    monkeypatch.setenv("NMTG_ATTN_PROBS", "0")
    with torch.no_grad():
        r = sa_native.forward(False, False, 2, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.0)
    assert r[1].shape == (4, 64, 64)


@pytest.mark.parametrize("split", ["0", "1"])
def test_inference_without_coverage_writes_no_probability_tensor(dev, monkeypatch, split):
    """A caller that does not return the coverage (return_coverage=False) gets the same outputs from an inference call
    under torch.no_grad(), and neither the scores nor the probabilities exist as tensors."""
    monkeypatch.setenv("NMTG_ATTN_PROBS_SPLIT", split)
    dtype, h = torch.bfloat16, 4
    d = inputs.self_attn_inputs(136, 2, 256, h, dtype, p=0.0, seed=77)
    g = lambda k: d[k].to(dev)
    args = (False, False, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.0)
    with torch.no_grad():
        full = sa_native.forward(*args)
        lean = sa_native.forward(*args, want_probs=False)
        out_func, cov_func = self_attn_func(False, False, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.0,
                                            False, None, False, None, False, False, False)
    assert lean[1].numel() == 0 and lean[2].numel() == 0 and full[2].shape == (2 * h, 136, 136)
    assert torch.equal(lean[4], full[4]) and torch.equal(lean[5], full[5]) and torch.equal(out_func, full[5]) and cov_func.numel() == 0
    e = inputs.encdec_attn_inputs(40, 300, 2, 256, h, dtype, p=0.0, seed=78)
    ge = lambda k: e[k].to(dev)
    eargs = (False, h, ge("x_q"), ge("x_kv"), ge("w_q"), ge("w_kv"), ge("w_out"), ge("b_q"), ge("b_kv"), ge("b_out"), ge("pad_mask"), 0.0)
    with torch.no_grad():
        full = ed_native.forward(*eargs)
        lean = ed_native.forward(*eargs, want_probs=False)
        res = encdec_attn_bias_func(False, False, h, ge("x_q"), ge("x_kv"), ge("w_q"), ge("w_kv"), ge("w_out"), ge("b_q"), ge("b_kv"),
                                    ge("b_out"), ge("pad_mask"), 0.0, False, None, False, None, None, False, False)
    assert lean[2].numel() == 0 and lean[3].numel() == 0 and torch.equal(lean[6], full[6])
    assert torch.equal(res[0] if isinstance(res, tuple) else res, full[6])
    # recorded by autograd (or in training mode) the tensors are kept whatever the caller asks for
    kept = sa_native.forward(*args, want_probs=False)
    assert kept[1].shape == (2 * h, 136, 136) and kept[2].shape == (2 * h, 136, 136)


@pytest.mark.parametrize("seed", range(4000, 4012))
def test_inference_kernel_on_randomly_drawn_shapes(dev, monkeypatch, seed):
    """Query counts around the block and wavefront sizes, key counts from 4 up (multiples of 4: around the 64-key tile,
    one tile, many), both head dimensions, both forms of the kernel, key-padding masks with fully masked sentences and
    time masks: probabilities and context against the score-keeping path, which shares no kernel with it."""
    import random
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    h, dh = rnd.choice([1, 2, 3]), rnd.choice([64, 128])
    e, b = h * dh, rnd.choice([1, 2, 3])
    monkeypatch.setenv("NMTG_ATTN_PROBS_SPLIT", rnd.choice(["0", "1"]))
    g = torch.Generator().manual_seed(seed)
    if rnd.random() < 0.5:                                                    # self-attention, key padding or time mask
        t = 4 * rnd.choice([1, 2, 8, 15, 16, 17, 31, 33, 48, 65])
        causal = rnd.random() < 0.5
        d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=seed, causal=causal)
        if not causal and b > 1 and rnd.random() < 0.5:
            d["pad_mask"][0, :] = True
        gd = lambda k: d[k].to(dev)
        args = (causal, False, h, gd("x"), gd("w_in"), gd("w_out"), gd("b_in"), gd("b_out"), gd("time_mask") if causal else gd("pad_mask"), 0.0)
        with torch.no_grad():
            lean = sa_native.forward(*args)
        full = sa_native.forward(*args)
        pairs = ((lean[2], full[2], "probabilities"), (lean[4], full[4], "context"), (lean[5], full[5], "outputs"))
        assert lean[1].numel() == 0
    else:                                                                     # encoder-decoder attention
        tq = rnd.choice([1, 5, 31, 32, 33, 64, 100, 128, 129, 200])
        tk = 4 * rnd.choice([1, 3, 15, 16, 17, 40, 100, 129, 375])
        d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=0.0, seed=seed)
        pad = d["pad_mask"] if rnd.random() < 0.7 else None
        if pad is not None and b > 1 and rnd.random() < 0.5:
            pad[-1, :] = True
        gd = lambda k: d[k].to(dev)
        args = (False, h, gd("x_q"), gd("x_kv"), gd("w_q"), gd("w_kv"), gd("w_out"), gd("b_q"), gd("b_kv"), gd("b_out"),
                None if pad is None else pad.to(dev), 0.0)
        with torch.no_grad():
            lean = ed_native.forward(*args)
        full = ed_native.forward(*args)
        pairs = ((lean[3], full[3], "probabilities"), (lean[5], full[5], "context"), (lean[6], full[6], "outputs"))
        assert lean[2].numel() == 0
    for got, want, what in pairs:
        assert not torch.isnan(got.float()).any(), what
        assert_close(got, want.cpu(), dtype, f"{what} (seed {seed})", atol=2e-3)


def test_a_mask_view_at_an_odd_address_is_accepted(dev):
    """A uint8 mask that is a view into a larger buffer (odd start address) reaches the kernels as an aligned copy."""
    d = inputs.self_attn_inputs(64, 2, 128, 2, torch.bfloat16, p=0.0, seed=5)
    g = lambda k: d[k].to(dev)
    buf = torch.zeros(2 * 64 + 3, dtype=torch.uint8, device=dev)
    buf[3:] = d["pad_mask"].to(torch.uint8).reshape(-1).to(dev)
    odd = buf[3:].view(2, 64)
    assert odd.data_ptr() % 4 != 0
    with torch.no_grad():
        a = sa_native.forward(False, False, 2, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), odd, 0.0)
        b = sa_native.forward(False, False, 2, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.0)
    assert torch.equal(a[5], b[5]) and torch.equal(a[2], b[2])
