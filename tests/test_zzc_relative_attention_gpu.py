"""Self-attention with relative position encodings against the fp32 oracle (oracle/relative_attention.py), and its
elementwise kernels (bias additions, relative shift, the shift's adjoint, column sums) bit for bit against index
arithmetic on the CPU.

What the reference computes here: RelativeShift and RelativeSelfAttnFunc
(onmt/modules/optimized/relative_self_attention_func.py:26-76, :79-726). The shift moves values without arithmetic, so
it is compared exactly; the attention results to the 16-bit tolerance of the other attention tests.
"""
import random

import pytest
import torch

from nmtgminor_amd.modules.linear import Linear, linear_function
from nmtgminor_amd.modules.relative_self_attention import RelativeSelfMultiheadAttn
from nmtgminor_amd.modules.relative_self_attention_func import RelativeShift, relative_self_attn_func
from nmtgminor_amd.native import linear_blaslt, linear_gemm, relative_position, relative_self_attn_blaslt
from oracle import inputs, relative_attention as orel
from util import assert_close, load_golden

pytestmark = pytest.mark.gpu
D = torch.float64


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("b,tq,tk,r", [(3, 16, 16, 16), (2, 9, 9, 13), (1, 40, 40, 48), (2, 7, 5, 8), (1, 1, 1, 1)])
def test_shift_add_and_its_adjoint_move_values_exactly(dev, dtype, b, tq, tk, r):
    g = torch.Generator().manual_seed(b * 100 + tq + r)
    ac = torch.randint(-8, 9, (b, tq, tk), generator=g).to(dtype)          # small integers: the sum is exact in every dtype
    bd = torch.randint(-8, 9, (b, tq, r), generator=g).to(dtype)
    got = relative_position.shift_add_(ac.clone().to(dev), bd.to(dev))
    want = ac.to(D) + orel.relative_shift(bd.to(D))[:, :, :tk]
    assert torch.equal(got.cpu().to(D), want)
    gs = torch.randint(-8, 9, (b, tq, tk), generator=g).to(dtype)
    back = relative_position.shift_backward(gs.to(dev), r)
    full = torch.cat([gs.to(D), torch.zeros(b, tq, r - tk, dtype=D)], dim=-1)
    assert back.shape == (b, tq, r) and torch.equal(back.cpu().to(D), orel.relative_shift_bwd(full))
    if tk == r:                                                              # the class the reference exposes
        assert torch.equal(RelativeShift.forward(bd.to(dev), True, False).cpu().to(D), orel.relative_shift(bd.to(D)))
        assert torch.equal(RelativeShift.backward(gs.to(dev), True, False).cpu().to(D), orel.relative_shift_bwd(gs.to(D)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bh,heads,tq,tk,r,mask,p", [
    (4, 2, 16, 16, 16, None, 0.0), (4, 2, 24, 24, 40, "pad", 0.25), (2, 1, 40, 16, 16, "time", 0.25), (6, 3, 5, 72, 80, "pad", 0.5),
    (2, 2, 9, 1032, 1032, None, 0.1), (2, 1, 3, 2048, 2049, "time", 0.1), (1, 1, 130, 64, 64, None, 0.3), (3, 1, 1, 8, 8, None, 0.0)])
def test_shift_folded_into_the_softmax_matches_the_separate_kernels(dev, dtype, bh, heads, tq, tk, r, mask, p):
    """One kernel for shift + sum + softmax + dropout, and one for their adjoints, against the chain of separate kernels:
    the same roundings in the same places. The summed scores that are kept for the backward and the movement of the
    score gradient into the position term's gradient are compared bit for bit (that buffer starts out as NaN, so an
    element left unwritten shows); probabilities and score gradients to four units in the last place of the dtype,
    because the separate softmax spreads a short row over the lanes differently and so adds the row up in another
    order. The keep mask that the fused kernel draws is replayed in the separate chain (the generator's stream depends
    on how a row is spread over the lanes)."""
    from nmtgminor_amd.native import mask_softmax_dropout_cuda as softmax_native
    assert relative_position.fused_ok((bh, tq, tk), dtype, r)
    g = torch.Generator().manual_seed(bh * 1000 + tq * 10 + r)
    ac, bd = torch.randn(bh, tq, tk, generator=g).to(dtype).to(dev), torch.randn(bh, tq, r, generator=g).to(dtype).to(dev)
    grad = torch.randn(bh, tq, tk, generator=g).to(dtype).to(dev)
    mask_kw, km, kind = {}, None, 0
    if mask == "pad":
        pad = torch.rand(bh // heads, tk, generator=g) < 0.3
        pad[:, 0] = False
        pad[-1, :] = tq > 5                                                 # one sentence without any live key
        mask_kw, km, kind = dict(pad_mask=pad.to(dev)), pad.to(torch.uint8).to(dev), 1
    elif mask == "time":
        tm = torch.triu(torch.ones(tq, tk), diagonal=1).bool()
        mask_kw, km, kind = dict(time_mask=tm.to(dev)), tm.to(torch.uint8).to(dev), 2
    training = p > 0
    s2 = ac.clone()
    dm2, dr2 = relative_position.shift_add_softmax_dropout(s2, bd, training, heads, p, km, kind)        # mask drawn in the kernel
    s1 = relative_position.shift_add_(ac.clone(), bd)
    dm1, _, dr1 = softmax_native.forward(training, heads, s1, p, want_softmax=False, dropout_mask=dm2 if training else None,
                                         **mask_kw)                                                     # the same mask replayed
    ulp2 = 4 * torch.finfo(dtype).eps
    assert torch.equal(s1, s2)
    torch.testing.assert_close(dr2.float(), dr1.float(), rtol=ulp2, atol=1e-4 * ulp2)
    if training:
        assert dm2.shape == (bh, tq, tk) and abs(dm2.float().mean().item() - (1 - p)) < 4 * (p * (1 - p) / dm2.numel()) ** 0.5 + 1e-3
        dm3, dr3 = relative_position.shift_add_softmax_dropout(ac.clone(), bd, training, heads, p, km, kind, dm2)   # replayed mask
        assert torch.equal(dr3.view(torch.uint8), dr2.view(torch.uint8)) and dm3 is not None
    gs1 = softmax_native.backward_recompute(heads, grad, None, s1, dm1, p, **mask_kw)
    gb1 = relative_position.shift_backward(gs1, r)
    gb2 = torch.full((bh, tq, r), float("nan"), dtype=dtype, device=dev)
    gs2, _ = relative_position.softmax_dropout_shift_backward(grad, s2, r, heads, dm2, p, km, kind, grad_bd=gb2)
    torch.testing.assert_close(gs2.float(), gs1.float(), rtol=ulp2, atol=ulp2)       # p (g - sum p g): a difference of O(1) terms
    assert not torch.isnan(gb2).any()
    assert torch.equal(gb2, relative_position.shift_backward(gs2, r))
    torch.testing.assert_close(gb2.float(), gb1.float(), rtol=ulp2, atol=ulp2)


def test_fused_shift_is_refused_for_rows_the_wide_kernels_cannot_take(dev):
    assert not relative_position.fused_ok((2, 8, 12, ), torch.bfloat16, 16)       # not a multiple of 16 bytes
    assert not relative_position.fused_ok((2, 8, 4104), torch.bfloat16, 4104)     # beyond one wavefront's row
    assert not relative_position.fused_ok((2, 8, 16), torch.bfloat16, 8)          # fewer positions than keys
    with pytest.raises(RuntimeError, match="multiple"):
        relative_position.shift_add_softmax_dropout(torch.zeros(1, 4, 12, dtype=torch.bfloat16, device=dev),
                                                    torch.zeros(1, 4, 16, dtype=torch.bfloat16, device=dev), False, 1, 0.0, None, 0)
    with pytest.raises(RuntimeError, match="len_r"):
        relative_position.softmax_dropout_shift_backward(torch.zeros(1, 4, 16, dtype=torch.bfloat16, device=dev),
                                                         torch.zeros(1, 4, 16, dtype=torch.bfloat16, device=dev), 8, 1, None, 0.0, None, 0)


def test_shift_refuses_fewer_positions_than_keys(dev):
    with pytest.raises(RuntimeError):
        relative_position.shift_add_(torch.zeros(1, 4, 8, dtype=torch.bfloat16, device=dev),
                                     torch.zeros(1, 4, 6, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError):
        relative_position.shift_backward(torch.zeros(1, 4, 8, dtype=torch.bfloat16, device=dev), 6)
    with pytest.raises(NotImplementedError):
        RelativeShift.forward(torch.zeros(4, 8, 2, dtype=torch.bfloat16, device=dev), False, True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("t,b,h,d", [(5, 2, 4, 64), (3, 1, 3, 20), (4, 2, 2, 7)])
def test_query_bias_adds_per_head_biases_to_queries_inside_the_projection(dev, dtype, t, b, h, d):
    g = torch.Generator().manual_seed(t + d)
    lin = torch.randn(t, b * h, 3, d, generator=g).to(dtype)
    u, w = torch.randn(h, d, generator=g).to(dtype), torch.randn(h, d, generator=g).to(dtype)
    rw, rr = relative_position.query_bias(lin.to(dev)[:, :, 0, :], u.to(dev), w.to(dev), h)
    q = lin[:, :, 0, :].reshape(t, b, h, d)
    assert torch.equal(rw.cpu(), (q + u).reshape(t, b * h, d)) and torch.equal(rr.cpu(), (q + w).reshape(t, b * h, d))
    with pytest.raises(RuntimeError):
        relative_position.query_bias(lin.to(dev)[:, :, 0, :], u.to(dev)[:, :d - 1], w.to(dev), h)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,cols,pitch", [(300, 64, 64), (129, 40, 48), (5, 7, 7), (1000, 520, 1024), (1, 16, 16)])
def test_column_sums(dev, dtype, rows, cols, pitch):
    g = torch.Generator().manual_seed(rows + cols)
    x = torch.randn(rows, pitch, generator=g).to(dtype)
    got = linear_gemm.colsum(x.to(dev)[:, :cols])
    assert got.dtype == dtype and got.shape == (cols,)
    assert_close(got, x[:, :cols].to(D).sum(0), dtype, "column sums", scale_atol=True)
    assert torch.equal(linear_gemm.colsum(x.to(dev)[:0, :cols]).cpu(), torch.zeros(cols, dtype=dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_linear_layer_and_its_three_gradients(dev, dtype):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(6, 5, 64, generator=g).to(dtype)
    w = (torch.randn(96, 64, generator=g) / 8).to(dtype)
    b = torch.randn(96, generator=g).to(dtype)
    gy = torch.randn(6, 5, 96, generator=g).to(dtype)
    y = linear_blaslt.forward(x.to(dev), w.to(dev), b.to(dev))
    assert y.shape == (6, 5, 96)
    assert_close(y, x.to(D) @ w.to(D).t() + b.to(D), dtype, "linear forward")
    dx, dw, db = linear_blaslt.backward(x.to(dev), w.to(dev), gy.to(dev), True)
    assert_close(dx, gy.to(D) @ w.to(D), dtype, "linear grad input")
    assert_close(dw, gy.to(D).reshape(30, 96).t() @ x.to(D).reshape(30, 64), dtype, "linear grad weight", scale_atol=True)
    assert_close(db, gy.to(D).reshape(30, 96).sum(0), dtype, "linear grad bias", scale_atol=True)
    assert linear_blaslt.backward(x.to(dev), w.to(dev), gy.to(dev), False)[0] is None


@pytest.mark.parametrize("bias", [True, False])
def test_linear_module_and_frozen_weight(dev, bias):
    torch.manual_seed(12)
    m = Linear(64, 96, bias=bias).to(dev).to(torch.bfloat16)
    ref = torch.nn.Linear(64, 96, bias=bias).double()
    ref.weight.data.copy_(m.weight.detach().cpu())
    if bias:
        ref.bias.data.copy_(m.bias.detach().cpu())
    g = torch.Generator().manual_seed(13)
    x = torch.randn(7, 3, 64, generator=g).to(torch.bfloat16)
    gy = torch.randn(7, 3, 96, generator=g).to(torch.bfloat16)
    xd, xr = x.to(dev).requires_grad_(), x.double().requires_grad_()
    m(xd).backward(gy.to(dev))
    ref(xr).backward(gy.double())
    assert_close(m(xd), ref(xr), torch.bfloat16, "linear module forward")
    assert_close(xd.grad, xr.grad, torch.bfloat16, "grad input")
    assert_close(m.weight.grad, ref.weight.grad, torch.bfloat16, "grad weight", scale_atol=True)
    if bias:
        assert_close(m.bias.grad, ref.bias.grad, torch.bfloat16, "grad bias", scale_atol=True)
    m.zero_grad()
    m.weight.requires_grad_(False)                              # frozen weight: only the input gradient is computed
    x2 = x.to(dev).requires_grad_()
    linear_function(x2, m.weight, m.bias).backward(gy.to(dev))
    assert_close(x2.grad, xr.grad, torch.bfloat16, "grad input, frozen weight")
    assert m.weight.grad is None


NAMES = ("x", "pos", "w_in", "w_out", "w_pos", "b_in", "b_out", "b_pos", "r_w_bias", "r_r_bias")
GRADS = (("x", "dx"), ("w_in", "dw_in"), ("w_out", "dw_out"), ("w_pos", "dw_pos"), ("b_in", "db_in"), ("b_out", "db_out"),
         ("b_pos", "db_pos"), ("r_w_bias", "dr_w_bias"), ("r_r_bias", "dr_r_bias"))


def _run(dev, d, heads, training, use_time_mask, p, return_coverage=True):
    t = {k: d[k].to(dev).requires_grad_() for k in NAMES}
    mask = d["time_mask"] if use_time_mask else d["pad_mask"]
    dm = d["dropout_mask"].to(dev) if (training and p > 0) else None
    res = relative_self_attn_func(t["x"], t["pos"], use_time_mask, training, heads, t["w_in"], t["w_out"], t["w_pos"],
                                  t["b_in"], t["b_out"], t["b_pos"], t["r_w_bias"], t["r_r_bias"],
                                  None if mask is None else mask.to(dev), p, False, None, False, False, return_coverage, False,
                                  dm)
    return t, res


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,b,e,h,len_r,pos_batch,causal,p", [
    (64, 2, 256, 4, None, 1, False, 0.1),      # encoder form: key padding, positions shared over the batch
    (48, 3, 128, 2, 80, 1, False, 0.0),        # more positions than keys (bidirectional 2T-1 style table), no dropout
    (40, 2, 128, 4, None, 2, True, 0.25),      # decoder form: time mask, positions per batch column
    (33, 1, 192, 3, 37, 1, False, 0.1),        # odd lengths: the unvectorised shift kernels, head_dim 64
])
def test_relative_attention_matches_oracle(dev, dtype, t, b, e, h, len_r, pos_batch, causal, p):
    d = inputs.rel_self_attn_inputs(t, b, e, h, dtype, p=p, seed=200 + t, len_r=len_r, pos_batch=pos_batch, causal=causal)
    leaves, (out, cov) = _run(dev, d, h, True, causal, p)
    out.backward(d["dout"].to(dev))
    f = orel.rel_self_attn_fwd(*(d[k] for k in NAMES), h, d["pad_mask"], d["time_mask"], p, d["dropout_mask"], D, round_to=dtype)
    g = orel.rel_self_attn_bwd(d["dout"], d["x"], d["pos"], d["w_in"], d["w_out"], d["w_pos"], h, f, p, d["dropout_mask"], D,
                               round_to=dtype)
    # the scores are rounded three times here (AC, BD, their sum) against once in plain self-attention, so a probability
    # moves by a 16-bit ulp of its score more often than there: at most one output in a thousand (those that cancel to near
    # zero, |out| ~ 1e-2 where the terms are ~ 1) may use an absolute tolerance of 2e-3 instead of 1e-3
    assert_close(out, f["outputs"], dtype, "outputs", flips=2e-3)
    assert_close(cov, f["dropout_results"], dtype, "coverage (dropped probabilities)")
    masked = (d["time_mask"].unsqueeze(0).expand(b * h, t, t) if causal
              else d["pad_mask"].view(b, 1, 1, t).expand(b, h, t, t).reshape(b * h, t, t))
    assert (cov.cpu()[masked] == 0).all()                                   # masked keys: probability exactly zero
    for name, key in GRADS:
        assert_close(leaves[name].grad, g[key], dtype, "grad " + name, scale_atol=name != "x")
    assert leaves["pos"].grad is None                                       # the reference returns no gradient for pos


def test_extension_stand_in_keeps_the_reference_argument_order_and_lists(dev):
    dtype, h, p = torch.bfloat16, 4, 0.1
    d = inputs.rel_self_attn_inputs(32, 2, 128, h, dtype, p=p, seed=31, pos_batch=2)
    a = {k: d[k].to(dev) for k in NAMES}
    pad, dm, dout = d["pad_mask"].to(dev), d["dropout_mask"].to(dev), d["dout"].to(dev)
    res = relative_self_attn_blaslt.forward(True, False, h, a["x"], a["pos"], a["w_in"], a["w_out"], a["w_pos"], a["b_in"],
                                            a["b_out"], a["b_pos"], a["r_w_bias"], a["r_r_bias"], pad, p, dropout_mask=dm)
    lin, pos_lin, scores, dropped, dmask, ctx, out = res
    assert [tuple(t.shape) for t in res] == [(32, 2, 384), (32, 2, 128), (8, 32, 32), (8, 32, 32), (8, 32, 32), (32, 2, 128),
                                             (32, 2, 128)]
    grads = relative_self_attn_blaslt.backward(h, dout, ctx, dropped, scores, lin, pos_lin, a["r_w_bias"], a["r_r_bias"], a["x"],
                                               a["pos"], a["w_in"], a["w_out"], a["w_pos"], dmask, p, pad_mask=pad)
    f = orel.rel_self_attn_fwd(*(d[k] for k in NAMES), h, d["pad_mask"], None, p, d["dropout_mask"], D, round_to=dtype)
    g = orel.rel_self_attn_bwd(d["dout"], d["x"], d["pos"], d["w_in"], d["w_out"], d["w_pos"], h, f, p, d["dropout_mask"], D,
                               round_to=dtype)
    assert_close(lin, f["input_lin_results"], dtype, "input_lin_results")
    assert_close(pos_lin, f["pos_lin_results"], dtype, "pos_lin_results")
    assert_close(ctx, f["matmul2_results"], dtype, "matmul2_results", flips=2e-3)
    finite = torch.isfinite(f["attn_scores"])                  # the stored scores are unmasked; compare where the oracle's are
    assert_close(scores.cpu().float()[finite], f["attn_scores"][finite], dtype, "attn_scores", atol=2e-2)   # one 16-bit ulp at |s| ~ 4
    order = ("dx", "dw_in", "dw_pos", "dw_out", "db_in", "db_pos", "db_out", "dr_w_bias", "dr_r_bias")
    assert len(grads) == 9
    for got, key in zip(grads, order):
        assert_close(got, g[key], dtype, key, scale_atol=key != "dx")


@pytest.mark.parametrize("t,b", [(0, 2), (5, 0)])
def test_empty_batch_gives_empty_results_and_zero_parameter_gradients(dev, t, b):
    d = inputs.rel_self_attn_inputs(5, 2, 64, 2, torch.bfloat16, p=0.0, seed=3)
    a = {k: d[k].to(dev).requires_grad_() for k in NAMES}
    x = d["x"][:t, :b].to(dev).requires_grad_()
    out, cov = relative_self_attn_func(x, a["pos"], False, True, 2, a["w_in"], a["w_out"], a["w_pos"], a["b_in"], a["b_out"], a["b_pos"],
                                       a["r_w_bias"], a["r_r_bias"], None, 0.0, False, None, False, False, True, False)
    assert out.shape == (t, b, 64) and cov.shape == (b * 2, t, t)
    out.float().sum().backward()
    assert x.grad.shape == x.shape
    for k in NAMES[2:]:
        assert a[k].grad is not None and not a[k].grad.any(), k


def test_inference_returns_probabilities_and_single_output_form(dev):
    dtype, h = torch.bfloat16, 4
    d = inputs.rel_self_attn_inputs(32, 2, 128, h, dtype, p=0.3, seed=9)
    f = orel.rel_self_attn_fwd(*(d[k] for k in NAMES), h, d["pad_mask"], None, 0.0, None, D, round_to=dtype)
    with torch.no_grad():
        _, (out, cov) = _run(dev, d, h, False, False, 0.3)
        _, only = _run(dev, d, h, False, False, 0.3, return_coverage=False)
    assert_close(out, f["outputs"], dtype, "inference outputs")
    assert_close(cov, f["softmax_results"], dtype, "inference coverage")
    assert torch.is_tensor(only) and torch.equal(only, out)


def test_module_has_the_reference_parameters_and_runs(dev):
    torch.manual_seed(4)
    m = RelativeSelfMultiheadAttn(128, 4, dropout=0.0).to(dev).to(torch.bfloat16)
    shapes = {k: tuple(v.shape) for k, v in m.named_parameters()}
    assert shapes == {"in_proj_weight": (384, 128), "out_proj_weight": (128, 128), "pos_proj_weight": (128, 128),
                      "pos_proj_bias": (128,), "in_proj_bias": (384,), "out_proj_bias": (128,), "r_w_bias": (4, 32),
                      "r_r_bias": (4, 32)}
    g = torch.Generator().manual_seed(5)
    x = torch.randn(24, 2, 128, generator=g).to(torch.bfloat16)
    pos = torch.randn(24, 1, 128, generator=g).to(torch.bfloat16)
    pad = torch.zeros(2, 24, dtype=torch.bool)
    pad[1, 17:] = True
    out, cov = m(x.to(dev), pos.to(dev), key_padding_mask=pad.t().unsqueeze(0).to(dev))        # the reference's [1, T, B] form
    P = {k: v.detach().cpu() for k, v in m.named_parameters()}
    f = orel.rel_self_attn_fwd(x, pos, P["in_proj_weight"], P["out_proj_weight"], P["pos_proj_weight"], P["in_proj_bias"],
                               P["out_proj_bias"], P["pos_proj_bias"], P["r_w_bias"], P["r_r_bias"], 4, pad, None, 0.0, None, D,
                               round_to=torch.bfloat16)
    assert_close(out, f["outputs"], torch.bfloat16, "module outputs")
    out.float().sum().backward()
    assert all(p.grad is not None for p in m.parameters())


def test_step_by_step_decoding_reproduces_the_causal_rows(dev):
    # Step i feeds one position and the positions of distances i..0; with the keys and values cached it must give row i of
    # the full causal pass (the shift is the identity on a single query row).
    dtype, t, b, e, h = torch.bfloat16, 10, 3, 128, 4
    d = inputs.rel_self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=21, causal=True)
    a = {k: d[k].to(dev) for k in NAMES}
    with torch.no_grad():
        full = relative_self_attn_func(a["x"], a["pos"], True, False, h, a["w_in"], a["w_out"], a["w_pos"], a["b_in"], a["b_out"],
                                       a["b_pos"], a["r_w_bias"], a["r_r_bias"], d["time_mask"].to(dev), 0.0, False, None, False,
                                       False, False, False)
        cache = {}
        for i in range(t):
            if i == 4:                                                     # beam search re-orders the hypotheses
                order = torch.tensor([2, 0, 1], device=dev)
                cache = {k: v.index_select(1, order) for k, v in cache.items()}
                a["x"], full = a["x"].index_select(1, order), full.index_select(1, order)
            step, cov = relative_self_attn_func(a["x"][i:i + 1], a["pos"][t - 1 - i:], False, False, h, a["w_in"], a["w_out"],
                                                a["w_pos"], a["b_in"], a["b_out"], a["b_pos"], a["r_w_bias"], a["r_r_bias"], None,
                                                0.0, True, cache, False, False, True, False)
            assert step.shape == (1, b, e) and cov.shape == (b * h, 1, i + 1) and cache["k"].shape == (i + 1, b, e)
            assert_close(step[0], full[i].float().cpu(), dtype, f"step {i}", flips=2e-3)
    with pytest.raises(RuntimeError):
        relative_self_attn_func(a["x"][:1], a["pos"], False, True, h, a["w_in"], a["w_out"], a["w_pos"], a["b_in"], a["b_out"],
                                a["b_pos"], a["r_w_bias"], a["r_r_bias"], None, 0.0, True, {}, False, False, True, False)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape,view", [((6, 8, 3, 16), "queries"), ((40, 24), "dense"), ((5, 7), "odd"), ((0, 8), "empty")])
def test_row_add_on_dense_and_pitched_rows(dev, dtype, shape, view):
    g = torch.Generator().manual_seed(len(shape))
    a, b = torch.randint(-8, 9, shape, generator=g).to(dtype), torch.randint(-8, 9, shape, generator=g).to(dtype)
    ad, bd = a.to(dev), b.to(dev)
    if view == "queries":                                       # the sum lands inside a [T, B*H, 3, D] gradient tensor
        out = torch.full(shape, 99, dtype=dtype, device=dev)
        got = relative_position.add_rows(ad[:, :, 0, :].contiguous(), bd[:, :, 1, :], out=out[:, :, 0, :])
        assert torch.equal(out[:, :, 0, :].cpu(), a[:, :, 0, :] + b[:, :, 1, :]) and (out[:, :, 1:, :] == 99).all()
        assert got.data_ptr() == out.data_ptr()
        with pytest.raises(RuntimeError):
            relative_position.add_rows(ad.transpose(0, 1)[:, :, 0, :], bd.transpose(0, 1)[:, :, 0, :])
    else:
        assert torch.equal(relative_position.add_rows(ad, bd).cpu(), a + b)
        assert torch.equal(relative_position.add_rows(ad, bd, out=ad).cpu(), a + b)          # in place


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,b,e,h,causal,p", [(48, 2, 128, 2, False, 0.1), (33, 3, 192, 3, True, 0.0)])
def test_learnable_position_attention_matches_oracle(dev, dtype, t, b, e, h, causal, p):
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=p, seed=300 + t, zero_bias=False, causal=causal)
    pos = (0.5 * torch.randn(t, t, e // h, generator=torch.Generator().manual_seed(t))).to(dtype)
    names = ("x", "w_in", "w_out", "b_in", "b_out")
    leaves = {k: d[k].to(dev).requires_grad_() for k in names}
    pl = pos.to(dev).requires_grad_()
    mask = d["time_mask"] if causal else d["pad_mask"]
    dm = d["dropout_mask"].to(dev) if p > 0 else None
    out, cov = relative_self_attn_func(leaves["x"], pl, causal, True, h, leaves["w_in"], leaves["w_out"], None, leaves["b_in"],
                                       leaves["b_out"], None, None, None, mask.to(dev), p, False, None, False, True, True,
                                       False, dm)
    out.backward(d["dout"].to(dev))
    # The HIP path stores the second score term in 16 bits before the sum; the reference accumulates it in fp32 into the
    # stored first term. The oracle models the first (round_bd=True) for the comparison at the 16-bit tolerance; against
    # the reference's own rounding points the outputs agree to 5e-3 absolute (a score whose final rounding flips moves its
    # probability by 2^-8 relative, which shows in outputs that cancel to near zero).
    args = (d["x"], pos, d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"], p, d["dropout_mask"], D)
    f = orel.rel_learnable_attn_fwd(*args, round_to=dtype, round_bd=True)
    g = orel.rel_learnable_attn_bwd(d["dout"], d["x"], pos, d["w_in"], d["w_out"], h, f, p, d["dropout_mask"], D, round_to=dtype)
    assert_close(out, orel.rel_learnable_attn_fwd(*args, round_to=dtype)["outputs"], dtype, "outputs, reference rounding", atol=5e-3)
    assert_close(out, f["outputs"], dtype, "outputs", flips=2e-3)
    assert_close(cov, f["dropout_results"], dtype, "coverage")
    for k, gk in (("x", "dx"), ("w_in", "dw_in"), ("w_out", "dw_out"), ("b_in", "db_in"), ("b_out", "db_out")):
        assert_close(leaves[k].grad, g[gk], dtype, "grad " + k, scale_atol=k != "x")
    assert_close(pl.grad, g["dpos"], dtype, "grad pos", scale_atol=True)


def test_module_with_learnable_positions(dev):
    torch.manual_seed(6)
    m = RelativeSelfMultiheadAttn(128, 4, dropout=0.0, learnable_pos=True, max_pos=16).to(dev).to(torch.bfloat16)
    assert m.pos_proj_weight is None and tuple(m.pos_emb.weight.shape) == (33, 32)
    t = 12
    x = torch.randn(t, 2, 128, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16)
    dist = (torch.arange(t).view(t, 1) - torch.arange(t).view(1, t)).clamp(-16, 16) + 16           # [T, T] distance indices
    out, cov = m(x.to(dev), dist.to(dev))
    P = {k: v.detach().cpu() for k, v in m.named_parameters()}
    f = orel.rel_learnable_attn_fwd(x, P["pos_emb.weight"][dist], P["in_proj_weight"], P["out_proj_weight"], P["in_proj_bias"],
                                    P["out_proj_bias"], 4, None, None, 0.0, None, D, round_to=torch.bfloat16, round_bd=True)
    assert_close(out, f["outputs"], torch.bfloat16, "module outputs", flips=2e-3)
    out.float().sum().backward()
    assert m.pos_emb.weight.grad is not None and m.in_proj_weight.grad is not None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("prefix", [1, 5])
def test_learnable_positions_step_by_step(dev, dtype, prefix):
    """Incremental decoding with learnable positions (relative_self_attention_func.py:187-204, :254-263): a prefix in one
    call, then one position per call onto the cache, each with the [new queries, all keys] rows of the distance table.
    Every decoded row is the row of the oracle's causal full-sequence result."""
    torch.manual_seed(8)
    t, b, e, h, max_pos = 11, 3, 128, 4, 16
    m = RelativeSelfMultiheadAttn(e, h, dropout=0.0, learnable_pos=True, max_pos=max_pos).to(dev).to(dtype).eval()
    x = torch.randn(t, b, e, generator=torch.Generator().manual_seed(9)).to(dtype)
    dist = (torch.arange(t).view(t, 1) - torch.arange(t).view(1, t)).clamp(-max_pos, max_pos) + max_pos
    causal = torch.ones(t, t, dtype=torch.bool).triu(1)
    P = {k: v.detach().cpu() for k, v in m.named_parameters()}
    want = orel.rel_learnable_attn_fwd(x, P["pos_emb.weight"][dist], P["in_proj_weight"], P["out_proj_weight"], P["in_proj_bias"],
                                       P["out_proj_bias"], h, None, causal, 0.0, None, D, round_to=dtype, round_bd=True)
    cache, rows, covs = {}, [], []
    with torch.no_grad():
        lo = 0
        for hi in [prefix] + list(range(prefix + 1, t + 1)):
            out, cov = m(x[lo:hi].to(dev), dist[lo:hi, :hi].to(dev), None, causal[lo:hi, :hi].to(dev), incremental=True,
                         incremental_cache=cache)
            assert out.shape == (hi - lo, b, e) and cov.shape == (b * h, hi - lo, hi) and cache["k"].shape == (hi, b, e)
            rows.append(out)
            covs.append(cov)
            lo = hi
    assert_close(torch.cat(rows, 0), want["outputs"], dtype, "decoded rows", flips=2e-3)
    for i, cov in enumerate(covs[1:], start=prefix):
        assert_close(cov[:, 0, :], want["dropout_results"][:, i, :i + 1], dtype, f"coverage of step {i}")
    with pytest.raises(RuntimeError):
        m(x[:1].to(dev), dist[:1, :3].to(dev), None, None, incremental=True, incremental_cache={})     # table wider than the keys


def test_relative_attention_golden_fixture(dev):
    # tests/golden/relative_attention.npz: the shift as an explicit gather, fp64 autograd with the bf16 rounding points
    BF = torch.bfloat16
    f = load_golden("relative_attention")
    p, h = float(f["p"]), int(f["heads"])
    names = ("x", "pos", "w_in", "w_out", "w_pos", "b_in", "b_out", "b_pos", "r_w_bias", "r_r_bias")
    t = {k: f[k].to(BF).to(dev).requires_grad_() for k in names}
    out, cov = relative_self_attn_func(t["x"], t["pos"], False, True, h, t["w_in"], t["w_out"], t["w_pos"], t["b_in"],
                                       t["b_out"], t["b_pos"], t["r_w_bias"], t["r_r_bias"], f["pad_mask"].bool().to(dev), p,
                                       False, None, False, False, True, False, f["dropout_mask"].to(dev))
    out.backward(f["dout"].to(BF).to(dev))
    assert_close(out, f["outputs"], BF, "outputs", flips=2e-3)      # scores rounded three times (AC, BD, sum): see the op's test
    assert_close(cov, f["dropout_results"], BF, "dropout_results")
    for k, gk in (("x", "dx"), ("w_in", "dw_in"), ("w_out", "dw_out"), ("w_pos", "dw_pos"), ("b_in", "db_in"),
                  ("b_out", "db_out"), ("b_pos", "db_pos"), ("r_w_bias", "dr_w_bias"), ("r_r_bias", "dr_r_bias")):
        assert_close(t[k].grad, f[gk], BF, gk, scale_atol=True)


@pytest.mark.parametrize("seed", range(2000, 2016))
def test_randomly_drawn_shapes(dev, seed):
    # sizes nobody picked by hand: the drawn case is part of the failure message
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
    g = torch.Generator().manual_seed(seed)
    b, tq = rnd.choice([1, 2, 5]), rnd.choice([1, 2, 7, 16, 33, 64, 100])
    tk = rnd.choice([t for t in (1, 3, 8, 16, 31, 64, 100) if t <= max(tq, 1) * 4])
    r = tk + rnd.choice([0, 0, 1, 5, 8, 29])
    case = f"seed {seed}: {dtype} batch {b} len_q {tq} len_k {tk} len_r {r}"
    ac = torch.randint(-8, 9, (b, tq, tk), generator=g).to(dtype)
    bd = torch.randint(-8, 9, (b, tq, r), generator=g).to(dtype)
    got = relative_position.shift_add_(ac.clone().to(dev), bd.to(dev))
    assert torch.equal(got.cpu().to(D), ac.to(D) + orel.relative_shift(bd.to(D))[:, :, :tk]), case
    back = relative_position.shift_backward(ac.to(dev), r)
    full = torch.cat([ac.to(D), torch.zeros(b, tq, r - tk, dtype=D)], dim=-1)
    assert torch.equal(back.cpu().to(D), orel.relative_shift_bwd(full)), case
    rows, cols, pad = rnd.choice([1, 3, 64, 129, 700]), rnd.choice([1, 8, 24, 100, 513]), rnd.choice([0, 0, 3, 8])
    x = torch.randn(rows, cols + pad, generator=g).to(dtype)
    assert_close(linear_gemm.colsum(x.to(dev)[:, :cols]), x[:, :cols].to(D).sum(0), dtype, case + f" colsum {rows}x{cols}+{pad}",
                 scale_atol=True)
    y = torch.randint(-8, 9, (rows, cols + pad), generator=g).to(dtype)
    xi = torch.randint(-8, 9, (rows, cols + pad), generator=g).to(dtype)
    assert torch.equal(relative_position.add_rows(xi.to(dev)[:, :cols], y.to(dev)[:, :cols]).cpu(), (xi + y)[:, :cols]), case
    if dtype != torch.float32:
        h, dh = rnd.choice([1, 2, 4]), rnd.choice([32, 64])
        t, bsz, p, causal = rnd.choice([1, 2, 9, 33, 70]), rnd.choice([1, 2, 3]), rnd.choice([0.0, 0.1]), rnd.random() < 0.4
        len_r = t + rnd.choice([0, 0, 3, 17])
        case += f"; attention T {t} B {bsz} H {h} D {dh} R {len_r} p {p} causal {causal}"
        d = inputs.rel_self_attn_inputs(t, bsz, h * dh, h, dtype, p=p, seed=seed, len_r=len_r, pos_batch=rnd.choice([1, bsz]),
                                        causal=causal)
        leaves, (out, cov) = _run(dev, d, h, True, causal, p)
        out.backward(d["dout"].to(dev))
        f = orel.rel_self_attn_fwd(*(d[k] for k in NAMES), h, d["pad_mask"], d["time_mask"], p, d["dropout_mask"], D, round_to=dtype)
        gr = orel.rel_self_attn_bwd(d["dout"], d["x"], d["pos"], d["w_in"], d["w_out"], d["w_pos"], h, f, p, d["dropout_mask"], D,
                                    round_to=dtype)
        assert_close(out, f["outputs"], dtype, case + " outputs", flips=2e-3)
        for name, key in GRADS:
            assert_close(leaves[name].grad, gr[key], dtype, case + " grad " + name, scale_atol=True)
