"""Strided (non-contiguous) arguments: every stand-in either gives exactly the result it gives for dense tensors, or
refuses. The C entry points read dense arrays, so a stand-in copies a strided argument first — and has to keep the
copy alive until the kernels are queued (a copy held only by the expression that takes its address is freed at once;
the kernels would then read whatever reuses that memory)."""
import pytest
import torch

from nmtgminor_amd.native import (encdec_multihead_attn_bias_blaslt as ed, fast_layer_norm_cuda as ln, fused_dropout_add_cuda as da,
                                  fused_mlp_gelu, mask_softmax_dropout_cuda as sm, self_multihead_attn_blaslt as sa, xentropy_cuda)
from oracle import inputs

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def strided(t, dev):
    """The values of `t` on `dev`, stored with an innermost stride of 2."""
    if t is None:
        return None
    big = torch.empty(*t.shape[:-1], t.shape[-1] * 2, dtype=t.dtype, device=dev)
    view = big[..., ::2]
    view.copy_(t)
    assert not view.is_contiguous() or view.numel() <= 1
    return view


def same(got, want, what):
    for i, (a, b) in enumerate(zip(got, want)):
        if a is None or b is None:
            assert a is None and b is None, (what, i)
        else:
            assert torch.equal(a, b), (what, i)


def test_self_attention_takes_strided_tensors(dev):
    t, b, e, h = 24, 2, 128, 2
    d = inputs.self_attn_inputs(t, b, e, h, BF, p=0.1, seed=3, zero_bias=False)
    g = lambda k: d[k].to(dev)
    s = lambda k: strided(d[k], dev)
    ref = sa.forward(False, True, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.1, dropout_mask=g("dropout_mask"))
    got = sa.forward(False, True, h, s("x"), s("w_in"), s("w_out"), s("b_in"), s("b_out"), g("pad_mask"), 0.1, dropout_mask=s("dropout_mask"))
    same(got, ref, "forward")
    lin, sc, dr, dm, ctx, out = ref
    want = sa.backward(False, h, g("dout"), ctx, dr, sc, lin, g("x"), g("w_in"), g("w_out"), dm, 0.1)
    z = lambda v: strided(v.cpu(), dev)
    got = sa.backward(False, h, s("dout"), z(ctx), z(dr), z(sc), z(lin), s("x"), s("w_in"), s("w_out"), z(dm), 0.1)
    same(got, want, "backward")


def test_cross_attention_takes_strided_tensors(dev):
    tq, tk, b, e, h = 9, 40, 2, 128, 2
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, BF, p=0.0, seed=6, zero_bias=False)
    g = lambda k: d[k].to(dev)
    s = lambda k: strided(d[k], dev)
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out", "b_q", "b_kv", "b_out")
    ref = ed.forward(True, h, *[g(k) for k in names], g("pad_mask"), 0.0)
    got = ed.forward(True, h, *[s(k) for k in names], g("pad_mask"), 0.0)
    same(got, ref, "forward")
    q_lin, kv_lin, sc, dr, dm, ctx, out = ref
    z = lambda v: strided(v.cpu(), dev)
    want = ed.backward(h, g("dout"), ctx, dr, sc, q_lin, kv_lin, g("x_q"), g("x_kv"), g("w_q"), g("w_kv"), g("w_out"), dm, 0.0)
    got = ed.backward(h, s("dout"), z(ctx), z(dr), z(sc), z(q_lin), z(kv_lin), s("x_q"), s("x_kv"), s("w_q"), s("w_kv"), s("w_out"), dm, 0.0)
    same(got, want, "backward")


def test_mlp_and_cross_entropy_take_strided_tensors(dev):
    m = inputs.mlp_inputs(64, 128, 256, BF, p=0.1, seed=4, zero_bias=False)
    names = ("x", "w1", "w2", "b1", "b2")
    ins = [m[k].to(dev) for k in names]
    ins[0].requires_grad_()
    ref = fused_mlp_gelu.forward(0.1, ins, m["mask"].to(dev))
    ins2 = [strided(m[k], dev) for k in names]
    ins2[0].requires_grad_()
    got = fused_mlp_gelu.forward(0.1, ins2, strided(m["mask"], dev))
    same(got, ref, "mlp forward")
    want = fused_mlp_gelu.backward(0.1, m["dy"].to(dev), ref, ins)
    got = fused_mlp_gelu.backward(0.1, strided(m["dy"], dev), [strided(v.cpu(), dev) for v in ref], ins2)
    same(got, want, "mlp backward")
    x = inputs.xentropy_inputs(16, 1000, BF, 0.1, 1, 0.1, seed=5)
    ref = xentropy_cuda.forward(x["logits"].to(dev), x["labels"].to(dev), 0.1, True, padding_idx=1)
    got = xentropy_cuda.forward(strided(x["logits"], dev), strided(x["labels"], dev), 0.1, True, padding_idx=1)
    same(got, ref, "cross-entropy forward")
    want = xentropy_cuda.backward(x["grad_loss"].to(dev), x["logits"].to(dev), ref[1], x["labels"].to(dev), 0.1, padding_idx=1)
    got = xentropy_cuda.backward(strided(x["grad_loss"], dev), strided(x["logits"], dev), strided(ref[1].cpu(), dev),
                                 strided(x["labels"], dev), 0.1, padding_idx=1)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("v,pitch,gpitch", [(1000, 1024, 1024), (517, 520, 576), (250, 251, 250)])
def test_cross_entropy_reads_and_writes_row_pitched_logits_in_place(dev, dtype, v, pitch, gpitch):
    # rows of `v` classes inside wider buffers: nothing is copied, and nothing beyond a row's classes is touched
    x = inputs.xentropy_inputs(12, v, dtype, 0.1, 1, 0.25, seed=6)
    big = torch.full((12, pitch), float("nan"), dtype=dtype, device=dev)
    view = big[:, :v]
    view.copy_(x["logits"])
    labels, gl = x["labels"].to(dev), x["grad_loss"].to(dev)
    widen = dtype != torch.float32
    ref = xentropy_cuda.forward(x["logits"].to(dev), labels, 0.1, widen, padding_idx=1)
    got = xentropy_cuda.forward(view, labels, 0.1, widen, padding_idx=1)
    # the reduction order within a row depends on where its 16-byte boundaries fall: equal to rounding
    for a, b in zip(got, ref):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)
    pad = x["labels"] == 1
    assert pad.any() and (got[0].cpu()[pad] == 0).all()
    want = xentropy_cuda.backward(gl, x["logits"].to(dev), ref[1], labels, 0.1, padding_idx=1)
    gbig = torch.full((12, gpitch), 7.0, dtype=dtype, device=dev)
    out = xentropy_cuda.backward(gl, view, ref[1], labels, 0.1, padding_idx=1, out=gbig[:, :v])
    assert out.data_ptr() == gbig.data_ptr() and torch.equal(out, want)                 # elementwise: bit for bit
    assert (gbig[:, v:] == 7.0).all() and (gbig.cpu()[pad][:, :v] == 0).all()
    with pytest.raises(RuntimeError):
        xentropy_cuda.backward(gl, view, ref[1], labels, 0.1, padding_idx=1, out=gbig[:, :v - 1])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_cross_entropy_backward_on_a_slice_of_the_classes(dev, dtype):
    # given the log-sum-exp of the whole row the backward is elementwise: any column slice gives the full result's columns
    v = 1000
    x = inputs.xentropy_inputs(10, v, dtype, 0.1, 1, 0.2, seed=8)
    logits, labels, gl = x["logits"].to(dev), x["labels"].to(dev), x["grad_loss"].to(dev)
    _, lse = xentropy_cuda.forward(logits, labels, 0.1, dtype != torch.float32, padding_idx=1)
    want = xentropy_cuda.backward(gl, logits, lse, labels, 0.1, padding_idx=1)
    for c0, c1 in ((0, 384), (384, 768), (768, 1000), (123, 130)):
        got = xentropy_cuda.backward(gl, logits[:, c0:c1], lse, labels, 0.1, padding_idx=1, class_offset=c0, total_classes=v)
        assert got.shape == (10, c1 - c0) and torch.equal(got, want[:, c0:c1]), (c0, c1)
    with pytest.raises(RuntimeError):
        xentropy_cuda.backward(gl, logits[:, 900:], lse, labels, 0.1, padding_idx=1, class_offset=950, total_classes=v)


def test_operators_that_work_in_place_or_on_rows_refuse_strided_tensors(dev):
    x = strided(torch.randn(8, 64), dev)
    w = torch.ones(64, device=dev)
    with pytest.raises(RuntimeError):
        ln.ln_fwd(x, w, w, 1e-5)
    with pytest.raises(RuntimeError):
        da.forward(True, x, x, 0.1)                      # the result is written into the first argument
    with pytest.raises(RuntimeError):
        sm.forward(False, 1, strided(torch.randn(2, 4, 16), dev), 0.0)
    # their remaining arguments may be strided
    g = strided(torch.randn(8, 64), dev)
    mask = strided((torch.rand(8, 64) < 0.9).to(torch.uint8), dev)
    want = da.backward(g.contiguous(), mask.contiguous(), 0.1)
    assert torch.equal(da.backward(g, mask, 0.1), want)
