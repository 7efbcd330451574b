"""The Python side of the build, end to end, without a GPU.

The C entry points are answered by tests/emulated_lib.py (oracle arithmetic written into the
caller's buffers), so what is under test here is everything ABOVE the C ABI: the stand-in modules'
argument order and buffer shapes, in-place aliasing, the autograd Functions' saved tensors and
gradient arity (the reference's contracts: SelfAttnFunc 18 inputs, EncdecAttnBiasFunc 21,
MlpFunction (p, recompute, mask, x, W.., b..)), the nn.Modules' parameter names. Expected values
come from PyTorch's own library routines and autograd, not from the oracle, so a swapped pair of
arguments anywhere in the stack shows up as a wrong number.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import emulated_lib
from nmtgminor_amd.modules import mlp as mmlp
from nmtgminor_amd.modules.attention_softmax import AttentionSoftmaxDropout
from nmtgminor_amd.modules.dropout_add import fused_dropout_add
from nmtgminor_amd.modules.encdec_attention import EncdecMultiheadAttn
from nmtgminor_amd.modules.encdec_attention_func_bias import encdec_attn_bias_compact_func, encdec_attn_bias_func
from nmtgminor_amd.modules.feed_forward import PositionWiseFeedForward
from nmtgminor_amd.modules.layer_norm import LayerNorm, fast_layer_norm_affine
from nmtgminor_amd.modules.self_attention import SelfMultiheadAttn
from nmtgminor_amd.modules.self_attention_func import self_attn_compact_func, self_attn_func
from nmtgminor_amd.modules.softmax_xentropy import SoftmaxCrossEntropyLoss
from util import assert_close

D = torch.float64
BF = torch.bfloat16


@pytest.fixture(autouse=True)
def emu(monkeypatch):
    emulated_lib.install(monkeypatch)


def gen(seed):
    return torch.Generator().manual_seed(seed)


def close16(actual, expected, what):
    """bf16 results of the stand-ins (intermediates rounded to bf16 as the kernels round them) against an
    unrounded fp64 reference: this file checks plumbing, so the tolerance leaves room for that rounding."""
    assert_close(actual, expected, BF, what, rtol=6e-2, atol=1e-2, scale_atol=True)


def bf(t):
    return t.to(BF)


# ------------------------------------------------------------------------------------------ LayerNorm
@pytest.mark.parametrize("memory_efficient", [False, True])
def test_layer_norm_function_and_module(memory_efficient):
    g = gen(1)
    x = torch.randn(5, 3, 48, generator=g)
    gamma, beta = 1 + 0.1 * torch.randn(48, generator=g), 0.1 * torch.randn(48, generator=g)
    dy = torch.randn(5, 3, 48, generator=g)
    leaves = [t.clone().requires_grad_() for t in (x, gamma, beta)]
    y = fast_layer_norm_affine(leaves[0], leaves[1], leaves[2], (48,), 1e-5, memory_efficient) \
        if memory_efficient else fast_layer_norm_affine(leaves[0], leaves[1], leaves[2], (48,), 1e-5)
    y.backward(dy)
    ref = [t.clone().double().requires_grad_() for t in (x, gamma, beta)]
    F.layer_norm(ref[0], (48,), ref[1], ref[2], 1e-5).backward(dy.double())
    assert_close(y, F.layer_norm(x.double(), (48,), gamma.double(), beta.double(), 1e-5), torch.float32, "y", atol=1e-5)
    for a, r, n in zip(leaves, ref, ("dx", "dgamma", "dbeta")):
        assert_close(a.grad, r.grad, torch.float32, n, atol=1e-5, scale_atol=True)
    m = LayerNorm(48)
    assert sorted(m.state_dict()) == ["bias", "weight"]
    assert m(x).shape == x.shape


# ------------------------------------------------------------------------------------------ dropout + add
def test_fused_dropout_add_aliases_its_input_and_routes_both_gradients():
    g = gen(2)
    x = torch.randn(7, 12, generator=g)
    r = torch.randn(7, 12, generator=g).requires_grad_()
    mask = (torch.rand(7, 12, generator=g) < 0.7).to(torch.uint8)
    go = torch.randn(7, 12, generator=g)
    xin = x.clone().requires_grad_()
    pre = xin * 1.0
    out = fused_dropout_add(pre, r, 0.3, True, mask)
    assert out.data_ptr() == pre.data_ptr()                       # in place, as the reference
    out.backward(go)
    assert_close(out, x.double() * mask.double() / 0.7 + r.detach().double(), torch.float32, "out")
    assert_close(xin.grad, go.double() * mask.double() / 0.7, torch.float32, "dx")
    assert torch.equal(r.grad, go)
    out2 = fused_dropout_add(x.clone(), r.detach(), 0.3, False)       # eval: plain add
    assert_close(out2, x.double() + r.detach().double(), torch.float32, "eval")


# ------------------------------------------------------------------------------------------ cross-entropy
def test_softmax_cross_entropy_function():
    g = gen(3)
    logits = (2 * torch.randn(11, 29, generator=g)).requires_grad_()
    labels = torch.randint(0, 29, (11,), generator=g)
    labels[3] = 1
    w = torch.rand(11, generator=g) + 0.5
    losses = SoftmaxCrossEntropyLoss.apply(logits, labels, 0.1, 1, False)
    (losses * w).sum().backward()
    ref = logits.detach().double().requires_grad_()
    want = F.cross_entropy(ref, labels, reduction="none", label_smoothing=0.1, ignore_index=1)
    (want * w.double()).sum().backward()
    assert_close(losses, want, torch.float32, "losses", rtol=2e-5, atol=2e-5)
    assert_close(logits.grad, ref.grad, torch.float32, "dlogits", atol=1e-6)
    assert losses[3] == 0 and (logits.grad[3] == 0).all()


# ------------------------------------------------------------------------------------------ softmax wrapper
def test_attention_softmax_dropout_wrapper():
    g = gen(4)
    s = torch.randn(4, 5, 12, generator=g)
    mask, sm, dr = AttentionSoftmaxDropout.forward(s, False, 0.0, False, 2)
    assert_close(dr, F.softmax(s.double(), -1), torch.float32, "softmax")
    go = torch.randn(4, 5, 12, generator=g)
    ds = AttentionSoftmaxDropout.backward(go, sm, torch.tensor([0.0]), torch.tensor([2]), mask)
    ref = s.double().requires_grad_()
    F.softmax(ref, -1).backward(go.double())
    assert_close(ds, ref.grad, torch.float32, "dscores", atol=1e-5)


# ------------------------------------------------------------------------------------------ fused MLP
ACTS = {"gelu": F.gelu, "relu": F.relu, "silu": F.silu, "agelu": lambda h: F.gelu(h, approximate="tanh")}


@pytest.mark.parametrize("act", sorted(ACTS))
def test_mlp_functions(act):
    g = gen(5)
    x, w1, w2 = bf(torch.randn(12, 16, generator=g)), bf(torch.randn(24, 16, generator=g) / 4), bf(torch.randn(16, 24, generator=g) / 5)
    b1, b2 = bf(0.1 * torch.randn(24, generator=g)), bf(0.1 * torch.randn(16, generator=g))
    mask = (torch.rand(12, 24, generator=g) < 0.8).to(torch.uint8)
    dy = bf(torch.randn(12, 16, generator=g))
    leaves = [t.clone().requires_grad_() for t in (x, w1, w2, b1, b2)]
    y = getattr(mmlp, f"mlp_{act}_function")(0.2, False, *leaves, mask=mask)
    y.backward(dy)
    ref = [t.double().requires_grad_() for t in (x, w1, w2, b1, b2)]
    h = ACTS[act](F.linear(ref[0], ref[1], ref[3])) * mask.double() / 0.8
    yr = F.linear(h, ref[2], ref[4])
    yr.backward(dy.double())
    close16(y, yr, "y")
    for a, r, n in zip(leaves, ref, ("dx", "dW1", "dW2", "db1", "db2")):
        close16(a.grad, r.grad, n)


def test_position_wise_feed_forward_module():
    ff = PositionWiseFeedForward(16, 32, dropout=0.0, activation="gelu").to(BF)
    assert sorted(ff.state_dict()) == ["in_proj_bias", "in_proj_weight", "out_proj_bias", "out_proj_weight"]
    x = bf(torch.randn(5, 2, 16, generator=gen(6)))
    y = ff.eval()(x)
    want = F.linear(F.gelu(F.linear(x.double(), ff.in_proj_weight.double(), ff.in_proj_bias.double())),
                    ff.out_proj_weight.double(), ff.out_proj_bias.double())
    close16(y, want, "ffn")


# ------------------------------------------------------------------------------------------ attention
def _self_reference(x, w_in, w_out, b_in, b_out, h, pad, tm, dm, p, dout):
    t, b, e = x.shape
    d = e // h
    leaves = [z.double().requires_grad_() for z in (x, w_in, w_out, b_in, b_out)]
    lin = F.linear(leaves[0], leaves[1], leaves[3]).view(t, b * h, 3, d)       # rows of W_in: (head, {q,k,v}, head_dim)
    q, k, v = [lin[:, :, i].transpose(0, 1) for i in range(3)]               # [B*H, T, D]
    s = q @ k.transpose(1, 2) / math.sqrt(d)
    if pad is not None:
        s = s.view(b, h, t, t).masked_fill(pad.view(b, 1, 1, t), float("-inf")).view(b * h, t, t)
    if tm is not None:
        s = s.masked_fill(tm.view(1, t, t), float("-inf"))
    pr = F.softmax(s, -1)
    if dm is not None:
        pr = pr * dm.double() / (1 - p)
    ctx = (pr @ v).transpose(0, 1).reshape(t, b, e)
    out = F.linear(ctx, leaves[2], leaves[4])
    out.backward(dout.double())
    return out.detach(), pr.detach(), [z.grad for z in leaves]


@pytest.mark.parametrize("causal", [False, True])
def test_self_attention_function(causal):
    g = gen(7)
    t, b, e, h, p = 7, 2, 32, 2, 0.25
    x = bf(torch.randn(t, b, e, generator=g))
    w_in, w_out = bf(torch.randn(3 * e, e, generator=g) / 6), bf(torch.randn(e, e, generator=g) / 6)
    b_in, b_out = bf(0.1 * torch.randn(3 * e, generator=g)), bf(0.1 * torch.randn(e, generator=g))
    pad = torch.arange(t).unsqueeze(0) >= torch.tensor([[5], [7]])
    tm = torch.triu(torch.ones(t, t), 1).bool()
    dm = (torch.rand(b * h, t, t, generator=g) < 0.75).to(torch.uint8)
    dout = bf(torch.randn(t, b, e, generator=g))
    leaves = [z.clone().requires_grad_() for z in (x, w_in, w_out, b_in, b_out)]
    out, cov = self_attn_func(causal, True, h, leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], tm if causal else pad, p,
                              False, None, False, None, True, True, False, dm)
    out.backward(dout)
    want, pr, grads = _self_reference(x, w_in, w_out, b_in, b_out, h, None if causal else pad, tm if causal else None, dm, p, dout)
    close16(out, want, "outputs")
    close16(cov, pr, "coverage")
    for a, r, n in zip(leaves, grads, ("dx", "dW_in", "dW_out", "db_in", "db_out")):
        close16(a.grad, r, n)
    # compact form: projection outside, context out, gradient of the projection's output back
    lin = F.linear(x.float(), w_in.float(), b_in.float()).to(BF).requires_grad_()
    ctx, cov2 = self_attn_compact_func(causal, True, h, lin, tm if causal else pad, p, False, None, False, None, True, True, False, dm)
    assert ctx.shape == (t, b, e) and cov2.shape == (b * h, t, t)
    ctx.backward(dout)
    assert lin.grad.shape == lin.shape and torch.isfinite(lin.grad.float()).all()


def test_encdec_attention_function():
    g = gen(8)
    tq, tk, b, e, h, p = 5, 9, 2, 32, 2, 0.2
    d = e // h
    mk = lambda *s, sc=1.0: bf(sc * torch.randn(*s, generator=g))
    x_q, x_kv = mk(tq, b, e), mk(tk, b, e)
    w_q, w_kv, w_out = mk(e, e, sc=1 / 6), mk(2 * e, e, sc=1 / 6), mk(e, e, sc=1 / 6)
    b_q, b_kv, b_out = mk(e, sc=0.1), mk(2 * e, sc=0.1), mk(e, sc=0.1)
    pad = torch.arange(tk).unsqueeze(0) >= torch.tensor([[9], [6]])
    dm = (torch.rand(b * h, tq, tk, generator=g) < 0.8).to(torch.uint8)
    dout = mk(tq, b, e)
    names = ("x_q", "x_kv", "w_q", "w_kv", "w_out", "b_q", "b_kv", "b_out")
    vals = (x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out)
    leaf = {n: z.clone().requires_grad_() for n, z in zip(names, vals)}
    out, cov = encdec_attn_bias_func(False, True, h, leaf["x_q"], leaf["x_kv"], leaf["w_q"], leaf["w_kv"], leaf["w_out"],
                                     leaf["b_q"], leaf["b_kv"], leaf["b_out"], pad, p, False, None, False, None, None, True, True,
                                     dm)
    out.backward(dout)
    ref = {n: z.double().requires_grad_() for n, z in zip(names, vals)}
    q = F.linear(ref["x_q"], ref["w_q"], ref["b_q"]).view(tq, b * h, d).transpose(0, 1)
    kv = F.linear(ref["x_kv"], ref["w_kv"], ref["b_kv"]).view(tk, b * h, 2, d)            # rows of W_kv: (head, {k,v}, head_dim)
    k, v = kv[:, :, 0].transpose(0, 1), kv[:, :, 1].transpose(0, 1)
    s = (q @ k.transpose(1, 2) / math.sqrt(d)).view(b, h, tq, tk).masked_fill(pad.view(b, 1, 1, tk), float("-inf"))
    pr = F.softmax(s.view(b * h, tq, tk), -1) * dm.double() / (1 - p)
    want = F.linear((pr @ v).transpose(0, 1).reshape(tq, b, e), ref["w_out"], ref["b_out"])
    want.backward(dout.double())
    close16(out, want, "outputs")
    close16(cov, pr, "coverage")
    for n in names:
        close16(leaf[n].grad, ref[n].grad, "d" + n)
    # compact form
    q_lin = F.linear(x_q.float(), w_q.float(), b_q.float()).to(BF).requires_grad_()
    kv_lin = F.linear(x_kv.float(), w_kv.float(), b_kv.float()).to(BF).requires_grad_()
    ctx, cov2 = encdec_attn_bias_compact_func(False, True, h, q_lin, kv_lin, pad, p, False, None, False, None, None, True, True, dm)
    ctx.backward(dout)
    assert q_lin.grad.shape == q_lin.shape and kv_lin.grad.shape == kv_lin.shape


def test_attention_modules_parameter_names_and_shapes():
    sa = SelfMultiheadAttn(32, 2, dropout=0.0).to(BF)
    assert sorted(sa.state_dict()) == ["in_proj_bias", "in_proj_weight", "out_proj_bias", "out_proj_weight"]
    assert sa.in_proj_weight.shape == (96, 32)
    x = bf(torch.randn(6, 3, 32, generator=gen(9)))
    pad = torch.zeros(3, 6, dtype=torch.bool)
    pad[1, 4:] = True
    y, cov = sa(x, None, key_padding_mask=pad)
    assert y.shape == x.shape and cov.shape == (6, 6, 6)
    ed = EncdecMultiheadAttn(2, 32).to(BF)
    assert sorted(ed.state_dict()) == ["in_proj_weight_kv", "in_proj_weight_q", "out_proj_weight"]
    mem = bf(torch.randn(8, 3, 32, generator=gen(10)))
    o, c = ed(x, mem, mem, attn_mask=torch.zeros(3, 8, dtype=torch.bool))
    assert o.shape == x.shape and c.shape == (6, 6, 8)
