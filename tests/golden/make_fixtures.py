#!/usr/bin/env python3
"""Writes the golden fixtures tests/golden/*.npz.

    python tests/golden/make_fixtures.py

The expected values come from PyTorch's own CPU library routines and autograd in fp64
(F.layer_norm, F.softmax, F.cross_entropy(label_smoothing, ignore_index), F.linear, F.gelu, F.relu,
F.silu, F.gelu(approximate="tanh"), torch.optim.Adam / AdamW, clip_grad_norm_) on small seeded inputs — the routines the reference's
PyTorch fallback itself calls (onmt/modules/layer_norm.py:29-33, onmt/modules/mlp/mlp.py:14-42,
onmt/modules/optimized/self_attention_func.py:141-287, encdec_attention_func_bias.py:141-351,
relative_self_attention_func.py:128-345 with the relative shift written as an explicit gather,
onmt/modules/optimized/softmax_xentropy.py). Neither oracle/ nor the HIP library is imported here,
so the fixtures are independent of both; tests/test_golden_cpu.py checks the oracle against them
and tests/test_zz_golden_gpu.py the HIP path.

The 16-bit cases (MLP, attention) store inputs that are exactly representable in bf16 AND fp16
and apply the fallback's rounding points (every tensor the fallback materialises is rounded to
bf16; autograd through the casts rounds the matching gradients) so that a bf16 run can be
compared at the 16-bit tolerance without slack for intermediate rounding.
"""
import math
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
D = torch.float64
BF = torch.bfloat16


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rnd16(t):
    """Values representable in both bf16 and fp16 (bf16 mantissa, magnitudes kept in fp16's normal range)."""
    t = t.to(BF).to(D)
    t = torch.where(t.abs() < 2.0 ** -10, torch.zeros_like(t), t)
    assert torch.equal(t.to(torch.float16).to(D), t) and torch.equal(t.to(BF).to(D), t)
    return t


def rb(t):
    """The fallback stores this tensor in the working dtype (bf16 here); differentiable."""
    return t.to(BF).to(D)


def save(name, f32=False, **arrays):
    """f32: store floating-point arrays as float32 (the 16-bit cases: inputs are exact in float32 and the
    expected values are compared at 16-bit tolerance)."""
    out = {}
    for k, v in arrays.items():
        if isinstance(v, torch.Tensor):
            v = v.detach().cpu().numpy()
        v = np.asarray(v)
        if f32 and v.dtype == np.float64 and v.ndim > 0:
            v = v.astype(np.float32)
        out[k] = v
    np.savez(os.path.join(HERE, name + ".npz"), **out)
    print(f"wrote {name}.npz: " + ", ".join(f"{k}{list(np.shape(v))}" for k, v in out.items()))


def layer_norm():
    g = gen(101)
    rows, hidden, eps = 6, 40, 1e-5
    x = torch.randn(rows, hidden, generator=g, dtype=D).requires_grad_()
    gamma = (1 + 0.1 * torch.randn(hidden, generator=g, dtype=D)).requires_grad_()
    beta = (0.1 * torch.randn(hidden, generator=g, dtype=D)).requires_grad_()
    dy = torch.randn(rows, hidden, generator=g, dtype=D)
    y = F.layer_norm(x, (hidden,), gamma, beta, eps)
    y.backward(dy)
    mu = x.detach().mean(1)
    rsigma = (x.detach().var(1, unbiased=False) + eps).rsqrt()
    save("layer_norm", x=x, gamma=gamma, beta=beta, dy=dy, eps=eps, y=y, mu=mu, rsigma=rsigma, dx=x.grad,
         dgamma=gamma.grad, dbeta=beta.grad)


def dropout_add():
    g = gen(102)
    n, p = 50, 0.2
    x = torch.randn(n, generator=g, dtype=D).requires_grad_()
    res = torch.randn(n, generator=g, dtype=D)
    mask = (torch.rand(n, generator=g) < 1 - p).to(torch.uint8)
    dout = torch.randn(n, generator=g, dtype=D)
    out = x * mask.to(D) / (1 - p) + res
    out.backward(dout)
    save("dropout_add", x=x, residual=res, mask=mask, p=p, dout=dout, out=out, dx=x.grad)


def softmax_dropout():
    g = gen(103)
    batch, heads, tq, tk, p = 2, 2, 5, 12, 0.25
    bh = batch * heads
    s = (3 * torch.randn(bh, tq, tk, generator=g, dtype=D)).requires_grad_()
    lengths = torch.tensor([7, 12])
    pad = torch.arange(tk).unsqueeze(0) >= lengths.unsqueeze(1)            # [B, Tk], True = padded key
    dm = (torch.rand(bh, tq, tk, generator=g) < 1 - p).to(torch.uint8)
    dout = torch.randn(bh, tq, tk, generator=g, dtype=D)
    masked = s.view(batch, heads, tq, tk).masked_fill(pad.view(batch, 1, 1, tk), float("-inf")).view(bh, tq, tk)
    sm = F.softmax(masked, -1)
    dropped = sm * dm.to(D) / (1 - p)
    dropped.backward(dout)
    save("softmax_dropout", scores=s, pad_mask=pad.to(torch.uint8), dropout_mask=dm, p=p, heads=heads, dout=dout,
         softmax=sm, dropped=dropped, dscores=s.grad)


def xentropy():
    g = gen(104)
    n, v, eps, pad = 9, 37, 0.1, 1
    logits = (2 * torch.randn(n, v, generator=g, dtype=D)).requires_grad_()
    labels = torch.randint(0, v, (n,), generator=g)
    labels[2] = pad
    labels[7] = pad
    gl = torch.rand(n, generator=g, dtype=D) + 0.5
    losses = F.cross_entropy(logits, labels, reduction="none", label_smoothing=eps, ignore_index=pad)
    lse = torch.logsumexp(logits.detach(), 1)
    losses.backward(gl)
    # the two closed forms of the reference's own test (extensions/xentropy/test_xentropy.py:44-62):
    # loss = lse - (1 - eps) x_label - eps mean(x)
    closed = lse - (1 - eps) * logits.detach().gather(1, labels.view(-1, 1)).squeeze(1) - eps * logits.detach().mean(1)
    closed[labels == pad] = 0
    assert torch.allclose(losses.detach(), closed, rtol=1e-12, atol=1e-12)
    save("xentropy", logits=logits, labels=labels, smoothing=eps, padding_idx=pad, grad_loss=gl, losses=losses, lse=lse,
         dlogits=logits.grad)


ACTS = {
    "gelu": lambda h: F.gelu(h),
    "relu": lambda h: F.relu(h),
    "silu": lambda h: F.silu(h),
    "agelu": lambda h: F.gelu(h, approximate="tanh"),
}


def mlp():
    g = gen(105)
    tokens, dm_, di, p = 24, 16, 32, 0.2
    x0 = rnd16(torch.randn(tokens, dm_, generator=g, dtype=D))
    w1_0 = rnd16(torch.randn(di, dm_, generator=g, dtype=D) / math.sqrt(dm_))
    w2_0 = rnd16(torch.randn(dm_, di, generator=g, dtype=D) / math.sqrt(di))
    b1_0 = rnd16(0.1 * torch.randn(di, generator=g, dtype=D))
    b2_0 = rnd16(0.1 * torch.randn(dm_, generator=g, dtype=D))
    mask = (torch.rand(tokens, di, generator=g) < 1 - p).to(torch.uint8)
    dy = rnd16(torch.randn(tokens, dm_, generator=g, dtype=D))
    out = dict(x=x0, w1=w1_0, w2=w2_0, b1=b1_0, b2=b2_0, mask=mask, p=p, dy=dy)
    for act, fn in ACTS.items():
        x, w1, w2, b1, b2 = (t.clone().requires_grad_() for t in (x0, w1_0, w2_0, b1_0, b2_0))
        pre = rb(F.linear(x, w1, b1))                       # stored pre-activation
        post = rb(fn(pre) * mask.to(D) / (1 - p))           # stored activation after dropout
        y = F.linear(post, w2, b2)
        y.backward(dy)
        out.update({f"{act}_pre": pre, f"{act}_post": post, f"{act}_y": y, f"{act}_dx": x.grad, f"{act}_dw1": w1.grad,
                    f"{act}_dw2": w2.grad, f"{act}_db1": b1.grad, f"{act}_db2": b2.grad})
    save("mlp", f32=True, **out)


def _attention_core(q, k, v, batch, heads, pad, time_mask, dm, p):
    """q [Tq, B*H, D], k / v [Tk, B*H, D] -> scores (stored, masked), softmax, dropped (stored), ctx [Tq, B*H, D] (stored)."""
    tq, bh, d = q.shape
    tk = k.shape[0]
    scores = rb(torch.matmul(q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) / math.sqrt(d))
    if pad is not None:
        scores = scores.view(batch, heads, tq, tk).masked_fill(pad.view(batch, 1, 1, tk), float("-inf")).view(bh, tq, tk)
    if time_mask is not None:
        scores = scores.masked_fill(time_mask.view(1, tq, tk), float("-inf"))
    sm = F.softmax(scores, -1)
    dropped = rb(sm * dm.to(D) / (1 - p)) if dm is not None else rb(sm)
    ctx = rb(torch.matmul(dropped, v.transpose(0, 1)).transpose(0, 1))
    return scores, sm, dropped, ctx


def self_attention():
    g = gen(106)
    t, b, e, h, p = 9, 2, 64, 2, 0.25
    d = e // h
    x0 = rnd16(torch.randn(t, b, e, generator=g, dtype=D))
    w_in0 = rnd16(torch.randn(3 * e, e, generator=g, dtype=D) / math.sqrt(e))
    w_out0 = rnd16(torch.randn(e, e, generator=g, dtype=D) / math.sqrt(e))
    b_in0 = rnd16(0.1 * torch.randn(3 * e, generator=g, dtype=D))
    b_out0 = rnd16(0.1 * torch.randn(e, generator=g, dtype=D))
    lengths = torch.tensor([5, 9])
    pad = torch.arange(t).unsqueeze(0) >= lengths.unsqueeze(1)
    dm = (torch.rand(b * h, t, t, generator=g) < 1 - p).to(torch.uint8)
    dout = rnd16(torch.randn(t, b, e, generator=g, dtype=D))
    x, w_in, w_out, b_in, b_out = (z.clone().requires_grad_() for z in (x0, w_in0, w_out0, b_in0, b_out0))
    lin = rb(F.linear(x, w_in, b_in)).view(t, b * h, 3, d)          # rows of W_in ordered (head, {q,k,v}, head_dim)
    q, k, v = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    scores, sm, dropped, ctx = _attention_core(q, k, v, b, h, pad, None, dm, p)
    out = F.linear(ctx.reshape(t, b, e), w_out, b_out)
    out.backward(dout)
    save("self_attention", f32=True, x=x0, w_in=w_in0, w_out=w_out0, b_in=b_in0, b_out=b_out0, pad_mask=pad.to(torch.uint8),
         dropout_mask=dm, p=p, heads=h, dout=dout, input_lin_results=lin.reshape(t, b, 3 * e), softmax_results=sm,
         dropout_results=dropped, matmul2_results=ctx.reshape(t, b, e), outputs=out, dx=x.grad, dw_in=w_in.grad,
         dw_out=w_out.grad, db_in=b_in.grad, db_out=b_out.grad)


def encdec_attention():
    g = gen(107)
    tq, tk, b, e, h = 5, 11, 2, 64, 2
    d = e // h
    mk = lambda *s, scale=1.0: rnd16(scale * torch.randn(*s, generator=g, dtype=D))
    x_q, x_kv = mk(tq, b, e), mk(tk, b, e)
    w_q, w_kv, w_out = mk(e, e, scale=1 / math.sqrt(e)), mk(2 * e, e, scale=1 / math.sqrt(e)), mk(e, e, scale=1 / math.sqrt(e))
    b_q, b_kv, b_out = mk(e, scale=0.1), mk(2 * e, scale=0.1), mk(e, scale=0.1)
    lengths = torch.tensor([11, 6])
    pad = torch.arange(tk).unsqueeze(0) >= lengths.unsqueeze(1)
    q = rb(F.linear(x_q, w_q, b_q)).view(tq, b * h, d)
    kv = rb(F.linear(x_kv, w_kv, b_kv)).view(tk, b * h, 2, d)       # rows of W_kv ordered (head, {k,v}, head_dim)
    scores, sm, dropped, ctx = _attention_core(q, kv[:, :, 0, :], kv[:, :, 1, :], b, h, pad, None, None, 0.0)
    out = F.linear(ctx.reshape(tq, b, e), w_out, b_out)
    save("encdec_attention", f32=True, x_q=x_q, x_kv=x_kv, w_q=w_q, w_kv=w_kv, w_out=w_out, b_q=b_q, b_kv=b_kv, b_out=b_out,
         pad_mask=pad.to(torch.uint8), heads=h, softmax_results=sm, matmul2_results=ctx.reshape(tq, b, e), outputs=out)


def relative_attention():
    """Self-attention with relative positions. The shift is a gather over an index table built element by element from
    its closed form (output (i, j) reads padded element i R + j + T of the zero-fronted [T, R + 1] matrix), not the
    reference's pad / view sequence."""
    g = gen(108)
    t, r, b, e, h, p = 9, 12, 2, 64, 2, 0.25
    d = e // h
    mk = lambda *s, scale=1.0: rnd16(scale * torch.randn(*s, generator=g, dtype=D))
    x0, pos0 = mk(t, b, e), mk(r, 1, e)
    w_in0, w_out0, w_pos0 = mk(3 * e, e, scale=1 / math.sqrt(e)), mk(e, e, scale=1 / math.sqrt(e)), mk(e, e, scale=1 / math.sqrt(e))
    b_in0, b_out0, b_pos0 = mk(3 * e, scale=0.1), mk(e, scale=0.1), mk(e, scale=0.1)
    u0, v0 = mk(h, d, scale=0.1), mk(h, d, scale=0.1)
    lengths = torch.tensor([9, 6])
    pad = torch.arange(t).unsqueeze(0) >= lengths.unsqueeze(1)
    dm = (torch.rand(b * h, t, t, generator=g) < 1 - p).to(torch.uint8)
    dout = mk(t, b, e)
    leaves = [z.clone().requires_grad_() for z in (x0, w_in0, w_out0, w_pos0, b_in0, b_out0, b_pos0, u0, v0)]
    x, w_in, w_out, w_pos, b_in, b_out, b_pos, u, v = leaves
    lin = rb(F.linear(x, w_in, b_in)).view(t, b * h, 3, d)
    q, k, val = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    r_k = rb(F.linear(pos0.expand(r, b, e), w_pos, b_pos)).view(r, b * h, d)
    rw_q = rb(q.view(t, b, h, d) + u).view(t, b * h, d)
    rr_q = rb(q.view(t, b, h, d) + v).view(t, b * h, d)
    ac = rb(torch.matmul(rw_q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) / math.sqrt(d))
    bd = rb(torch.matmul(rr_q.transpose(0, 1), r_k.transpose(0, 1).transpose(1, 2)) / math.sqrt(d))       # [B*H, T, R]
    src = torch.zeros(t, t, dtype=torch.long)            # index into the flattened zero-fronted [T, R + 1] matrix
    for i in range(t):
        for j in range(t):
            src[i, j] = i * r + j + t
    padded = torch.cat([bd.new_zeros(b * h, t, 1), bd], dim=2).reshape(b * h, t * (r + 1))
    shifted = padded.gather(1, src.view(1, t * t).expand(b * h, t * t)).view(b * h, t, t)
    scores = rb(ac + shifted)
    scores = scores.view(b, h, t, t).masked_fill(pad.view(b, 1, 1, t), float("-inf")).view(b * h, t, t)
    sm = F.softmax(scores, -1)
    dropped = rb(sm * dm.to(D) / (1 - p))
    ctx = rb(torch.matmul(dropped, val.transpose(0, 1)).transpose(0, 1))
    out = F.linear(ctx.reshape(t, b, e), w_out, b_out)
    out.backward(dout)
    save("relative_attention", f32=True, x=x0, pos=pos0, w_in=w_in0, w_out=w_out0, w_pos=w_pos0, b_in=b_in0, b_out=b_out0,
         b_pos=b_pos0, r_w_bias=u0, r_r_bias=v0, pad_mask=pad.to(torch.uint8), dropout_mask=dm, p=p, heads=h, dout=dout,
         softmax_results=sm, dropout_results=dropped, matmul2_results=ctx.reshape(t, b, e), outputs=out, dx=x.grad,
         dw_in=w_in.grad, dw_out=w_out.grad, dw_pos=w_pos.grad, db_in=b_in.grad, db_out=b_out.grad, db_pos=b_pos.grad,
         dr_w_bias=u.grad, dr_r_bias=v.grad)


def fused_optim():
    """Four AdamW steps and four Adam (L2) steps of torch.optim on three small fp32 tensors, the joint L2 norm of the last
    gradients (torch.linalg.vector_norm) and those gradients clipped by torch.nn.utils.clip_grad_norm_."""
    g = gen(109)
    shapes = [(5, 7), (33,), (2, 3, 4)]
    p0 = [torch.randn(s, generator=g, dtype=D) for s in shapes]
    grads = [[torch.randn(s, generator=g, dtype=D) for s in shapes] for _ in range(4)]
    kw = dict(lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.05)
    out = {}
    for name, cls in (("adamw", torch.optim.AdamW), ("adam", torch.optim.Adam)):
        ps = [t.clone().requires_grad_() for t in p0]
        opt = cls(ps, **kw)
        for step in grads:
            for p, gr in zip(ps, step):
                p.grad = gr.clone()
            opt.step()
        for i, p in enumerate(ps):
            out[f"{name}_p{i}"] = p.detach()
            out[f"{name}_m{i}"] = opt.state[p]["exp_avg"]
            out[f"{name}_v{i}"] = opt.state[p]["exp_avg_sq"]
    holders = [torch.zeros(s, dtype=D).requires_grad_() for s in shapes]
    for h, gr in zip(holders, grads[-1]):
        h.grad = gr.clone()
    norm = torch.nn.utils.clip_grad_norm_(holders, 1.5)
    save("fused_optim", lr=kw["lr"], beta1=kw["betas"][0], beta2=kw["betas"][1], eps=kw["eps"], weight_decay=kw["weight_decay"],
         max_norm=1.5, norm=norm, **{f"p{i}": t for i, t in enumerate(p0)},
         **{f"g{s}_{i}": t for s, step in enumerate(grads) for i, t in enumerate(step)},
         **{f"clipped{i}": h.grad for i, h in enumerate(holders)}, **out)


if __name__ == "__main__":
    torch.set_num_threads(1)
    for f in (layer_norm, dropout_add, softmax_dropout, xentropy, mlp, self_attention, encdec_attention, relative_attention, fused_optim):
        f()
