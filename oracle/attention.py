"""Multi-head attention oracle in the reference's time-first, head-interleaved layouts.

Self-attention — reference fallback branch of SelfAttnFunc
(onmt/modules/optimized/self_attention_func.py:141-287 forward, :361-504 backward):
  x [T, B, E];  W_in [3E, E] whose rows are ordered (head, {q,k,v}, head_dim), so that
  lin = x W_in^T + b_in viewed [T, B*H, 3, D] yields q, k, v;  scores = (q k^T) / sqrt(D) as
  [B*H, Tq, Tk];  masked_fill(-inf) with a key-padding mask [B, Tk] or a time mask [Tq, Tk];
  softmax;  dropout (explicit mask);  NaN -> 0;  ctx = P v -> [T, B, E];  out = ctx W_out^T + b_out.

Encoder-decoder attention — EncdecAttnBiasFunc
(onmt/modules/optimized/encdec_attention_func_bias.py:141-351 forward, :455-668 backward):
  q = x_q W_q^T + b_q viewed [Tq, B*H, D];  kv = x_kv W_kv^T + b_kv viewed [Tk, B*H, 2, D];
  key-padding mask only; otherwise the same pipeline.

Biases may be None (Whisper passes None for the k bias, whisper_decoder.py:118-125).
"""
import torch

from .softmax_dropout import masked_scores, softmax_dropout_bwd, softmax_dropout_fwd

# round_to (all functions): the dtype in which the fallback stores its intermediate tensors
# (projections, scores, dropped probabilities, context, and their gradients). The arithmetic in
# between stays in ctype. The probabilities used by the backward are the ones recomputed from
# the stored (rounded) scores, which is what the reference's fused backward does
# (softmax_apex.h:4039-4075), so `softmax_results` is returned unrounded.


def _r(t, round_to):
    return t if round_to is None else t.to(round_to).to(t.dtype)


def _linear(x2d, w, b):
    y = x2d @ w.t()
    return y + b if b is not None else y


def _core_fwd(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to=None):
    """q [Tq, BH, D], k/v [Tk, BH, D] (views allowed). -> scores(masked), softmax, dropped, ctx [Tq, BH, D]."""
    d = q.shape[-1]
    scale = d ** -0.5
    scores = _r(torch.matmul(q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) * scale, round_to)
    scores = masked_scores(scores, pad_mask, time_mask, heads)
    sm, dr = softmax_dropout_fwd(scores, dropout_mask, p, ctype)
    dr = _r(dr, round_to)
    ctx = _r(torch.matmul(dr, v.transpose(0, 1)).transpose(0, 1), round_to)  # [Tq, BH, D]
    return scores, sm, dr, ctx


def _core_bwd(dctx, q, k, v, sm, dr, p, dropout_mask, ctype, round_to=None):
    """dctx [Tq, BH, D] -> dq, dk, dv (each [T*, BH, D])."""
    d = q.shape[-1]
    scale = d ** -0.5
    dctx_b = dctx.transpose(0, 1)                                  # [BH, Tq, D]
    d_dr = _r(torch.matmul(dctx_b, v.transpose(0, 1).transpose(1, 2)), round_to)  # [BH, Tq, Tk]
    dv = _r(torch.matmul(dr.transpose(1, 2), dctx_b).transpose(0, 1), round_to)   # [Tk, BH, D]
    ds = _r(softmax_dropout_bwd(d_dr, sm, dropout_mask, p, ctype), round_to)
    dq = _r((torch.matmul(ds, k.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    dk = _r((torch.matmul(ds.transpose(1, 2), q.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    return dq, dk, dv


def self_attn_fwd(x, w_in, w_out, b_in, b_out, heads, pad_mask=None, time_mask=None, p=0.0,
                  dropout_mask=None, ctype=torch.float32, round_to=None):
    """-> dict(input_lin_results [T,B,3E], attn_scores, softmax_results, dropout_results
    [B*H,T,T], matmul2_results [T,B,E], outputs [T,B,E])."""
    t, b, e = x.shape
    d = e // heads
    x = x.to(ctype)
    w_in, w_out = w_in.to(ctype), w_out.to(ctype)
    b_in = b_in.to(ctype) if b_in is not None else None
    b_out = b_out.to(ctype) if b_out is not None else None
    lin = _r(_linear(x.reshape(t * b, e), w_in, b_in), round_to).view(t, b * heads, 3, d)
    q, k, v = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    scores, sm, dr, ctx = _core_fwd(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to)
    ctx = ctx.reshape(t, b, e)
    out = _linear(ctx.reshape(t * b, e), w_out, b_out).view(t, b, e)
    return dict(input_lin_results=lin.reshape(t, b, 3 * e), attn_scores=scores, softmax_results=sm,
                dropout_results=dr, matmul2_results=ctx, outputs=out)


def self_attn_bwd(dout, x, w_in, w_out, heads, fwd, p=0.0, dropout_mask=None, ctype=torch.float32, round_to=None):
    """fwd = dict returned by self_attn_fwd. -> dict(dx, dw_in, dw_out, db_in, db_out)."""
    t, b, e = x.shape
    d = e // heads
    x2 = x.to(ctype).reshape(t * b, e)
    w_in, w_out = w_in.to(ctype), w_out.to(ctype)
    g = dout.to(ctype).reshape(t * b, e)
    ctx = fwd["matmul2_results"].to(ctype).reshape(t * b, e)
    dw_out = g.t() @ ctx
    db_out = g.sum(0)
    dctx = _r(g @ w_out, round_to).view(t, b * heads, d)
    lin = fwd["input_lin_results"].to(ctype).view(t, b * heads, 3, d)
    q, k, v = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    dq, dk, dv = _core_bwd(dctx, q, k, v, fwd["softmax_results"].to(ctype), fwd["dropout_results"].to(ctype),
                           p, dropout_mask, ctype, round_to)
    dlin = torch.stack([dq, dk, dv], dim=2).reshape(t * b, 3 * e)
    dx = (dlin @ w_in).view(t, b, e)
    dw_in = dlin.t() @ x2
    db_in = dlin.sum(0)
    return dict(dx=dx, dw_in=dw_in, dw_out=dw_out, db_in=db_in, db_out=db_out, dlin=dlin.view(t, b, 3 * e))


def encdec_attn_fwd(x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, heads, pad_mask=None, p=0.0,
                    dropout_mask=None, ctype=torch.float32, round_to=None):
    """x_q [Tq,B,E], x_kv [Tk,B,E]; w_kv [2E,E] rows ordered (head, {k,v}, head_dim)."""
    tq, b, e = x_q.shape
    tk = x_kv.shape[0]
    d = e // heads
    cv = lambda z: z.to(ctype) if z is not None else None
    x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out = map(cv, (x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out))
    q_lin = _r(_linear(x_q.reshape(tq * b, e), w_q, b_q), round_to).view(tq, b * heads, d)
    kv_lin = _r(_linear(x_kv.reshape(tk * b, e), w_kv, b_kv), round_to).view(tk, b * heads, 2, d)
    k, v = kv_lin[:, :, 0, :], kv_lin[:, :, 1, :]
    scores, sm, dr, ctx = _core_fwd(q_lin, k, v, heads, pad_mask, None, p, dropout_mask, ctype, round_to)
    ctx = ctx.reshape(tq, b, e)
    out = _linear(ctx.reshape(tq * b, e), w_out, b_out).view(tq, b, e)
    return dict(input_lin_q_results=q_lin.reshape(tq, b, e), input_lin_kv_results=kv_lin.reshape(tk, b, 2 * e),
                attn_scores=scores, softmax_results=sm, dropout_results=dr, matmul2_results=ctx, outputs=out)


def encdec_attn_bwd(dout, x_q, x_kv, w_q, w_kv, w_out, heads, fwd, p=0.0, dropout_mask=None,
                    ctype=torch.float32, round_to=None):
    tq, b, e = x_q.shape
    tk = x_kv.shape[0]
    d = e // heads
    cv = lambda z: z.to(ctype)
    x_q2, x_kv2 = cv(x_q).reshape(tq * b, e), cv(x_kv).reshape(tk * b, e)
    w_q, w_kv, w_out = cv(w_q), cv(w_kv), cv(w_out)
    g = cv(dout).reshape(tq * b, e)
    ctx = cv(fwd["matmul2_results"]).reshape(tq * b, e)
    dw_out = g.t() @ ctx
    db_out = g.sum(0)
    dctx = _r(g @ w_out, round_to).view(tq, b * heads, d)
    q = cv(fwd["input_lin_q_results"]).view(tq, b * heads, d)
    kv = cv(fwd["input_lin_kv_results"]).view(tk, b * heads, 2, d)
    k, v = kv[:, :, 0, :], kv[:, :, 1, :]
    dq, dk, dv = _core_bwd(dctx, q, k, v, cv(fwd["softmax_results"]), cv(fwd["dropout_results"]), p,
                           dropout_mask, ctype, round_to)
    dq2 = dq.reshape(tq * b, e)
    dkv2 = torch.stack([dk, dv], dim=2).reshape(tk * b, 2 * e)
    return dict(dx_q=(dq2 @ w_q).view(tq, b, e), dx_kv=(dkv2 @ w_kv).view(tk, b, e), dw_q=dq2.t() @ x_q2,
                dw_kv=dkv2.t() @ x_kv2, dw_out=dw_out, db_q=dq2.sum(0), db_kv=dkv2.sum(0), db_out=db_out)


def interleave_qkv(wq, wk, wv, heads):
    """Separate q/k/v projection weights [E, E] (or biases [E]) -> the head-interleaved
    in_proj layout [3E, E] ([3E]) (onmt/models/whisper/whisper_encoder.py:246-274)."""
    e = wq.shape[0]
    d = e // heads
    rest = wq.shape[1:]
    st = torch.stack([wq.reshape(heads, d, *rest), wk.reshape(heads, d, *rest), wv.reshape(heads, d, *rest)], dim=1)
    return st.reshape(3 * e, *rest)


def interleave_kv(wk, wv, heads):
    e = wk.shape[0]
    d = e // heads
    rest = wk.shape[1:]
    st = torch.stack([wk.reshape(heads, d, *rest), wv.reshape(heads, d, *rest)], dim=1)
    return st.reshape(2 * e, *rest)
