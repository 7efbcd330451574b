"""Oracle for self-attention with relative position encodings (TEST INFRASTRUCTURE ONLY, like the rest of this package).

Restates RelativeShift and the non-learnable-position branch of RelativeSelfAttnFunc of the reference
(onmt/modules/optimized/relative_self_attention_func.py:26-76 shift, :128-345 forward, :513-727 backward):

  lin = x W_in^T + b_in viewed [T, B*H, 3, D] -> q, k, v;   r_k = pos W_pos^T + b_pos viewed [R, B*H, D]
  (pos [R, 1, E] is repeated over the batch first, :146-147);
  rw_q = q + r_w_bias, rr_q = q + r_r_bias (biases [H, D], :210-214);
  AC = rw_q k^T / sqrt(D) [B*H, T, T];  BD = shift(rr_q r_k^T / sqrt(D))[:, :, :T]  (:222-251);
  scores = AC + BD; masked_fill(-inf) with a key-padding mask [B, T] or a time mask [T, T]; softmax; dropout
  (explicit keep-mask); NaN -> 0; ctx = P v -> [T, B, E]; out = ctx W_out^T + b_out.

How it is pinned (tests/test_oracle_pins.py): the shift against the closed form of its index arithmetic evaluated by
Python loops and against the Transformer-XL property it exists for (out[i][j] = x[i][R - 1 - (i - j)] for j <= i when
R = T); its backward as the adjoint (<shift(x), y> = <x, shift_bwd(y)>) and against autograd of the forward; the
attention forward against a per-element loop of the Transformer-XL definition under a causal mask; the attention
backward against autograd of the forward in fp64; the learnable-position branch (rel_learnable_attn_*) likewise against a
per-element loop of its definition and fp64 autograd.
"""
import torch

from .attention import _linear, _r
from .softmax_dropout import masked_scores, softmax_dropout_bwd, softmax_dropout_fwd


def relative_shift(x):
    """x [B, Tq, R] -> [B, Tq, R]: zero column in front, read as [B, R + 1, Tq], first row dropped, read as [B, Tq, R]
    (relative_self_attention_func.py:29-50, batch_first form)."""
    b, tq, r = x.shape
    padded = torch.cat([x.new_zeros(b, tq, 1), x], dim=2)             # [B, Tq, R + 1]
    return padded.reshape(b, r + 1, tq)[:, 1:].reshape(b, tq, r)


def relative_shift_bwd(g):
    """The adjoint of relative_shift (relative_self_attention_func.py:53-76): g [B, Tq, R] read as [B, R, Tq], a zero
    row in front, read as [B, Tq, R + 1], first column dropped."""
    b, tq, r = g.shape
    padded = torch.cat([g.new_zeros(b, 1, tq), g.reshape(b, r, tq)], dim=1)   # [B, R + 1, Tq]
    return padded.reshape(b, tq, r + 1)[:, :, 1:]


def _split(x, pos, w_in, w_pos, b_in, b_pos, heads, ctype, round_to):
    t, b, e = x.shape
    d = e // heads
    if pos.shape[1] == 1:
        pos = pos.repeat(1, b, 1)
    r = pos.shape[0]
    x, pos = x.to(ctype), pos.to(ctype)
    lin = _r(_linear(x.reshape(t * b, e), w_in.to(ctype), None if b_in is None else b_in.to(ctype)), round_to)
    pos_lin = _r(_linear(pos.reshape(r * b, e), w_pos.to(ctype), None if b_pos is None else b_pos.to(ctype)), round_to)
    return x, pos, lin.view(t, b * heads, 3, d), pos_lin.view(r, b * heads, d)


def _biased(q, bias, heads, ctype, round_to):
    t, bh, d = q.shape
    return _r(q.reshape(t, bh // heads, heads, d) + bias.to(ctype).view(heads, d), round_to).reshape(t, bh, d)


def rel_self_attn_fwd(x, pos, w_in, w_out, w_pos, b_in, b_out, b_pos, r_w_bias, r_r_bias, heads, pad_mask=None,
                      time_mask=None, p=0.0, dropout_mask=None, ctype=torch.float32, round_to=None):
    """x [T, B, E], pos [R, 1 or B, E] (R >= T). -> dict(input_lin_results [T,B,3E], pos_lin_results [R,B,E], rw_head_q,
    rr_head_q [T,B*H,D], attn_scores, softmax_results, dropout_results [B*H,T,T], matmul2_results, outputs [T,B,E])."""
    t, b, e = x.shape
    d = e // heads
    scale = d ** -0.5
    x, pos, lin, r_k = _split(x, pos, w_in, w_pos, b_in, b_pos, heads, ctype, round_to)
    q, k, v = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    rw_q = _biased(q, r_w_bias, heads, ctype, round_to)
    rr_q = _biased(q, r_r_bias, heads, ctype, round_to)
    ac = _r(torch.matmul(rw_q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) * scale, round_to)
    bd = _r(torch.matmul(rr_q.transpose(0, 1), r_k.transpose(0, 1).transpose(1, 2)) * scale, round_to)
    scores = _r(ac + relative_shift(bd)[:, :, :t], round_to)
    scores = masked_scores(scores, pad_mask, time_mask, heads)
    sm, dr = softmax_dropout_fwd(scores, dropout_mask, p, ctype)
    dr = _r(dr, round_to)
    ctx = _r(torch.matmul(dr, v.transpose(0, 1)).transpose(0, 1), round_to).reshape(t, b, e)
    out = _linear(ctx.reshape(t * b, e), w_out.to(ctype), None if b_out is None else b_out.to(ctype)).view(t, b, e)
    return dict(input_lin_results=lin.reshape(t, b, 3 * e), pos_lin_results=r_k.reshape(-1, b, e), rw_head_q=rw_q,
                rr_head_q=rr_q, attn_scores=scores, softmax_results=sm, dropout_results=dr, matmul2_results=ctx,
                outputs=out)


def rel_self_attn_bwd(dout, x, pos, w_in, w_out, w_pos, heads, fwd, p=0.0, dropout_mask=None, ctype=torch.float32,
                      round_to=None):
    """fwd = dict returned by rel_self_attn_fwd. -> dict(dx, dw_in, dw_out, dw_pos, db_in, db_out, db_pos, dr_w_bias,
    dr_r_bias)."""
    t, b, e = x.shape
    d = e // heads
    scale = d ** -0.5
    if pos.shape[1] == 1:
        pos = pos.repeat(1, b, 1)
    r = pos.shape[0]
    x2, pos2 = x.to(ctype).reshape(t * b, e), pos.to(ctype).reshape(r * b, e)
    w_in, w_out = w_in.to(ctype), w_out.to(ctype)
    g = dout.to(ctype).reshape(t * b, e)
    ctx = fwd["matmul2_results"].to(ctype).reshape(t * b, e)
    dw_out, db_out = g.t() @ ctx, g.sum(0)
    dctx = _r(g @ w_out, round_to).view(t, b * heads, d).transpose(0, 1)                    # [BH, T, D]
    lin = fwd["input_lin_results"].to(ctype).view(t, b * heads, 3, d)
    k, v = lin[:, :, 1, :], lin[:, :, 2, :]
    r_k = fwd["pos_lin_results"].to(ctype).view(r, b * heads, d)
    rw_q, rr_q = fwd["rw_head_q"].to(ctype), fwd["rr_head_q"].to(ctype)
    sm, dr = fwd["softmax_results"].to(ctype), fwd["dropout_results"].to(ctype)
    d_dr = _r(torch.matmul(dctx, v.transpose(0, 1).transpose(1, 2)), round_to)
    dv = _r(torch.matmul(dr.transpose(1, 2), dctx).transpose(0, 1), round_to)
    ds = _r(softmax_dropout_bwd(d_dr, sm, dropout_mask, p, ctype), round_to)                # [BH, T, T], both terms
    dq_ac = _r((torch.matmul(ds, k.transpose(0, 1)) * scale).transpose(0, 1), round_to)     # [T, BH, D]
    dk = _r((torch.matmul(ds.transpose(1, 2), rw_q.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    ds_full = torch.cat([ds, ds.new_zeros(ds.shape[0], t, r - t)], dim=-1) if r > t else ds
    dbd = relative_shift_bwd(ds_full)                                                        # [BH, T, R]
    dq_bd = _r((torch.matmul(dbd, r_k.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    dr_k = _r((torch.matmul(dbd.transpose(1, 2), rr_q.transpose(0, 1)) * scale).transpose(0, 1), round_to)   # [R, BH, D]
    dr_w_bias = dq_ac.reshape(t * b, heads, d).sum(0)
    dr_r_bias = dq_bd.reshape(t * b, heads, d).sum(0)
    dq = _r(dq_ac + dq_bd, round_to)
    dlin = torch.stack([dq, dk, dv], dim=2).reshape(t * b, 3 * e)
    dpos_lin = dr_k.reshape(r * b, e)
    return dict(dx=(dlin @ w_in).view(t, b, e), dw_in=dlin.t() @ x2, db_in=dlin.sum(0), dw_out=dw_out, db_out=db_out,
                dw_pos=dpos_lin.t() @ pos2, db_pos=dpos_lin.sum(0), dr_w_bias=dr_w_bias, dr_r_bias=dr_r_bias)


def rel_learnable_attn_fwd(x, pos, w_in, w_out, b_in, b_out, heads, pad_mask=None, time_mask=None, p=0.0,
                           dropout_mask=None, ctype=torch.float32, round_to=None, round_bd=False):
    """The learnable-position branch (relative_self_attention_func.py:215-217, :254-263): pos [T, T, D] is an embedding of
    the relative distance of every (query, key) pair, shared by heads and batch;
    scores[bh][i][j] = (q[i][bh] . k[j][bh] + q[i][bh] . pos[i][j]) / sqrt(D); no shift, no r_w_bias / r_r_bias. The
    reference accumulates the second product into the stored (rounded) first one and rounds the sum once; round_bd=True
    models an implementation that stores the second product in `round_to` before the sum (one more rounding of one term)."""
    t, b, e = x.shape
    d = e // heads
    scale = d ** -0.5
    x, pos = x.to(ctype), pos.to(ctype)
    lin = _r(_linear(x.reshape(t * b, e), w_in.to(ctype), None if b_in is None else b_in.to(ctype)), round_to)
    lin = lin.view(t, b * heads, 3, d)
    q, k, v = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    ac = _r(torch.matmul(q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) * scale, round_to)          # [BH, T, T]
    bd = (torch.matmul(q, pos.transpose(1, 2)) * scale).transpose(0, 1)                                     # [T, BH, T] -> [BH, T, T]
    if round_bd:
        bd = _r(bd, round_to)
    scores = masked_scores(_r(ac + bd, round_to), pad_mask, time_mask, heads)
    sm, dr = softmax_dropout_fwd(scores, dropout_mask, p, ctype)
    dr = _r(dr, round_to)
    ctx = _r(torch.matmul(dr, v.transpose(0, 1)).transpose(0, 1), round_to).reshape(t, b, e)
    out = _linear(ctx.reshape(t * b, e), w_out.to(ctype), None if b_out is None else b_out.to(ctype)).view(t, b, e)
    return dict(input_lin_results=lin.reshape(t, b, 3 * e), attn_scores=scores, softmax_results=sm, dropout_results=dr,
                matmul2_results=ctx, outputs=out)


def rel_learnable_attn_bwd(dout, x, pos, w_in, w_out, heads, fwd, p=0.0, dropout_mask=None, ctype=torch.float32,
                           round_to=None):
    """Backward of the learnable-position branch (relative_self_attention_func.py:584-706). -> dict(dx, dpos [T, T, D],
    dw_in, dw_out, db_in, db_out)."""
    t, b, e = x.shape
    d = e // heads
    scale = d ** -0.5
    x2, pos = x.to(ctype).reshape(t * b, e), pos.to(ctype)
    w_in, w_out = w_in.to(ctype), w_out.to(ctype)
    g = dout.to(ctype).reshape(t * b, e)
    ctx = fwd["matmul2_results"].to(ctype).reshape(t * b, e)
    dw_out, db_out = g.t() @ ctx, g.sum(0)
    dctx = _r(g @ w_out, round_to).view(t, b * heads, d).transpose(0, 1)
    lin = fwd["input_lin_results"].to(ctype).view(t, b * heads, 3, d)
    q, k, v = lin[:, :, 0, :], lin[:, :, 1, :], lin[:, :, 2, :]
    sm, dr = fwd["softmax_results"].to(ctype), fwd["dropout_results"].to(ctype)
    d_dr = _r(torch.matmul(dctx, v.transpose(0, 1).transpose(1, 2)), round_to)
    dv = _r(torch.matmul(dr.transpose(1, 2), dctx).transpose(0, 1), round_to)
    ds = _r(softmax_dropout_bwd(d_dr, sm, dropout_mask, p, ctype), round_to)                               # [BH, T, T]
    dq_ac = _r((torch.matmul(ds, k.transpose(0, 1)) * scale).transpose(0, 1), round_to)                    # [T, BH, D]
    dk = _r((torch.matmul(ds.transpose(1, 2), q.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    by_query = ds.transpose(0, 1)                                                                           # [T, BH, T]
    dq_bd = _r(torch.matmul(by_query, pos) * scale, round_to)                                               # [T, BH, D]
    dpos = torch.matmul(by_query.transpose(1, 2), q) * scale                                                # [T, T, D]
    dq = _r(dq_ac + dq_bd, round_to)
    dlin = torch.stack([dq, dk, dv], dim=2).reshape(t * b, 3 * e)
    return dict(dx=(dlin @ w_in).view(t, b, e), dpos=dpos, dw_in=dlin.t() @ x2, db_in=dlin.sum(0), dw_out=dw_out,
                db_out=db_out)
