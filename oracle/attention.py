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


# core="tiled": the rounding points of the tiled attention core (nmtgminor_amd/csrc/flash_attn.hip), which replaces the
# reference's bmm / softmax / dropout / bmm chain when no caller reads the coverage. The mathematics is the same
# (self_attention_func.py:141-287); what differs from the stored-tensor chain is where a 16-bit rounding happens:
#   forward   scores and softmax statistics stay in fp32; the operand of the second product is round(keep * exp(s - m)),
#             not yet normalised and not yet scaled by 1 / (1 - p) (a relative rounding, so the reference point m does not
#             matter); the context is (sum of products) * (1 / (1 - p)) / l with l = sum(exp(s - m)) unrounded, rounded once
#   backward  P = exp(s - lse) in fp32;  D = rowsum(dctx * ctx) from the stored (rounded) context;  dP unrounded;
#             dV = round((round(keep * P)^T dctx) / (1 - p));  dS = round(P * (keep * dP / (1 - p) - D));
#             dQ = round((dS K) * scale),  dK = round((dS^T Q) * scale)
TILED_KEYS = 64        # keys per tile of the forward kernel (FA_TILE in flash_attn.hip)
TILED_LAZY = 8.0       # the kernel moves a row's reference point when the row maximum has grown by more than 2^8


def tiled_operand(scores, keep, round_to):
    """The second product's left operand as the tiled forward forms it, and the row sums. scores [..., Tq, Tk] already
    scaled, -inf on masked keys. The kernel walks the keys in tiles of 64 and writes each probability relative to a
    reference point m (in log2 units) that starts at the first tile's row maximum and moves to a later tile's maximum only
    when that exceeds m + 8; exp2(s2 - m) is rounded to the 16-bit type as the matrix cores' operand, and sums formed
    before m moved are rescaled in fp32. Rounding is not invariant under a scale that is not a power of two, so the
    reference point is part of the rounding model.
    -> (operand [..., Tq, Tk] = round(keep * exp2(s2 - m_tile)) * 2^(m_tile - m_last), l = sum exp2(s2 - m_last)
    [..., Tq, 1]); the context is (operand @ V) / (1 - p) / l."""
    log2e = 1.4426950408889634
    s2 = scores * log2e
    tk = s2.shape[-1]
    neg = -1e30
    m = torch.full_like(s2[..., :1], neg)
    refs = []
    for t0 in range(0, tk, TILED_KEYS):
        mx = s2[..., t0:t0 + TILED_KEYS].max(dim=-1, keepdim=True).values.clamp_min(neg)
        m = torch.where(mx > m + TILED_LAZY, mx, m)
        refs.append(m.expand(*s2.shape[:-1], min(TILED_KEYS, tk - t0)))
    m_tile = torch.cat(refs, dim=-1)                                   # the reference point each key was written against
    live = torch.isfinite(s2)
    e = torch.where(live, torch.exp2(torch.where(live, s2, torch.zeros_like(s2)) - m_tile), torch.zeros_like(s2))
    e = _r(e * keep, round_to)
    # Keys of a tile that came before the row's first live key were written against the initial reference point; the
    # kernel zeroes those by hand, and live is false for them here.
    operand = e * torch.exp2(m_tile - m)
    l = torch.where(live, torch.exp2(torch.where(live, s2, torch.zeros_like(s2)) - m), torch.zeros_like(s2)).sum(-1, keepdim=True)
    return operand, l


def _core_fwd_tiled(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to):
    """-> scores (masked, unrounded), P (normalised, unrounded), keep [BH, Tq, Tk], ctx [Tq, BH, D] (rounded)."""
    d = q.shape[-1]
    scale = d ** -0.5
    scores = torch.matmul(q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)) * scale
    scores = masked_scores(scores, pad_mask, time_mask, heads)
    keep = dropout_mask.to(ctype) if p > 0.0 else torch.ones_like(scores)
    operand, l = tiled_operand(scores, keep, round_to)
    inv = torch.where(l > 0, (1.0 / (1.0 - p)) / l, torch.zeros_like(l))
    ctx = _r((torch.matmul(operand, v.transpose(0, 1)) * inv).transpose(0, 1), round_to)
    sm, _ = softmax_dropout_fwd(scores, None, 0.0, ctype)
    return scores, sm, keep, ctx


def _core_bwd_tiled(dctx, ctx, q, k, v, prob, keep, p, ctype, round_to):
    d = q.shape[-1]
    scale = d ** -0.5
    rp = 1.0 / (1.0 - p)
    dctx_b = dctx.transpose(0, 1)                                          # [BH, Tq, D]
    delta = (dctx_b * ctx.transpose(0, 1)).sum(-1, keepdim=True)           # from the rounded context
    dp = torch.matmul(dctx_b, v.transpose(0, 1).transpose(1, 2))
    dv = _r((torch.matmul(_r(prob * keep, round_to).transpose(1, 2), dctx_b) * rp).transpose(0, 1), round_to)
    ds = _r(prob * (dp * keep * rp - delta), round_to)
    dq = _r((torch.matmul(ds, k.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    dk = _r((torch.matmul(ds.transpose(1, 2), q.transpose(0, 1)) * scale).transpose(0, 1), round_to)
    return dq, dk, dv


class _TiledCore(torch.autograd.Function):
    """The tiled core for callers that differentiate through the oracle (oracle/transformer_layers.py): its backward is
    the written-out one with the kernels' rounding points, not autograd's of the forward."""

    @staticmethod
    def forward(ctx, q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to):
        scores, sm, keep, out = _core_fwd_tiled(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to)
        ctx.save_for_backward(q, k, v, sm, keep, out)
        ctx.args = (p, ctype, round_to)
        ctx.mark_non_differentiable(scores, sm, keep)
        return scores, sm, keep, out

    @staticmethod
    def backward(ctx, _ds, _dsm, _dkeep, dout):
        q, k, v, sm, keep, out = ctx.saved_tensors
        dq, dk, dv = _core_bwd_tiled(dout, out, q, k, v, sm, keep, *ctx.args)
        return dq, dk, dv, None, None, None, None, None, None, None


def self_attn_fwd(x, w_in, w_out, b_in, b_out, heads, pad_mask=None, time_mask=None, p=0.0,
                  dropout_mask=None, ctype=torch.float32, round_to=None, core="stored"):
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
    if core == "tiled":
        scores, sm, dr, ctx = _TiledCore.apply(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to)
    else:
        scores, sm, dr, ctx = _core_fwd(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to)
    ctx = ctx.reshape(t, b, e)
    out = _linear(ctx.reshape(t * b, e), w_out, b_out).view(t, b, e)
    return dict(input_lin_results=lin.reshape(t, b, 3 * e), attn_scores=scores, softmax_results=sm,
                dropout_results=dr, matmul2_results=ctx, outputs=out)


def self_attn_bwd(dout, x, w_in, w_out, heads, fwd, p=0.0, dropout_mask=None, ctype=torch.float32, round_to=None,
                  core="stored"):
    """fwd = dict returned by self_attn_fwd (with the same `core`; for "tiled" its dropout_results entry holds the
    keep mask). -> dict(dx, dw_in, dw_out, db_in, db_out)."""
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
    if core == "tiled":
        dq, dk, dv = _core_bwd_tiled(dctx, ctx.view(t, b * heads, d), q, k, v, fwd["softmax_results"].to(ctype),
                                     fwd["dropout_results"].to(ctype), p, ctype, round_to)
    else:
        dq, dk, dv = _core_bwd(dctx, q, k, v, fwd["softmax_results"].to(ctype), fwd["dropout_results"].to(ctype),
                               p, dropout_mask, ctype, round_to)
    dlin = torch.stack([dq, dk, dv], dim=2).reshape(t * b, 3 * e)
    dx = (dlin @ w_in).view(t, b, e)
    dw_in = dlin.t() @ x2
    db_in = dlin.sum(0)
    return dict(dx=dx, dw_in=dw_in, dw_out=dw_out, db_in=db_in, db_out=db_out, dlin=dlin.view(t, b, 3 * e))


def encdec_attn_fwd(x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, heads, pad_mask=None, p=0.0,
                    dropout_mask=None, ctype=torch.float32, round_to=None, core="stored"):
    """x_q [Tq,B,E], x_kv [Tk,B,E]; w_kv [2E,E] rows ordered (head, {k,v}, head_dim)."""
    tq, b, e = x_q.shape
    tk = x_kv.shape[0]
    d = e // heads
    cv = lambda z: z.to(ctype) if z is not None else None
    x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out = map(cv, (x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out))
    q_lin = _r(_linear(x_q.reshape(tq * b, e), w_q, b_q), round_to).view(tq, b * heads, d)
    kv_lin = _r(_linear(x_kv.reshape(tk * b, e), w_kv, b_kv), round_to).view(tk, b * heads, 2, d)
    k, v = kv_lin[:, :, 0, :], kv_lin[:, :, 1, :]
    core_fwd = _TiledCore.apply if core == "tiled" else _core_fwd
    scores, sm, dr, ctx = core_fwd(q_lin, k, v, heads, pad_mask, None, p, dropout_mask, ctype, round_to)
    ctx = ctx.reshape(tq, b, e)
    out = _linear(ctx.reshape(tq * b, e), w_out, b_out).view(tq, b, e)
    return dict(input_lin_q_results=q_lin.reshape(tq, b, e), input_lin_kv_results=kv_lin.reshape(tk, b, 2 * e),
                attn_scores=scores, softmax_results=sm, dropout_results=dr, matmul2_results=ctx, outputs=out)


def encdec_attn_bwd(dout, x_q, x_kv, w_q, w_kv, w_out, heads, fwd, p=0.0, dropout_mask=None,
                    ctype=torch.float32, round_to=None, core="stored"):
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
    if core == "tiled":
        dq, dk, dv = _core_bwd_tiled(dctx, ctx.view(tq, b * heads, d), q, k, v, cv(fwd["softmax_results"]),
                                     cv(fwd["dropout_results"]), p, ctype, round_to)
    else:
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
