"""CPU restatement of variable-length ("flash") attention over packed sequences. Test infrastructure only: nothing
under nmtgminor_amd/ imports this.

Reference: the reference binds the third-party module `flash_attn_cuda` (flash-attention 1.x of Dao et al.; not in the
reference tree, no version pinned there) at onmt/modules/optimized/flash_mha.py:32-75 and calls it from
FlashAttnQKVPackedFunc / FlashAttnKVPackedFunc (:104-183) and the Whisper / wav2vec encoders
(onmt/models/speech_recognizer/whisper_encoder.py:329-356). Its published algorithm (Dao et al., "FlashAttention",
NeurIPS 2022, algorithm 1 / 4) computes, per sequence b of the batch and per head h, exact attention
    S = scale * Q_b K_b^T        (causal: S[i, j] = -inf for j > i)
    P = softmax_rows(S),  L = logsumexp_rows(S)
    O = (keep * P / (1 - p)) V_b
on the tokens cu_seqlens[b] .. cu_seqlens[b+1]-1 of tensors packed as [total_tokens, heads, head_dim], and returns O in
the same packing plus L as [batch, heads, max_seqlen_q]; the backward returns dQ, dK, dV in the packing of their inputs
and D = rowsum(dO * O) as [batch, heads, max_seqlen_q]. That is restated here one sequence and one head at a time;
gradients come from autograd (fp64 in the tests). Which elements dropout keeps is the generator's business: the
restatement takes the keep-mask as an input, [batch, heads, max_seqlen_q, max_seqlen_k]."""
import math

import torch


from .attention import _r, tiled_operand


def _scores(qb, kb, scale, causal):
    s = torch.einsum("ihd,jhd->hij", qb, kb) * scale
    if causal:
        s = s.masked_fill(torch.ones(qb.shape[0], kb.shape[0], dtype=torch.bool).triu(1), -math.inf)
    return s


def flash_attn_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale=None, causal=False, p=0.0,
                   keep_mask=None, ctype=torch.float64, round_to=None):
    """q [total_q, H, D], k / v [total_k, H, D] -> (out [total_q, H, D] in ctype, lse [B, H, max_seqlen_q]).
    Differentiable in q, k, v when round_to is None. lse entries past a sequence's length are 0. round_to: the 16-bit type
    of the tensors; the result then carries the roundings of the tiled kernel (oracle/attention.py, tiled_operand: the
    unnormalised probabilities rounded as matrix-core operands against the kernel's reference point, normalisation and
    dropout scale in full precision afterwards, the output rounded once)."""
    total_q, heads, d = q.shape
    scale = d ** -0.5 if softmax_scale is None else softmax_scale
    cu_q = [int(c) for c in cu_seqlens_q]
    cu_k = [int(c) for c in cu_seqlens_k]
    batch = len(cu_q) - 1
    out = torch.zeros(total_q, heads, d, dtype=ctype)
    lse = torch.zeros(batch, heads, max_seqlen_q, dtype=ctype)
    outs = []
    for b in range(batch):
        qb, kb, vb = q[cu_q[b]:cu_q[b + 1]].to(ctype), k[cu_k[b]:cu_k[b + 1]].to(ctype), v[cu_k[b]:cu_k[b + 1]].to(ctype)
        lq, lk = qb.shape[0], kb.shape[0]
        if lk == 0:
            outs.append(torch.zeros(lq, heads, d, dtype=ctype))
            lse[b, :, :lq] = -math.inf
            continue
        s = _scores(qb, kb, scale, causal)
        l = torch.logsumexp(s, dim=-1)
        keep = keep_mask[b, :, :lq, :lk].to(ctype) if p > 0.0 else torch.ones_like(s)
        if round_to is None:
            pr = torch.exp(s - l[..., None]) * keep / (1.0 - p)
            outs.append(torch.einsum("hij,jhd->ihd", pr, vb))
        else:
            operand, rowsum = tiled_operand(s, keep, round_to)
            o = torch.einsum("hij,jhd->ihd", operand, vb) * ((1.0 / (1.0 - p)) / rowsum).permute(1, 0, 2)
            outs.append(_r(o, round_to))
        lse[b, :, :lq] = l.detach()
    out = torch.cat(outs, dim=0) if outs else out
    return out, lse


def flash_attn_bwd(dout, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale=None, causal=False, p=0.0,
                   keep_mask=None, ctype=torch.float64, round_to=None, explicit=None, out=None):
    """-> (dq, dk, dv, softmax_d [B, H, max_seqlen_q]). out: the forward's stored output, which the backward entry point
    takes as an input (explicit form only; None: the restated forward's). Two statements of the same gradient: by autograd through
    flash_attn_fwd (round_to None), and written out as the kernels compute it (explicit; the default when round_to is
    given, which puts the kernels' 16-bit roundings in):  P = exp(S - lse);  D = rowsum(dO * O) from the rounded output;
    dP = dO V^T;  dV = round(round(keep * P)^T dO / (1 - p));  dS = round(P * (keep * dP / (1 - p) - D));
    dQ = round(dS K * scale);  dK = round(dS^T Q * scale). With round_to None the two agree to rounding error of ctype
    (tests/test_oracle_pins.py)."""
    explicit = (round_to is not None) if explicit is None else explicit
    cu_q = [int(c) for c in cu_seqlens_q]
    cu_k = [int(c) for c in cu_seqlens_k]
    heads, d = q.shape[1:]
    scale = d ** -0.5 if softmax_scale is None else softmax_scale
    delta = torch.zeros(len(cu_q) - 1, heads, max_seqlen_q, dtype=ctype)
    if not explicit:
        qr, kr, vr = (t.detach().to(ctype).requires_grad_(True) for t in (q, k, v))
        out, _ = flash_attn_fwd(qr, kr, vr, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale, causal, p, keep_mask, ctype)
        out.backward(dout.to(ctype))
        rows = (dout.to(ctype) * out.detach()).sum(-1)                     # [total_q, H]
        for b in range(len(cu_q) - 1):
            delta[b, :, :cu_q[b + 1] - cu_q[b]] = rows[cu_q[b]:cu_q[b + 1]].t()
        return qr.grad, kr.grad, vr.grad, delta
    if out is None:
        out, _ = flash_attn_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale, causal, p, keep_mask, ctype, round_to)
    out = out.to(ctype)
    rp = 1.0 / (1.0 - p)
    dq, dk, dv = (torch.zeros(t.shape, dtype=ctype) for t in (q, k, v))
    for b in range(len(cu_q) - 1):
        sq, sk = slice(cu_q[b], cu_q[b + 1]), slice(cu_k[b], cu_k[b + 1])
        qb, kb, vb, gb, ob = q[sq].to(ctype), k[sk].to(ctype), v[sk].to(ctype), dout[sq].to(ctype), out[sq]
        lq, lk = qb.shape[0], kb.shape[0]
        dl = (gb * ob).sum(-1).t()                                         # [H, lq]
        delta[b, :, :lq] = dl
        if lk == 0 or lq == 0:
            continue
        s = _scores(qb, kb, scale, causal)
        pr = torch.softmax(s, dim=-1)
        keep = keep_mask[b, :, :lq, :lk].to(ctype) if p > 0.0 else torch.ones_like(s)
        dp = torch.einsum("ihd,jhd->hij", gb, vb)
        dv[sk] = _r(torch.einsum("hij,ihd->jhd", _r(pr * keep, round_to), gb) * rp, round_to)
        ds = _r(pr * (dp * keep * rp - dl[..., None]), round_to)
        dq[sq] = _r(torch.einsum("hij,jhd->ihd", ds, kb) * scale, round_to)
        dk[sk] = _r(torch.einsum("hij,ihd->jhd", ds, qb) * scale, round_to)
    return dq, dk, dv, delta


def pack(padded, lengths):
    """[B, T, ...] padded batch -> ([sum(lengths), ...], cu_seqlens int32 [B + 1])."""
    parts = [padded[b, :n] for b, n in enumerate(lengths)]
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.as_tensor(lengths), 0)
    return torch.cat(parts, dim=0), cu
