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


def _r(t, round_to):
    if round_to is None:
        return t
    return t + (t.detach().to(round_to).to(t.dtype) - t.detach())     # value rounded, gradient passed through


def flash_attn_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale=None, causal=False, p=0.0,
                   keep_mask=None, ctype=torch.float64, round_to=None):
    """q [total_q, H, D], k / v [total_k, H, D] -> (out [total_q, H, D] in ctype, lse [B, H, max_seqlen_q]).
    Differentiable in q, k, v. lse entries past a sequence's length are 0. round_to: the 16-bit type the probabilities
    are rounded to before they multiply V (the kernel feeds them to the matrix cores in that type)."""
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
        s = torch.einsum("ihd,jhd->hij", qb, kb) * scale
        if causal:
            s = s.masked_fill(torch.ones(lq, lk, dtype=torch.bool).triu(1), -math.inf)
        if lk == 0:
            outs.append(torch.zeros(lq, heads, d, dtype=ctype))
            lse[b, :, :lq] = -math.inf
            continue
        l = torch.logsumexp(s, dim=-1)
        pr = torch.exp(s - l[..., None])
        if p > 0.0:
            keep = keep_mask[b, :, :lq, :lk].to(ctype)
            pr = pr * keep / (1.0 - p)
        outs.append(torch.einsum("hij,jhd->ihd", _r(pr, round_to), vb))
        lse[b, :, :lq] = l.detach()
    out = torch.cat(outs, dim=0) if outs else out
    return out, lse


def flash_attn_bwd(dout, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale=None, causal=False, p=0.0,
                   keep_mask=None, ctype=torch.float64, round_to=None):
    """-> (dq, dk, dv, softmax_d [B, H, max_seqlen_q]) by autograd through flash_attn_fwd."""
    qr, kr, vr = (t.detach().to(ctype).requires_grad_(True) for t in (q, k, v))
    out, _ = flash_attn_fwd(qr, kr, vr, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, softmax_scale, causal, p, keep_mask,
                            ctype, round_to)
    out.backward(dout.to(ctype))
    cu_q = [int(c) for c in cu_seqlens_q]
    delta = torch.zeros(len(cu_q) - 1, q.shape[1], max_seqlen_q, dtype=ctype)
    rows = (dout.to(ctype) * _r(out.detach(), round_to)).sum(-1)       # [total_q, H], from the stored (rounded) output
    for b in range(len(cu_q) - 1):
        delta[b, :, :cu_q[b + 1] - cu_q[b]] = rows[cu_q[b]:cu_q[b + 1]].t()
    return qr.grad, kr.grad, vr.grad, delta


def pack(padded, lengths):
    """[B, T, ...] padded batch -> ([sum(lengths), ...], cu_seqlens int32 [B + 1])."""
    parts = [padded[b, :n] for b, n in enumerate(lengths)]
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.as_tensor(lengths), 0)
    return torch.cat(parts, dim=0), cu
