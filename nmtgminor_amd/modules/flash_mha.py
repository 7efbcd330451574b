"""Attention over packed variable-length sequences: the autograd functions and entry points of the reference's
onmt/modules/optimized/flash_mha.py on the HIP kernels.

    flash_bert_mha(qkv [total, 3, H, D], cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, return_softmax)
    flash_encdec_mha(q [total_q, H, D], kv [total_k, 2, H, D], cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                     dropout_p, softmax_scale, causal, return_softmax)

mirror FlashAttnQKVPackedFunc (flash_mha.py:104-140) and FlashAttnKVPackedFunc (:143-183): same positional arguments,
same outputs (out, or (out, softmax_lse, S_dmask) with return_softmax, where S_dmask is the dropout keep-mask here),
gradients written into the slots of one packed tensor. The backward regenerates the dropout mask from the Philox
(seed, offset) pair that the forward drew, which the context carries instead of the reference's saved generator state."""
import torch

from ..native import flash_attn_cuda
from ._autocast import cast_if_autocast_enabled, no_autocast


def _flash_attn_forward(q, k, v, out, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
                        causal, return_softmax, num_splits=0, generator=None):
    softmax_lse, *rest = flash_attn_cuda.fwd(q, k, v, out, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                             dropout_p, softmax_scale, False, causal, return_softmax, num_splits, generator)
    return out, softmax_lse, (rest[0] if return_softmax else None), flash_attn_cuda.last_rng


def _flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                         max_seqlen_k, dropout_p, softmax_scale, causal, num_splits=0, generator=None, rng=None):
    if dout.stride(-1) != 1:
        dout = dout.contiguous()
    _, _, _, softmax_d = flash_attn_cuda.bwd(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
                                             max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, False, causal,
                                             num_splits, generator, rng=rng)
    return dq, dk, dv, softmax_d


class FlashAttnQKVPackedFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, return_softmax):
        if softmax_scale is None:
            softmax_scale = qkv.shape[-1] ** (-0.5)
        out, softmax_lse, s_dmask, ctx.rng = _flash_attn_forward(
            qkv[:, 0], qkv[:, 1], qkv[:, 2], torch.empty_like(qkv[:, 0]), cu_seqlens, cu_seqlens, max_seqlen, max_seqlen,
            dropout_p, softmax_scale, causal=causal, return_softmax=return_softmax)
        ctx.save_for_backward(qkv, out, softmax_lse, cu_seqlens)
        ctx.dropout_p, ctx.max_seqlen, ctx.softmax_scale, ctx.causal = dropout_p, max_seqlen, softmax_scale, causal
        if not return_softmax:
            return out
        ctx.mark_non_differentiable(softmax_lse, s_dmask) if s_dmask is not None else ctx.mark_non_differentiable(softmax_lse)
        return out, softmax_lse, s_dmask

    @staticmethod
    def backward(ctx, dout, *args):
        qkv, out, softmax_lse, cu_seqlens = ctx.saved_tensors
        dqkv = torch.empty_like(qkv)
        _flash_attn_backward(dout, qkv[:, 0], qkv[:, 1], qkv[:, 2], out, softmax_lse, dqkv[:, 0], dqkv[:, 1], dqkv[:, 2],
                             cu_seqlens, cu_seqlens, ctx.max_seqlen, ctx.max_seqlen, ctx.dropout_p, ctx.softmax_scale,
                             ctx.causal, rng=ctx.rng)
        return dqkv, None, None, None, None, None, None


class FlashAttnKVPackedFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, kv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal,
                return_softmax):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        out, softmax_lse, s_dmask, ctx.rng = _flash_attn_forward(
            q, kv[:, 0], kv[:, 1], torch.empty_like(q), cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
            softmax_scale, causal=causal, return_softmax=return_softmax)
        ctx.save_for_backward(q, kv, out, softmax_lse, cu_seqlens_q, cu_seqlens_k)
        ctx.dropout_p, ctx.max_seqlen_q, ctx.max_seqlen_k = dropout_p, max_seqlen_q, max_seqlen_k
        ctx.softmax_scale, ctx.causal = softmax_scale, causal
        if not return_softmax:
            return out
        ctx.mark_non_differentiable(softmax_lse, s_dmask) if s_dmask is not None else ctx.mark_non_differentiable(softmax_lse)
        return out, softmax_lse, s_dmask

    @staticmethod
    def backward(ctx, dout, *args):
        q, kv, out, softmax_lse, cu_seqlens_q, cu_seqlens_k = ctx.saved_tensors
        dq = torch.empty_like(q)
        dkv = torch.empty_like(kv)
        _flash_attn_backward(dout, q, kv[:, 0], kv[:, 1], out, softmax_lse, dq, dkv[:, 0], dkv[:, 1], cu_seqlens_q,
                             cu_seqlens_k, ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.dropout_p, ctx.softmax_scale, ctx.causal,
                             rng=ctx.rng)
        return dq, dkv, None, None, None, None, None, None, None, None


def flash_bert_mha(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        return FlashAttnQKVPackedFunc.apply(*args)


def flash_encdec_mha(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        return FlashAttnKVPackedFunc.apply(*args)
