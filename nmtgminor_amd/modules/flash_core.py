"""Training calls of self_attn_func / encdec_attn_bias_func that nobody asks the coverage of.

The reference's fused extensions write the scores, the probabilities and the dropped probabilities as [B*H, len_q, len_k]
tensors because their backward reads them and because return_coverage hands one of them out
(onmt/modules/optimized/self_attention_func.py:102-131, :284-287; encdec_attention_func_bias.py:105-135). With
return_coverage=False nothing outside the function sees them, and the attention core runs as the tiled kernels of
nmtg_flash_attn_batched_fwd / _bwd on the slots of the projections (queries, keys and values are read where the
projection GEMM left them, and their gradients are written into the slots of one gradient buffer): per call the forward
keeps the projections, the context, one fp32 per (sequence, head, query) and one bit per element of the dropout mask.

Taken when: training mode, return_coverage false, no recompute, 16-bit tensors, head dimension 64 or 128.
The mask is the reference's key padding mask ([B, len_k] or [B, 1, 1, len_k], 1 = masked), its time mask ([len_q, len_k]
with use_time_mask, any pattern) or None. A query whose keys are all masked gets a zero context here (the reference's
softmax gives NaN). NMTG_ATTN_FLASH_TRAIN=0 keeps such calls on
the extension's path."""
import os

import torch

from ..native import flash_attn_cuda as fa
from .rotary import _linear, _linear_bwd


def eligible(is_training, return_coverage, recompute, x, heads):
    if not is_training or return_coverage or recompute:
        return False
    if os.environ.get("NMTG_ATTN_FLASH_TRAIN", "1") == "0":
        return False
    e = x.shape[-1]
    return x.dtype in (torch.float16, torch.bfloat16) and x.dim() == 3 and e % heads == 0 and e // heads in (64, 128)


def _pad(mask, batch, len_k):
    if mask is None or mask.numel() == 0:
        return None
    if mask.numel() != batch * len_k:
        raise RuntimeError("key padding mask must be [batch, len_k]")
    mask = mask.reshape(batch, len_k).contiguous()
    return mask.view(torch.uint8) if mask.dtype == torch.bool else mask.to(torch.uint8)     # a bool mask is its bytes


def _time(mask, len_q, len_k):
    if mask is None or mask.numel() == 0:
        return None
    if mask.numel() != len_q * len_k:
        raise RuntimeError("time mask must be [len_q, len_k]")
    return _pad(mask, len_q, len_k)


class SelfAttnFlashFunc(torch.autograd.Function):
    """apply(use_time_mask, heads, inputs, input_weights, output_weights, input_biases, output_biases, mask, dropout_prob,
    dropout_mask=None) -> outputs [T, B, E]; mask: key padding [B, T], or with use_time_mask a time mask [T, T]"""

    @staticmethod
    def forward(ctx, use_time_mask, heads, inputs, w_in, w_out, b_in, b_out, mask, p, dropout_mask=None):
        inputs = inputs.contiguous()
        t, bsz, e = inputs.shape
        d = e // heads
        lin = _linear(inputs, w_in, b_in)                               # [T, B, H, 3, D]
        slots = lin.view(t, bsz, heads, 3, d)
        pad = None if use_time_mask else _pad(mask, bsz, t)
        tm = _time(mask, t, t) if use_time_mask else None
        ctx_t, lse, state = fa.fwd_batched(slots[:, :, :, 0], slots[:, :, :, 1], slots[:, :, :, 2], pad, p, d ** -0.5, False,
                                           dropout_mask=dropout_mask, time_mask=tm)
        outputs = _linear(ctx_t.view(t, bsz, e), w_out, b_out)
        ctx.heads, ctx.p, ctx.state = heads, p, state
        ctx.has_bias = (b_in is not None, b_out is not None)
        ctx.save_for_backward(inputs, w_in, w_out, lin, ctx_t, lse, pad, tm)
        return outputs

    @staticmethod
    def backward(ctx, output_grads):
        inputs, w_in, w_out, lin, ctx_t, lse, pad, tm = ctx.saved_tensors
        t, bsz, e = inputs.shape
        heads = ctx.heads
        d = e // heads
        want_w = w_in.requires_grad
        dctx, dw_out, db_out = _linear_bwd(output_grads.contiguous(), ctx_t.view(t, bsz, e), w_out, want_w,
                                           want_w and ctx.has_bias[1])
        slots = lin.view(t, bsz, heads, 3, d)
        dlin = torch.empty_like(lin)
        dslots = dlin.view(t, bsz, heads, 3, d)
        fa.bwd_batched(dctx.view(t, bsz, heads, d), slots[:, :, :, 0], slots[:, :, :, 1], slots[:, :, :, 2], ctx_t, lse,
                       dslots[:, :, :, 0], dslots[:, :, :, 1], dslots[:, :, :, 2], pad, ctx.p, d ** -0.5, False, ctx.state,
                       time_mask=tm)
        dx, dw_in, db_in = _linear_bwd(dlin, inputs, w_in, want_w, want_w and ctx.has_bias[0])
        return (None, None, dx, dw_in, dw_out, db_in, db_out, None, None, None)


class EncdecAttnFlashFunc(torch.autograd.Function):
    """apply(heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, dropout_prob, dropout_mask=None)
    -> outputs [Tq, B, E]"""

    @staticmethod
    def forward(ctx, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, p, dropout_mask=None):
        inputs_q, inputs_kv = inputs_q.contiguous(), inputs_kv.contiguous()
        tq, bsz, e = inputs_q.shape
        tk = inputs_kv.shape[0]
        d = e // heads
        q_lin = _linear(inputs_q, w_q, b_q)                             # [Tq, B, H, D]
        kv_lin = _linear(inputs_kv, w_kv, b_kv)                         # [Tk, B, H, 2, D]
        kv = kv_lin.view(tk, bsz, heads, 2, d)
        pad = _pad(mask, bsz, tk)
        ctx_t, lse, state = fa.fwd_batched(q_lin.view(tq, bsz, heads, d), kv[:, :, :, 0], kv[:, :, :, 1], pad, p, d ** -0.5,
                                           False, dropout_mask=dropout_mask)
        outputs = _linear(ctx_t.view(tq, bsz, e), w_out, b_out)
        ctx.heads, ctx.p, ctx.state = heads, p, state
        ctx.has_bias = (b_q is not None, b_kv is not None, b_out is not None)
        ctx.save_for_backward(inputs_q, inputs_kv, w_q, w_kv, w_out, q_lin, kv_lin, ctx_t, lse, pad)
        return outputs

    @staticmethod
    def backward(ctx, output_grads):
        inputs_q, inputs_kv, w_q, w_kv, w_out, q_lin, kv_lin, ctx_t, lse, pad = ctx.saved_tensors
        tq, bsz, e = inputs_q.shape
        tk = inputs_kv.shape[0]
        heads = ctx.heads
        d = e // heads
        hb = ctx.has_bias
        want_w = w_q.requires_grad
        dctx, dw_out, db_out = _linear_bwd(output_grads.contiguous(), ctx_t.view(tq, bsz, e), w_out, want_w, want_w and hb[2])
        kv = kv_lin.view(tk, bsz, heads, 2, d)
        dq_lin, dkv_lin = torch.empty_like(q_lin), torch.empty_like(kv_lin)
        dkv = dkv_lin.view(tk, bsz, heads, 2, d)
        fa.bwd_batched(dctx.view(tq, bsz, heads, d), q_lin.view(tq, bsz, heads, d), kv[:, :, :, 0], kv[:, :, :, 1], ctx_t, lse,
                       dq_lin.view(tq, bsz, heads, d), dkv[:, :, :, 0], dkv[:, :, :, 1], pad, ctx.p, d ** -0.5, False, ctx.state)
        dxq, dw_q, db_q = _linear_bwd(dq_lin, inputs_q, w_q, want_w, want_w and hb[0])
        dxkv, dw_kv, db_kv = _linear_bwd(dkv_lin, inputs_kv, w_kv, want_w, want_w and hb[1])
        return (None, dxq, dxkv, dw_q, dw_kv, dw_out, db_q, db_kv, db_out, None, None, None)
