"""Bias-free encoder-decoder attention autograd function on the HIP kernels.

Mirrors EncdecAttnFunc / encdec_attn_func of the reference (onmt/modules/optimized/encdec_attention_func.py:36-568, the
function its own EncdecMultiheadAttn module binds, encdec_attention.py:6,35,147): the same 17 positional arguments
(recompute, is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, mask,
dropout_prob, incremental, incremental_cache, rotary_pos_enc, pos_emb_q, pos_emb_k, double_precision, return_coverage)
and 17 gradient slots. As in the reference's fused branch (:81-126) the coverage returned is `softmax_results`, the
probabilities BEFORE dropout (its Python fallback returns the dropped ones, :288-293). The mask is a key-padding mask
[B, Tk] (or the broadcast form [B, 1, Tk]). Incremental decoding runs in nmtgminor_amd/modules/incremental.py; rotary
encodings are applied by nmtgminor_amd/modules/rotary.py around the compact core. An 18th optional argument replays an
explicit dropout keep-mask. A training call with return_coverage false runs the tiled attention core of
nmtgminor_amd/modules/flash_core.py."""
import torch

from ..native import encdec_multihead_attn_cuda as native
from ._autocast import cast_if_autocast_enabled, no_autocast


class EncdecAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, recompute, is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights,
                mask, dropout_prob, incremental, incremental_cache, rotary_pos_enc, pos_emb_q, pos_emb_k, double_precision,
                return_coverage, dropout_mask=None):
        if rotary_pos_enc:
            raise NotImplementedError("encdec_attn_func: rotary position encoding takes the path in encdec_attn_func()")
        if incremental:
            raise NotImplementedError("encdec_attn_func: incremental decoding takes the path in encdec_attn_func()")
        if double_precision:
            raise RuntimeError("encdec_attn_func: the MFMA path computes in fp16 / bf16 with fp32 accumulation")
        if mask is not None and mask.dim() == 3:
            mask = mask.squeeze(1)
        ctx.heads, ctx.p, ctx.recompute, ctx.return_coverage = heads, dropout_prob, recompute, return_coverage
        q_lin, kv_lin, softmax, dropped, dmask, ctx_t, outputs = native.forward(
            is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, mask, dropout_prob,
            dropout_mask=dropout_mask)
        if recompute:
            ctx.save_for_backward(inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, mask, dmask)
        else:
            ctx.save_for_backward(inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, ctx_t, dropped,
                                  softmax, q_lin, kv_lin, dmask)
        if return_coverage:
            ctx.mark_non_differentiable(softmax)
            return outputs, softmax
        return (outputs,)

    @staticmethod
    def backward(ctx, *output_grads):
        g = output_grads[0].contiguous()
        heads, p = ctx.heads, ctx.p
        if ctx.recompute:
            x_q, x_kv, w_q, w_kv, w_out, mask, dmask = ctx.saved_tensors
            grads = native.backward_recompute(heads, g, x_q, x_kv, w_q, w_kv, w_out, dmask, mask, p)
        else:
            x_q, x_kv, w_q, w_kv, w_out, ctx_t, dropped, softmax, q_lin, kv_lin, dmask = ctx.saved_tensors
            grads = native.backward(heads, g, ctx_t, dropped, softmax, q_lin, kv_lin, x_q, x_kv, w_q, w_kv, w_out, dmask, p)
        dxq, dxkv, dwq, dwkv, dwo = grads
        return (None, None, None, dxq, dxkv, dwq, dwkv, dwo, None, None, None, None, None, None, None, None, None, None)


def encdec_attn_func(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        if len(args) > 11 and args[10]:               # incremental decoding: encoder keys / values come from the cache
            from .incremental import encdec_attn_step
            (_, _, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, mask, _, _, cache, rotary) = args[:13]
            if rotary:
                raise NotImplementedError("encdec_attn_func: rotary position encoding with incremental decoding")
            if cache is None:
                raise RuntimeError("encdec_attn_func: incremental decoding needs an incremental_cache dict")
            if mask is not None and mask.dim() == 3:
                mask = mask.squeeze(1)
            outputs, probs = encdec_attn_step(heads, inputs_q, inputs_kv, w_q, w_kv, w_out, None, None, None, mask, cache)
            return (outputs, probs) if args[16] else (outputs,)
        if len(args) > 12 and args[12]:               # rotary position encodings
            from .rotary import EncdecAttnRotaryFunc
            (_, is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, mask, p, _, _, _, pos_q, pos_k) = args[:15]
            if pos_q is None or pos_k is None:
                raise RuntimeError("encdec_attn_func: rotary_pos_enc needs pos_emb_q and pos_emb_k, each (cos, sin)")
            if mask is not None and mask.dim() == 3:
                mask = mask.squeeze(1)
            r = EncdecAttnRotaryFunc.apply(is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, None, None, None, mask, p,
                                           pos_q[0], pos_q[1], pos_k[0], pos_k[1], args[17] if len(args) > 17 else None)
            return r if args[16] else (r[0],)
        if len(args) >= 17 and not args[15]:          # training call whose coverage nobody reads: no [B*H, Tq, Tk] tensor
            from . import flash_core
            (recompute, is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, mask, p) = args[:10]
            if flash_core.eligible(is_training, args[16], recompute, inputs_q, heads) and inputs_kv.dtype == inputs_q.dtype:
                return (flash_core.EncdecAttnFlashFunc.apply(heads, inputs_q, inputs_kv, w_q, w_kv, w_out, None, None, None, mask, p,
                                                             args[17] if len(args) > 17 else None),)
        return EncdecAttnFunc.apply(*args)
