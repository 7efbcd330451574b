"""Encoder-decoder attention autograd function on the HIP kernels.

Mirrors EncdecAttnBiasFunc / encdec_attn_bias_func and the compact variant of the reference
(onmt/modules/optimized/encdec_attention_func_bias.py:41-668, :687-1011): the same 20 positional
arguments and 20 gradient slots; biases may be None (the reference then leaves its fused path,
:69-73; here the fused path takes them). Rotary encodings take the composed path of nmtgminor_amd/modules/rotary.py;
incremental decoding (inference with a cache
dict) runs in nmtgminor_amd/modules/incremental.py. A 21st
optional argument replays an explicit dropout keep-mask. A training call with return_coverage false runs the tiled
attention core of nmtgminor_amd/modules/flash_core.py."""
import torch

from ..native import encdec_multihead_attn_bias_blaslt as native
from ._autocast import cast_if_autocast_enabled, no_autocast


class EncdecAttnBiasFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, recompute, is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv,
                output_weights, input_bias_q, input_bias_kv, output_bias, mask, dropout_prob, incremental,
                incremental_cache, rotary_pos_enc, pos_emb_q, pos_emb_k, low_precision, return_coverage,
                dropout_mask=None):
        if rotary_pos_enc or incremental:           # encdec_attn_bias_func routes both before it gets here
            raise RuntimeError("EncdecAttnBiasFunc: call encdec_attn_bias_func for rotary encodings / incremental decoding")
        ctx.heads, ctx.p, ctx.recompute, ctx.return_coverage = heads, dropout_prob, recompute, return_coverage
        ctx.has_bias = (input_bias_q is not None, input_bias_kv is not None, output_bias is not None)
        q_lin, kv_lin, scores, dropped, dmask, ctx_t, outputs = native.forward(
            is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, input_bias_q,
            input_bias_kv, output_bias, mask, dropout_prob, dropout_mask=dropout_mask, want_probs=bool(return_coverage),
            need_backward=any(ctx.needs_input_grad))
        if recompute:
            ctx.save_for_backward(inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, input_bias_q,
                                  input_bias_kv, mask, dmask)
        else:
            ctx.save_for_backward(inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, ctx_t, dropped,
                                  scores, q_lin, kv_lin, dmask)
        ctx.mark_non_differentiable(dropped)
        if return_coverage:
            return outputs, dropped
        return (outputs,)

    @staticmethod
    def backward(ctx, *output_grads):
        g = output_grads[0].contiguous()
        heads, p = ctx.heads, ctx.p
        if ctx.recompute:
            x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, mask, dmask = ctx.saved_tensors
            grads = native.backward_recompute(heads, g, x_q, x_kv, w_q, w_kv, b_q, b_kv, w_out, dmask, mask, p)
        else:
            x_q, x_kv, w_q, w_kv, w_out, ctx_t, dropped, scores, q_lin, kv_lin, dmask = ctx.saved_tensors
            if w_q.requires_grad:
                grads = native.backward(heads, g, ctx_t, dropped, scores, q_lin, kv_lin, x_q, x_kv, w_q, w_kv, w_out,
                                        dmask, p)
            else:
                grads = native.backward_input_only(heads, g, ctx_t, dropped, scores, q_lin, kv_lin, x_q, x_kv, w_q, w_kv,
                                                   w_out, dmask, p) + [None] * 6
        dxq, dxkv, dwq, dwkv, dwo, dbq, dbkv, dbo = grads
        hb = ctx.has_bias
        return (None, None, None, dxq, dxkv, dwq, dwkv, dwo, dbq if hb[0] else None, dbkv if hb[1] else None,
                dbo if hb[2] else None, None, None, None, None, None, None, None, None, None, None)


def encdec_attn_bias_func(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        if len(args) > 14 and args[13]:               # incremental decoding: encoder keys / values come from the cache
            from .incremental import encdec_attn_step
            (_, _, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, _, _, cache, rotary) = args[:16]
            if rotary:
                raise NotImplementedError("encdec_attn_bias_func: rotary position encoding has no HIP kernel")
            if cache is None:
                raise RuntimeError("encdec_attn_bias_func: incremental decoding needs an incremental_cache dict")
            outputs, probs = encdec_attn_step(heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, cache)
            return (outputs, probs) if args[19] else (outputs,)
        if len(args) > 15 and args[15]:               # rotary position encodings
            from .rotary import EncdecAttnRotaryFunc
            (_, is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, p, _, _, _, pos_q,
             pos_k) = args[:18]
            if pos_q is None or pos_k is None:
                raise RuntimeError("encdec_attn_bias_func: rotary_pos_enc needs pos_emb_q and pos_emb_k, each (cos, sin)")
            r = EncdecAttnRotaryFunc.apply(is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, p,
                                           pos_q[0], pos_q[1], pos_k[0], pos_k[1], args[20] if len(args) > 20 else None)
            return r if args[19] else (r[0],)
        if len(args) >= 20:                           # training call whose coverage nobody reads: no [B*H, Tq, Tk] tensor
            from . import flash_core
            (recompute, is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, p) = args[:13]
            if flash_core.eligible(is_training, args[19], recompute, inputs_q, heads) and inputs_kv.dtype == inputs_q.dtype:
                return (flash_core.EncdecAttnFlashFunc.apply(heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask,
                                                             p, args[20] if len(args) > 20 else None),)
        return EncdecAttnBiasFunc.apply(*args)


class EncdecAttnBiasCompactFunc(torch.autograd.Function):
    """Projections done by the caller: (recompute, is_training, heads, input_lin_q_results
    [Tq,B,E], input_lin_kv_results [Tk,B,2E], mask, dropout_prob, incremental, incremental_cache,
    rotary_pos_enc, pos_emb_q, pos_emb_k, low_precision, return_coverage) -> context [Tq,B,E]."""

    @staticmethod
    def forward(ctx, recompute, is_training, heads, q_lin, kv_lin, mask, dropout_prob, incremental, incremental_cache,
                rotary_pos_enc, pos_emb_q, pos_emb_k, low_precision, return_coverage, dropout_mask=None):
        if rotary_pos_enc or incremental:
            raise NotImplementedError("encdec_attn_bias_compact_func: rotary / incremental modes have no HIP kernel")
        q_lin, kv_lin = q_lin.contiguous(), kv_lin.contiguous()
        scores, dropped, dmask, ctx_t = native.forward_compact(is_training, heads, q_lin, kv_lin, mask, dropout_prob,
                                                               dropout_mask=dropout_mask,
                                                               need_backward=any(ctx.needs_input_grad))
        ctx.heads, ctx.p, ctx.return_coverage = heads, dropout_prob, return_coverage
        ctx.save_for_backward(q_lin, kv_lin, scores, dropped, dmask)
        ctx.mark_non_differentiable(dropped)
        if return_coverage:
            return ctx_t, dropped
        return (ctx_t,)

    @staticmethod
    def backward(ctx, *output_grads):
        q_lin, kv_lin, scores, dropped, dmask = ctx.saved_tensors
        dq, dkv = native.backward_compact(ctx.heads, output_grads[0].contiguous(), dropped, scores, q_lin, kv_lin, dmask,
                                          ctx.p)
        return (None, None, None, dq, dkv, None, None, None, None, None, None, None, None, None, None)


def encdec_attn_bias_compact_func(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        return EncdecAttnBiasCompactFunc.apply(*args)
