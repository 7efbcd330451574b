"""Self-attention autograd function on the HIP kernels.

Mirrors SelfAttnFunc / self_attn_func and SelfAttnCompactFunc / self_attn_compact_func of the
reference (onmt/modules/optimized/self_attention_func.py:50-520, :523-837): the same 17
positional arguments and 17 gradient slots. Every call takes the fused path (fp16 or bf16, biases
optional, T <= 4096). Rotary position encodings take the composed path of nmtgminor_amd/modules/rotary.py (projection
GEMM, rotation kernel, compact core); rotary together with incremental decoding raises. Incremental decoding (inference, `incremental=True` with a cache dict) runs in
nmtgminor_amd/modules/incremental.py. As in the reference's fused branch the result is always
the pair (outputs, dropout_results). An 18th optional argument replays an explicit dropout
keep-mask. A training call with return_coverage false (key padding mask, time mask or none) runs the tiled attention core
of nmtgminor_amd/modules/flash_core.py instead and returns an empty tensor as dropout_results."""
import torch

from ..native import self_multihead_attn_blaslt as native
from ._autocast import cast_if_autocast_enabled, no_autocast


def _unsupported(rotary_pos_enc, incremental):
    if rotary_pos_enc:
        raise NotImplementedError("self_attn_func: rotary position encoding has no HIP kernel")
    if incremental:
        raise NotImplementedError("self_attn_func: incremental decoding has no HIP kernel")


class SelfAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, use_time_mask, is_training, heads, inputs, input_weights, output_weights, input_biases,
                output_biases, mask, dropout_prob, rotary_pos_enc, pos_emb, incremental, incremental_cache,
                low_precision, return_coverage, recompute, dropout_mask=None):
        _unsupported(rotary_pos_enc, incremental)
        inputs = inputs.contiguous()
        ctx.heads = heads
        ctx.p = dropout_prob
        ctx.use_time_mask = use_time_mask
        ctx.recompute = recompute
        ctx.return_coverage = return_coverage
        ctx.has_in_bias = input_biases is not None
        ctx.has_out_bias = output_biases is not None
        lin, scores, dropped, dmask, ctx_t, outputs = native.forward(
            use_time_mask, is_training, heads, inputs, input_weights, output_weights, input_biases, output_biases, mask,
            dropout_prob, dropout_mask=dropout_mask, want_probs=bool(return_coverage),
            need_backward=any(ctx.needs_input_grad))
        if recompute:
            ctx.save_for_backward(inputs, input_weights, output_weights, input_biases, output_biases, mask, dmask)
        else:
            ctx.save_for_backward(inputs, input_weights, output_weights, ctx_t, dropped, scores, lin, dmask)
        ctx.mark_non_differentiable(dropped)
        return outputs, dropped

    @staticmethod
    def backward(ctx, output_grads, coverage_grads=None):
        p, heads = ctx.p, ctx.heads
        output_grads = output_grads.contiguous()
        if ctx.recompute:
            inputs, w_in, w_out, b_in, b_out, mask, dmask = ctx.saved_tensors
            grads = native.backward_recompute(ctx.use_time_mask, heads, output_grads, inputs, w_in, w_out, b_in, b_out,
                                              mask, dmask, p)
        else:
            inputs, w_in, w_out, ctx_t, dropped, scores, lin, dmask = ctx.saved_tensors
            if w_in.requires_grad:
                grads = native.backward(ctx.use_time_mask, heads, output_grads, ctx_t, dropped, scores, lin, inputs, w_in,
                                        w_out, dmask, p)
            else:
                dx = native.backward_input_only(ctx.use_time_mask, heads, output_grads, ctx_t, dropped, scores, lin,
                                                inputs, w_in, w_out, dmask, p)
                grads = [dx, None, None, None, None]
        dx, dw_in, dw_out, db_in, db_out = grads
        if not ctx.has_in_bias:
            db_in = None
        if not ctx.has_out_bias:
            db_out = None
        return (None, None, None, dx, dw_in, dw_out, db_in, db_out, None, None, None, None, None, None, None, None, None,
                None)


def self_attn_func(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        if len(args) > 13 and args[12]:               # incremental decoding: cache in, one more position out
            from .incremental import self_attn_step
            (use_time_mask, is_training, heads, inputs, w_in, w_out, b_in, b_out, mask, p, rotary, pos_emb, _, cache) = args[:14]
            if rotary:
                raise NotImplementedError("self_attn_func: rotary position encoding has no HIP kernel")
            if cache is None:
                raise RuntimeError("self_attn_func: incremental decoding needs an incremental_cache dict")
            return self_attn_step(heads, inputs, w_in, w_out, b_in, b_out, mask, cache, bool(use_time_mask))
        if len(args) > 11 and args[10]:               # rotary position encodings: projection, rotation, compact core
            from .rotary import SelfAttnRotaryFunc
            (use_time_mask, is_training, heads, inputs, w_in, w_out, b_in, b_out, mask, p, _, pos_emb) = args[:12]
            if pos_emb is None:
                raise RuntimeError("self_attn_func: rotary_pos_enc needs pos_emb = (cos, sin)")
            cos, sin = pos_emb
            return SelfAttnRotaryFunc.apply(use_time_mask, is_training, heads, inputs, w_in, w_out, b_in, b_out, mask, p, cos,
                                            sin, args[17] if len(args) > 17 else None)
        if len(args) >= 17:                           # training call whose coverage nobody reads: no [B*H, T, T] tensor
            from . import flash_core
            (use_time_mask, is_training, heads, inputs, w_in, w_out, b_in, b_out, mask, p) = args[:10]
            if flash_core.eligible(is_training, args[15], args[16], inputs, heads):
                outputs = flash_core.SelfAttnFlashFunc.apply(bool(use_time_mask), heads, inputs, w_in, w_out, b_in, b_out, mask, p,
                                                             args[17] if len(args) > 17 else None)
                return outputs, outputs.new_empty(0)
        return SelfAttnFunc.apply(*args)


class SelfAttnCompactFunc(torch.autograd.Function):
    """The input projection is the caller's: `input_lin_results` [T, B, 3E] comes in, the context
    [T, B, E] goes out (reference signature: use_time_mask, is_training, heads, input_lin_results,
    mask, dropout_prob, rotary_pos_enc, pos_emb, incremental, incremental_cache, low_precision,
    return_coverage, recompute)."""

    @staticmethod
    def forward(ctx, use_time_mask, is_training, heads, input_lin_results, mask, dropout_prob, rotary_pos_enc, pos_emb,
                incremental, incremental_cache, low_precision, return_coverage, recompute, dropout_mask=None):
        _unsupported(rotary_pos_enc, incremental)
        lin = input_lin_results.contiguous()
        scores, dropped, dmask, ctx_t = native.forward_compact(use_time_mask, is_training, heads, lin, mask, dropout_prob,
                                                               dropout_mask=dropout_mask)
        ctx.heads, ctx.p, ctx.use_time_mask = heads, dropout_prob, use_time_mask
        ctx.save_for_backward(lin, scores, dropped, dmask)
        ctx.mark_non_differentiable(dropped)
        return ctx_t, dropped

    @staticmethod
    def backward(ctx, output_grads, coverage_grads=None):
        lin, scores, dropped, dmask = ctx.saved_tensors
        (dlin,) = native.backward_compact(ctx.use_time_mask, ctx.heads, output_grads.contiguous(), dropped, scores, lin,
                                          dmask, ctx.p)
        return (None, None, None, dlin, None, None, None, None, None, None, None, None, None, None)


def self_attn_compact_func(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        return SelfAttnCompactFunc.apply(*args)
