"""Attention with rotary position encodings on the HIP kernels.

The reference leaves its fused extensions when rotary_pos_enc is set and runs PyTorch ops
(onmt/modules/optimized/self_attention_func.py:84-86, :178-184, :467-469;
onmt/modules/optimized/encdec_attention_func.py:21-34, :81-82). Here the same computation is the projection GEMM, the
rotation kernel in place on the query / key slots of the projection (as the reference's `queries.copy_(queries_)` does),
the compact attention core, and the output GEMM; the backward runs them in reverse with the transposed rotation on the
gradient of the projection. pos_emb is the reference's pair (cos, sin), each [T, 1, D]. As in the reference's
non-fused branch the coverage is dropout_results."""
import torch

from ..native import encdec_multihead_attn_bias_blaslt as ed_native
from ..native import rotary_position as rot
from ..native import self_multihead_attn_blaslt as sa_native
from ..native.linear_gemm import colsum, gemm


def _linear(x3, w, b):
    t, bsz, e = x3.shape
    return gemm(x3.reshape(t * bsz, e), w, False, True, bias=b).view(t, bsz, w.shape[0])


def _linear_bwd(dy3, x3, w, want_w, want_b):
    """-> dx [T, B, in], dW [out, in] | None, db [out] | None."""
    t, bsz, out_f = dy3.shape
    dy2 = dy3.reshape(t * bsz, out_f)
    dx = gemm(dy2, w).view(t, bsz, w.shape[1])
    dw = gemm(dy2, x3.reshape(t * bsz, x3.shape[2]), trans_a=True) if want_w else None
    db = colsum(dy2) if want_b else None
    return dx, dw, db


class SelfAttnRotaryFunc(torch.autograd.Function):
    """apply(use_time_mask, is_training, heads, inputs, input_weights, output_weights, input_biases, output_biases, mask,
    dropout_prob, cos, sin, dropout_mask=None) -> (outputs, dropout_results)."""

    @staticmethod
    def forward(ctx, use_time_mask, is_training, heads, inputs, w_in, w_out, b_in, b_out, mask, p, cos, sin, dropout_mask=None):
        inputs = inputs.contiguous()
        t, bsz, e = inputs.shape
        d = e // heads
        lin = _linear(inputs, w_in, b_in)
        rot.rotate_qk_(lin, cos, sin, bsz * heads, d)
        scores, dropped, dmask, ctx_t = sa_native.forward_compact(use_time_mask, is_training, heads, lin, mask, p,
                                                                  dropout_mask=dropout_mask)
        outputs = _linear(ctx_t, w_out, b_out)
        ctx.heads, ctx.p, ctx.use_time_mask = heads, p, use_time_mask
        ctx.has_bias = (b_in is not None, b_out is not None)
        ctx.save_for_backward(inputs, w_in, w_out, lin, scores, dropped, dmask, ctx_t, cos, sin)
        ctx.mark_non_differentiable(dropped)
        return outputs, dropped

    @staticmethod
    def backward(ctx, output_grads, coverage_grads=None):
        inputs, w_in, w_out, lin, scores, dropped, dmask, ctx_t, cos, sin = ctx.saved_tensors
        t, bsz, e = inputs.shape
        heads = ctx.heads
        want_w = w_in.requires_grad
        dctx, dw_out, db_out = _linear_bwd(output_grads.contiguous(), ctx_t, w_out, want_w, want_w and ctx.has_bias[1])
        (dlin,) = sa_native.backward_compact(ctx.use_time_mask, heads, dctx, dropped, scores, lin, dmask, ctx.p)
        rot.rotate_qk_(dlin, cos, sin, bsz * heads, e // heads, inverse=True)
        dx, dw_in, db_in = _linear_bwd(dlin, inputs, w_in, want_w, want_w and ctx.has_bias[0])
        return (None, None, None, dx, dw_in, dw_out, db_in, db_out, None, None, None, None, None)


class EncdecAttnRotaryFunc(torch.autograd.Function):
    """apply(is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, dropout_prob, cos_q, sin_q,
    cos_k, sin_k, dropout_mask=None) -> (outputs, dropout_results); the queries are rotated with the query positions'
    table and the keys with the key positions' (encdec_attention_func.py:150-160)."""

    @staticmethod
    def forward(ctx, is_training, heads, inputs_q, inputs_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, mask, p, cos_q, sin_q, cos_k,
                sin_k, dropout_mask=None):
        inputs_q, inputs_kv = inputs_q.contiguous(), inputs_kv.contiguous()
        tq, bsz, e = inputs_q.shape
        d = e // heads
        q_lin = _linear(inputs_q, w_q, b_q)
        kv_lin = _linear(inputs_kv, w_kv, b_kv)
        rot.rotate_q_(q_lin, cos_q, sin_q, bsz * heads, d)
        rot.rotate_k_(kv_lin, cos_k, sin_k, bsz * heads, d)
        scores, dropped, dmask, ctx_t = ed_native.forward_compact(is_training, heads, q_lin, kv_lin, mask, p,
                                                                  dropout_mask=dropout_mask,
                                                                  need_backward=any(ctx.needs_input_grad))
        outputs = _linear(ctx_t, w_out, b_out)
        ctx.heads, ctx.p = heads, p
        ctx.has_bias = (b_q is not None, b_kv is not None, b_out is not None)
        ctx.save_for_backward(inputs_q, inputs_kv, w_q, w_kv, w_out, q_lin, kv_lin, scores, dropped, dmask, ctx_t, cos_q, sin_q,
                              cos_k, sin_k)
        ctx.mark_non_differentiable(dropped)
        return outputs, dropped

    @staticmethod
    def backward(ctx, output_grads, coverage_grads=None):
        (inputs_q, inputs_kv, w_q, w_kv, w_out, q_lin, kv_lin, scores, dropped, dmask, ctx_t, cos_q, sin_q, cos_k,
         sin_k) = ctx.saved_tensors
        tq, bsz, e = inputs_q.shape
        heads = ctx.heads
        d = e // heads
        want_w = w_q.requires_grad
        hb = ctx.has_bias
        dctx, dw_out, db_out = _linear_bwd(output_grads.contiguous(), ctx_t, w_out, want_w, want_w and hb[2])
        dq, dkv = ed_native.backward_compact(heads, dctx, dropped, scores, q_lin, kv_lin, dmask, ctx.p)
        rot.rotate_q_(dq, cos_q, sin_q, bsz * heads, d, inverse=True)
        rot.rotate_k_(dkv, cos_k, sin_k, bsz * heads, d, inverse=True)
        dxq, dw_q, db_q = _linear_bwd(dq, inputs_q, w_q, want_w, want_w and hb[0])
        dxkv, dw_kv, db_kv = _linear_bwd(dkv, inputs_kv, w_kv, want_w, want_w and hb[1])
        return (None, None, dxq, dxkv, dw_q, dw_kv, dw_out, db_q, db_kv, db_out, None, None, None, None, None, None, None)
