"""Self-attention with relative position encodings (Transformer-XL form) on the HIP kernels.

Mirrors RelativeShift, RelativeSelfAttnFunc and relative_self_attn_func of the reference
(onmt/modules/optimized/relative_self_attention_func.py:26-76, :79-726, :738-766): the same 21 positional arguments and
21 gradient slots. The projected-position form runs in native/relative_self_attn_blaslt.py (the stand-in of the reference's
extension of that name). Every product is an MFMA GEMM (nmtg_gemm through native/linear_gemm.py and native/linear_blaslt.py),
the additions of r_w_bias / r_r_bias are a kernel of native/relative_position.py, the relative shift with the sum of the two
score terms runs inside the softmax + dropout kernel and the shift's adjoint inside that kernel's backward (mask fused,
probabilities recomputed from the saved scores in the backward; separate shift kernels for key lengths the wide kernels do
not take), the bias gradients are column-sum kernels and the two
query-gradient terms are joined by the row-add kernel. What is left to PyTorch: views and allocation.

Covered: sinusoidal positions projected by pos_weights (learnable_pos=False) and learnable position embeddings
(learnable_pos=True: pos [len_q, len_k, head_dim], shared by heads and batch, no shift, no r_w_bias / r_r_bias, a gradient
for pos), key-padding or time mask, training and inference, fp16 / bf16, and incremental decoding with either kind of
positions (`incremental=True` with the reference's cache entries `k`, `v`, time-first [T, B, E]: the new keys and values
are appended, the queries attend to everything cached; learnable positions then come as [new queries, cached + new keys,
head_dim]; inference only). `recompute` is accepted and gives the same numbers; the intermediate tensors are kept either way. A 22nd
optional argument replays an explicit dropout keep-mask."""
import torch

from ..native import (linear_blaslt, linear_gemm, mask_softmax_dropout_cuda as softmax_native, relative_position,
                      relative_self_attn_blaslt as native)
from ._autocast import cast_if_autocast_enabled, no_autocast


class RelativeShift(object):
    """x [B, len_q, len_r]: zero column in front, read as [B, len_r + 1, len_q], first row dropped
    (relative_self_attention_func.py:26-76). Only the batch-first form exists, as in the reference."""

    @staticmethod
    def forward(x, batch_first, emb_last):
        assert len(x.shape) == 3, "Input must have 3 dimensions B x len_q x len_r or len_q x len_r x demb!"
        assert (batch_first or emb_last) and not (batch_first and emb_last), \
            "Batch first and Embedding last must be mutually exclusive"
        if not batch_first:
            raise NotImplementedError
        x = x.contiguous()
        return relative_position.shift_add_(torch.zeros_like(x), x)

    @staticmethod
    def backward(grad_x, batch_first, emb_last):
        if not batch_first:
            raise NotImplementedError
        return relative_position.shift_backward(grad_x, grad_x.size(2))


class RelativeSelfAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inputs, pos, use_time_mask, is_training, heads, input_weights, output_weights, pos_weights,
                input_biases, output_biases, pos_biases, r_w_bias, r_r_bias, mask, dropout_prob, incremental,
                incremental_cache, low_precision, learnable_pos, return_coverage, recompute, dropout_mask=None):
        if incremental and (is_training or torch.is_grad_enabled() and inputs.requires_grad):
            raise RuntimeError("relative_self_attn_func: incremental decoding is an inference path (no backward)")
        inputs = inputs.contiguous()
        len_q, bsz, embed = inputs.shape
        head_dim = embed // heads
        scale = head_dim ** -0.5
        mask_kw = native._mask_kwargs(mask, use_time_mask)
        ctx.heads, ctx.p = heads, dropout_prob if is_training else 0.0
        ctx.empty = inputs.numel() == 0 and not incremental
        if ctx.empty:
            # no positions or no sentences: empty results, and zero gradients for every parameter
            ctx.shapes = [None if t is None else (t.shape, t.dtype, t.device) for t in
                          (inputs, pos if learnable_pos else None, input_weights, output_weights, pos_weights, input_biases,
                           output_biases, pos_biases, r_w_bias, r_r_bias)]
            outputs = inputs.new_empty(len_q, bsz, embed)
            coverage = inputs.new_empty(bsz * heads, len_q, len_q)
            ctx.mark_non_differentiable(coverage)
            return (outputs, coverage) if return_coverage else outputs
        ctx.use_time_mask, ctx.return_coverage, ctx.learnable_pos = use_time_mask, return_coverage, learnable_pos

        if not learnable_pos:
            if pos.size(1) == 1:
                pos = pos.repeat(1, bsz, 1)      # one position projection per batch column, as the reference lays it out
            pos = pos.contiguous()
            if not incremental:
                lin, pos_lin, scores, dropped, dmask, matmul2_results, outputs = native.forward(
                    is_training, use_time_mask, heads, inputs, pos, input_weights, output_weights, pos_weights, input_biases,
                    output_biases, pos_biases, r_w_bias, r_r_bias, mask, dropout_prob, dropout_mask=dropout_mask)
                ctx.save_for_backward(inputs, pos, input_weights, output_weights, pos_weights, lin, pos_lin, r_w_bias, r_r_bias,
                                      scores, dropped, dmask, matmul2_results, mask)
                if return_coverage:
                    ctx.mark_non_differentiable(dropped)
                    return outputs, dropped
                return outputs

        lin = linear_blaslt.forward(inputs, input_weights, input_biases)                  # [T, B, 3E]
        lin4 = lin.view(len_q, bsz * heads, 3, head_dim)
        queries, keys, values = lin4[:, :, 0, :], lin4[:, :, 1, :], lin4[:, :, 2, :]
        if incremental:
            # the cache holds keys and values time-first as [T, B, E] (beam search re-indexes its batch dimension)
            keys, values = keys.reshape(len_q, bsz, embed), values.reshape(len_q, bsz, embed)
            if 'k' in incremental_cache and 'v' in incremental_cache:
                keys = torch.cat([incremental_cache['k'], keys], dim=0)
                values = torch.cat([incremental_cache['v'], values], dim=0)
            incremental_cache['k'], incremental_cache['v'] = keys, values
            len_k = keys.size(0)
            keys, values = keys.view(len_k, bsz * heads, head_dim), values.view(len_k, bsz * heads, head_dim)
        else:
            len_k = len_q
        if not learnable_pos:
            pos_lin = linear_blaslt.forward(pos, pos_weights, pos_biases)                 # [R, B, E]
            scores = native.relative_scores(queries, keys, pos_lin.view(pos.size(0), bsz * heads, head_dim), r_w_bias,
                                            r_r_bias, heads, scale)
        else:
            # learnable positions, pos [len_q, len_k, head_dim]: scores[bh][i][j] = scale (q[i][bh] k[j][bh] + q[i][bh]
            # pos[i][j]); the second product is batched over the query positions and written through the strides of the
            # [B*H, T, T] layout. Incremental decoding: len_k counts the cached keys too, pos has a row per new query
            # (relative_self_attention_func.py:187-204, :254-263).
            pos = pos.contiguous()
            if pos.dim() != 3 or pos.shape != (len_q, len_k, head_dim):
                raise RuntimeError("relative_self_attn_func: learnable positions must be [len_q, len_k, head_dim]")
            scores = linear_gemm.gemm(queries.transpose(0, 1), keys.transpose(0, 1), trans_b=True, alpha=scale)
            matmul_bd = torch.empty_like(scores)
            linear_gemm.gemm(queries, pos, trans_b=True, alpha=scale, out=matmul_bd.transpose(0, 1))
            relative_position.add_rows(scores, matmul_bd, out=scores)
            del matmul_bd
        dmask, dropped, context = native.attend(scores, values, is_training, heads, dropout_prob, mask_kw, dropout_mask)
        matmul2_results = context.view(len_q, bsz, embed)
        outputs = linear_blaslt.forward(matmul2_results, output_weights, output_biases)
        if not incremental:
            ctx.save_for_backward(inputs, pos, input_weights, output_weights, lin, scores, dropped, dmask, matmul2_results, mask)
            if return_coverage:
                ctx.mark_non_differentiable(dropped)
        return (outputs, dropped) if return_coverage else outputs

    @staticmethod
    def backward(ctx, *output_grads):
        heads, p = ctx.heads, ctx.p
        tail = (None,) * 9                                      # mask ... recompute, dropout_mask
        if ctx.empty:
            z = [None if s is None else torch.zeros(s[0], dtype=s[1], device=s[2]) for s in ctx.shapes]
            return (z[0], z[1], None, None, None, z[2], z[3], z[4], z[5], z[6], z[7], z[8], z[9]) + tail
        if not ctx.learnable_pos:
            (inputs, pos, input_weights, output_weights, pos_weights, lin, pos_lin, r_w_bias, r_r_bias, scores, dropped, dmask,
             matmul2_results, mask) = ctx.saved_tensors
            (input_grads, input_weight_grads, pos_weight_grads, output_weight_grads, input_bias_grads, pos_bias_grads,
             output_bias_grads, r_w_bias_grads, r_r_bias_grads) = native.backward(
                heads, output_grads[0], matmul2_results, dropped, scores, lin, pos_lin, r_w_bias, r_r_bias, inputs, pos,
                input_weights, output_weights, pos_weights, dmask, p, **native._mask_kwargs(mask, ctx.use_time_mask))
            return (input_grads, None, None, None, None, input_weight_grads, output_weight_grads, pos_weight_grads,
                    input_bias_grads, output_bias_grads, pos_bias_grads, r_w_bias_grads, r_r_bias_grads) + tail

        inputs, pos, input_weights, output_weights, lin, scores, dropped, dmask, matmul2_results, mask = ctx.saved_tensors
        grads = output_grads[0].contiguous()
        len_q, bsz, embed = inputs.shape
        head_dim = embed // heads
        scale = head_dim ** -0.5
        lin4 = lin.view(len_q, bsz * heads, 3, head_dim)
        queries, keys, values = lin4[:, :, 0, :], lin4[:, :, 1, :], lin4[:, :, 2, :]
        output_lin_grads, output_weight_grads, output_bias_grads = linear_blaslt.backward(matmul2_results, output_weights, grads, True)
        output_lin_grads = output_lin_grads.view(len_q, bsz * heads, head_dim).transpose(0, 1)      # [B*H, T, D]
        lin_grads = torch.empty_like(lin4)
        queries_grads, keys_grads, values_grads = lin_grads[:, :, 0, :], lin_grads[:, :, 1, :], lin_grads[:, :, 2, :]
        matmul2_dgrad1 = linear_gemm.gemm(output_lin_grads, values.transpose(0, 1), trans_b=True)  # [B*H, T, T]
        linear_gemm.gemm(dropped, output_lin_grads, trans_a=True, out=values_grads.transpose(0, 1))
        score_grads = softmax_native.backward_recompute(heads, matmul2_dgrad1, None, scores, dmask, p,
                                                        **native._mask_kwargs(mask, ctx.use_time_mask))
        del matmul2_dgrad1
        queries_grads_ac = torch.empty(len_q, bsz * heads, head_dim, dtype=lin.dtype, device=lin.device)
        queries_grads_bd = torch.empty_like(queries_grads_ac)
        linear_gemm.gemm(score_grads, keys.transpose(0, 1), alpha=scale, out=queries_grads_ac.transpose(0, 1))
        linear_gemm.gemm(score_grads, queries.transpose(0, 1), trans_a=True, alpha=scale, out=keys_grads.transpose(0, 1))
        # both products with the positions are batched over the query positions
        by_query = score_grads.transpose(0, 1)                                                     # [T, B*H, T]
        linear_gemm.gemm(by_query, pos, alpha=scale, out=queries_grads_bd)
        pos_grads = linear_gemm.gemm(by_query, queries, trans_a=True, alpha=scale)                 # [T, T, D]
        del score_grads
        relative_position.add_rows(queries_grads_ac, queries_grads_bd, out=queries_grads)
        input_grads, input_weight_grads, input_bias_grads = \
            linear_blaslt.backward(inputs, input_weights, lin_grads.view(len_q, bsz, 3 * embed), True)
        return (input_grads, pos_grads, None, None, None, input_weight_grads, output_weight_grads, None, input_bias_grads,
                output_bias_grads, None, None, None) + tail


def relative_self_attn_func(input, pos, use_mask, is_training, num_heads, in_proj_weight, out_proj_weight,
                            pos_proj_weight, in_proj_bias, out_proj_bias, pos_proj_bias, r_w_bias, r_r_bias, mask, dropout,
                            incremental, incremental_cache, low_precision, learnable_pos, return_coverage, recompute,
                            dropout_mask=None):
    (input, pos, in_proj_weight, out_proj_weight, pos_proj_weight, in_proj_bias, out_proj_bias, pos_proj_bias, r_w_bias,
     r_r_bias) = cast_if_autocast_enabled(input, pos, in_proj_weight, out_proj_weight, pos_proj_weight, in_proj_bias,
                                          out_proj_bias, pos_proj_bias, r_w_bias, r_r_bias)
    with no_autocast():
        return RelativeSelfAttnFunc.apply(input, pos, use_mask, is_training, num_heads, in_proj_weight, out_proj_weight,
                                          pos_proj_weight, in_proj_bias, out_proj_bias, pos_proj_bias, r_w_bias, r_r_bias,
                                          mask, dropout, incremental, incremental_cache, low_precision, learnable_pos,
                                          return_coverage, recompute, dropout_mask)
