"""Stand-in for the reference's extension module `relative_self_attn_blaslt`
(onmt/modules/extensions/multihead_attn_blaslt/relative_self_attn.cpp:72-196, bindings :263-264; kernels and GEMM calls
relative_self_attn_cuda.cu): self-attention with projected relative positions, forward and backward, with the reference's
argument order and returned lists.

forward -> [input_lin_results [T,B,3E], pos_lin_results [R,B,E], attn_scores [B*H,T,T], dropout_results [B*H,T,T],
dropout_mask, matmul2_results [T,B,E], outputs [T,B,E]]; attn_scores are the scores before the mask and the softmax (the
backward recomputes the probabilities from them with the mask fused, which is why it takes the mask as a keyword).
backward -> [input_grads, input_weight_grads, pos_weight_grads, output_weight_grads, input_bias_grads, pos_bias_grads,
output_bias_grads, r_w_bias_grads, r_r_bias_grads].

Every product is nmtg_gemm; q + r_w_bias / q + r_r_bias, the relative shift fused with the sum of the two score terms, the
shift's adjoint, the sum of the two query-gradient terms and the bias gradients are the kernels of relative_position.py and
linear_gemm.colsum; softmax + dropout is mask_softmax_dropout_cuda. Extras (keyword only): `dropout_mask` replays an explicit
keep-mask in forward; `pad_mask` / `time_mask` in backward."""
import torch

from . import linear_blaslt, linear_gemm, mask_softmax_dropout_cuda as softmax_native, relative_position


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _mask_kwargs(mask, use_time_mask):
    if mask is None:
        return {}
    if use_time_mask:
        _check(mask.dim() == 2, "Timing mask is not 2D!")
        return dict(time_mask=mask)
    return dict(pad_mask=mask)


def relative_scores(queries, keys, r_head_k, r_w_bias, r_r_bias, heads, scale):
    """queries [Tq, B*H, D], keys [Tk, B*H, D], r_head_k [R, B*H, D] (views allowed) -> (q + r_w_bias) k^T * scale +
    shift((q + r_r_bias) r_k^T * scale)[:, :, :Tk], [B*H, Tq, Tk]."""
    _check(r_head_k.size(0) >= keys.size(0), "relative attention: %d relative positions for %d keys" % (r_head_k.size(0), keys.size(0)))
    rw_head_q, rr_head_q = relative_position.query_bias(queries, r_w_bias, r_r_bias, heads)
    scores = linear_gemm.gemm(rw_head_q.transpose(0, 1), keys.transpose(0, 1), trans_b=True, alpha=scale)
    matmul_bd = linear_gemm.gemm(rr_head_q.transpose(0, 1), r_head_k.transpose(0, 1), trans_b=True, alpha=scale)
    return relative_position.shift_add_(scores, matmul_bd)


def attend(scores, values, is_training, heads, dropout_prob, mask_kw, dropout_mask=None):
    """scores [B*H, Tq, Tk], values [Tk, B*H, D] -> (dropout_mask, dropout_results, context [Tq, B*H, D])."""
    dmask, _, dropped = softmax_native.forward(is_training, heads, scores, dropout_prob, dropout_mask=dropout_mask,
                                               want_softmax=False, **mask_kw)
    context = torch.empty(scores.size(1), values.size(1), values.size(2), dtype=values.dtype, device=values.device)
    linear_gemm.gemm(dropped, values.transpose(0, 1), out=context.transpose(0, 1))
    return dmask, dropped, context


def forward(is_training, use_time_mask, heads, inputs, pos, input_weights, output_weights, pos_weights, input_biases,
            output_biases, pos_biases, r_w_bias, r_r_bias, pad_mask, dropout_prob, *, dropout_mask=None):
    _check(inputs.dim() == 3 and pos.dim() == 3 and pos.size(1) == inputs.size(1) and pos.size(2) == inputs.size(2),
           "relative_self_attn: inputs [T, B, E] and pos [R, B, E] required")
    inputs, pos = inputs.contiguous(), pos.contiguous()
    len_q, bsz, embed = inputs.shape
    _check(embed % heads == 0, "relative_self_attn: embed_dim must be divisible by heads")
    head_dim = embed // heads
    lin = linear_blaslt.forward(inputs, input_weights, input_biases)
    pos_lin = linear_blaslt.forward(pos, pos_weights, pos_biases)
    lin4 = lin.view(len_q, bsz * heads, 3, head_dim)
    scores = relative_scores(lin4[:, :, 0, :], lin4[:, :, 1, :], pos_lin.view(pos.size(0), bsz * heads, head_dim), r_w_bias,
                             r_r_bias, heads, head_dim ** -0.5)
    dmask, dropped, context = attend(scores, lin4[:, :, 2, :], is_training, heads, dropout_prob,
                                     _mask_kwargs(pad_mask, use_time_mask), dropout_mask)
    matmul2_results = context.view(len_q, bsz, embed)
    outputs = linear_blaslt.forward(matmul2_results, output_weights, output_biases)
    return [lin, pos_lin, scores, dropped, dmask, matmul2_results, outputs]


def backward(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_results, pos_lin_results, r_w_bias,
             r_r_bias, inputs, pos, input_weights, output_weights, pos_weights, dropout_mask, dropout_prob, *, pad_mask=None,
             time_mask=None):
    _check(pad_mask is None or time_mask is None, "relative_self_attn: give a key-padding mask or a time mask, not both")
    output_grads = output_grads.contiguous()
    len_q, bsz, embed = inputs.shape
    head_dim = embed // heads
    scale = head_dim ** -0.5
    len_r = pos.size(0)
    lin4 = input_lin_results.view(len_q, bsz * heads, 3, head_dim)
    queries, keys, values = lin4[:, :, 0, :], lin4[:, :, 1, :], lin4[:, :, 2, :]
    r_head_k = pos_lin_results.view(len_r, bsz * heads, head_dim)
    rw_head_q, rr_head_q = relative_position.query_bias(queries, r_w_bias, r_r_bias, heads)      # recomputed, not saved

    output_lin_grads, output_weight_grads, output_bias_grads = \
        linear_blaslt.backward(matmul2_results, output_weights, output_grads, True)
    output_lin_grads = output_lin_grads.view(len_q, bsz * heads, head_dim).transpose(0, 1)        # [B*H, T, D]
    lin_grads = torch.empty_like(lin4)
    queries_grads, keys_grads, values_grads = lin_grads[:, :, 0, :], lin_grads[:, :, 1, :], lin_grads[:, :, 2, :]
    matmul2_dgrad1 = linear_gemm.gemm(output_lin_grads, values.transpose(0, 1), trans_b=True)    # [B*H, T, T]
    linear_gemm.gemm(dropout_results, output_lin_grads, trans_a=True, out=values_grads.transpose(0, 1))
    # dropout and softmax backward in one kernel, probabilities recomputed from the saved scores (mask fused)
    score_grads = softmax_native.backward_recompute(heads, matmul2_dgrad1, None, attn_scores, dropout_mask, dropout_prob,
                                                    pad_mask=pad_mask, time_mask=time_mask)
    del matmul2_dgrad1

    # the score gradient flows to both terms: AC directly, BD through the adjoint of the shift
    queries_grads_ac = torch.empty(len_q, bsz * heads, head_dim, dtype=inputs.dtype, device=inputs.device)
    queries_grads_bd = torch.empty_like(queries_grads_ac)
    linear_gemm.gemm(score_grads, keys.transpose(0, 1), alpha=scale, out=queries_grads_ac.transpose(0, 1))
    linear_gemm.gemm(score_grads, rw_head_q.transpose(0, 1), trans_a=True, alpha=scale, out=keys_grads.transpose(0, 1))
    r_w_bias_grads = linear_gemm.colsum(queries_grads_ac.view(len_q * bsz, embed)).view(heads, head_dim)
    matmul_bd_grads = relative_position.shift_backward(score_grads, len_r)                        # [B*H, T, R]
    del score_grads
    linear_gemm.gemm(matmul_bd_grads, r_head_k.transpose(0, 1), alpha=scale, out=queries_grads_bd.transpose(0, 1))
    r_head_k_grad = torch.empty(len_r, bsz * heads, head_dim, dtype=inputs.dtype, device=inputs.device)
    linear_gemm.gemm(matmul_bd_grads, rr_head_q.transpose(0, 1), trans_a=True, alpha=scale, out=r_head_k_grad.transpose(0, 1))
    del matmul_bd_grads
    r_r_bias_grads = linear_gemm.colsum(queries_grads_bd.view(len_q * bsz, embed)).view(heads, head_dim)
    relative_position.add_rows(queries_grads_ac, queries_grads_bd, out=queries_grads)

    _, pos_weight_grads, pos_bias_grads = linear_blaslt.backward(pos, pos_weights, r_head_k_grad.view(len_r, bsz, embed), False)
    input_grads, input_weight_grads, input_bias_grads = \
        linear_blaslt.backward(inputs, input_weights, lin_grads.view(len_q, bsz, 3 * embed), True)
    return [input_grads, input_weight_grads, pos_weight_grads, output_weight_grads, input_bias_grads, pos_bias_grads,
            output_bias_grads, r_w_bias_grads, r_r_bias_grads]
