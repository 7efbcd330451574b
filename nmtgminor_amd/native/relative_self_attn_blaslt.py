"""Stand-in for the reference's extension module `relative_self_attn_blaslt`
(onmt/modules/extensions/multihead_attn_blaslt/relative_self_attn.cpp:72-196, bindings :263-264; kernels and GEMM calls
relative_self_attn_cuda.cu): self-attention with projected relative positions, forward and backward, with the reference's
argument order and returned lists.

forward -> [input_lin_results [T,B,3E], pos_lin_results [R,B,E], attn_scores [B*H,T,T], dropout_results [B*H,T,T],
dropout_mask, matmul2_results [T,B,E], outputs [T,B,E]]; attn_scores are the scores before the mask and the softmax (the
backward recomputes the probabilities from them with the mask fused, which is why it takes the mask as a keyword).
backward -> [input_grads, input_weight_grads, pos_weight_grads, output_weight_grads, input_bias_grads, pos_bias_grads,
output_bias_grads, r_w_bias_grads, r_r_bias_grads].

Every product is nmtg_gemm; q + r_w_bias / q + r_r_bias, the sum of the two query-gradient terms and the bias gradients are
the kernels of relative_position.py and linear_gemm.colsum. The relative shift, the sum of the two score terms, the mask,
the softmax and the dropout are one kernel and their adjoints another (relative_position.shift_add_softmax_dropout /
softmax_dropout_shift_backward) for key lengths of a multiple of 16 bytes up to 4096; other shapes run the shift kernels and
mask_softmax_dropout_cuda one after the other. Extras (keyword only): `dropout_mask` replays an explicit
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


def _kernel_mask(mask_kw, len_q, len_k):
    """The keyword form of the mask -> (uint8 tensor or None, kind code of the softmax kernels)."""
    if "pad_mask" in mask_kw:
        return mask_kw["pad_mask"].reshape(-1, len_k).to(torch.uint8).contiguous(), 1
    if "time_mask" in mask_kw:
        _check(mask_kw["time_mask"].shape == (len_q, len_k), "softmax: time mask must be [len_q, len_k]")
        return mask_kw["time_mask"].to(torch.uint8).contiguous(), 2
    return None, 0


def scores_and_attend(queries, keys, values, r_head_k, r_w_bias, r_r_bias, heads, scale, is_training, dropout_prob, mask_kw,
                      dropout_mask=None):
    """relative_scores followed by attend -> (scores, dropout_mask, dropout_results, context). Where the shapes allow it the
    shift of the position term, its sum with the content term, the softmax and the dropout are one kernel."""
    _check(r_head_k.size(0) >= keys.size(0), "relative attention: %d relative positions for %d keys" % (r_head_k.size(0), keys.size(0)))
    shape = (queries.size(1), queries.size(0), keys.size(0))
    if not relative_position.fused_ok(shape, queries.dtype, r_head_k.size(0)):
        scores = relative_scores(queries, keys, r_head_k, r_w_bias, r_r_bias, heads, scale)
        return (scores,) + attend(scores, values, is_training, heads, dropout_prob, mask_kw, dropout_mask)
    rw_head_q, rr_head_q = relative_position.query_bias(queries, r_w_bias, r_r_bias, heads)
    scores = linear_gemm.gemm(rw_head_q.transpose(0, 1), keys.transpose(0, 1), trans_b=True, alpha=scale)
    matmul_bd = linear_gemm.gemm(rr_head_q.transpose(0, 1), r_head_k.transpose(0, 1), trans_b=True, alpha=scale)
    km, kind = _kernel_mask(mask_kw, shape[1], shape[2])
    _check(kind != 1 or km.shape[0] * heads == shape[0], "softmax: pad mask batch does not match inputs")
    dmask, dropped = relative_position.shift_add_softmax_dropout(scores, matmul_bd, is_training, heads, dropout_prob, km, kind,
                                                                 dropout_mask)
    context = torch.empty(shape[1], values.size(1), values.size(2), dtype=values.dtype, device=values.device)
    linear_gemm.gemm(dropped, values.transpose(0, 1), out=context.transpose(0, 1))
    return scores, dmask, dropped, context


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
    scores, dmask, dropped, context = scores_and_attend(
        lin4[:, :, 0, :], lin4[:, :, 1, :], lin4[:, :, 2, :], pos_lin.view(pos.size(0), bsz * heads, head_dim), r_w_bias, r_r_bias,
        heads, head_dim ** -0.5, is_training, dropout_prob, _mask_kwargs(pad_mask, use_time_mask), dropout_mask)
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
    fused = relative_position.fused_ok(attn_scores.shape, attn_scores.dtype, len_r)
    if fused:
        mask_kw = dict(pad_mask=pad_mask) if pad_mask is not None else dict(time_mask=time_mask) if time_mask is not None else {}
        km, kind = _kernel_mask(mask_kw, len_q, attn_scores.size(2))
        score_grads, matmul_bd_grads = relative_position.softmax_dropout_shift_backward(
            matmul2_dgrad1, attn_scores, len_r, heads, dropout_mask, dropout_prob, km, kind)
    else:
        score_grads = softmax_native.backward_recompute(heads, matmul2_dgrad1, None, attn_scores, dropout_mask, dropout_prob,
                                                        pad_mask=pad_mask, time_mask=time_mask)
    del matmul2_dgrad1

    # the score gradient flows to both terms: AC directly, BD through the adjoint of the shift
    queries_grads_ac = torch.empty(len_q, bsz * heads, head_dim, dtype=inputs.dtype, device=inputs.device)
    queries_grads_bd = torch.empty_like(queries_grads_ac)
    linear_gemm.gemm(score_grads, keys.transpose(0, 1), alpha=scale, out=queries_grads_ac.transpose(0, 1))
    linear_gemm.gemm(score_grads, rw_head_q.transpose(0, 1), trans_a=True, alpha=scale, out=keys_grads.transpose(0, 1))
    r_w_bias_grads = linear_gemm.colsum(queries_grads_ac.view(len_q * bsz, embed)).view(heads, head_dim)
    if not fused:
        matmul_bd_grads = relative_position.shift_backward(score_grads, len_r)                    # [B*H, T, R]
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
