"""Stand-in for the reference module `self_multihead_attn_blaslt`
(onmt/modules/extensions/multihead_attn_blaslt/self_multihead_attn.cpp:95-354): forward, backward,
forward_compact, backward_compact, backward_recompute; plus backward_input_only of the older
`self_multihead_attn_cuda` (onmt/modules/extensions/multihead_attn/self_multihead_attn.cpp:195-197).

Extras: biases may be None; fp16 and bf16 are accepted (the reference is fp16 only); `forward`
and `forward_compact` take an optional keyword `dropout_mask` to replay an explicit keep-mask."""
import torch

from .. import _lib as L
from . import _attn_common as A


def _dims(inputs, heads, last):
    A.check(inputs.dim() == 3, "expected 3D tensor")
    t, b, w = inputs.shape
    A.check(w % last == 0 and (w // last) % heads == 0, "embedding size does not match the number of heads")
    return t, b, w // last


def forward(use_time_mask, is_training, heads, inputs, input_weights, output_weights, input_biases, output_biases,
            pad_mask, dropout_prob, *, dropout_mask=None, want_probs=True, need_backward=None):
    """-> [input_lin_results, attn_scores, dropout_results, dropout_mask, matmul2_results, outputs]; attn_scores is empty
    for an inference call under torch.no_grad() (see _attn_common.scores_needed); such a call with want_probs=False
    (the caller does not return the coverage) leaves dropout_results empty too: no [B*H, T, T] tensor exists then."""
    L.require_cuda(inputs, input_weights, output_weights, input_biases, output_biases, pad_mask, dropout_mask)
    A.check(input_weights.dim() == 2 and output_weights.dim() == 2, "expected 2D tensor")
    A.check_half(inputs, input_weights, output_weights, input_biases, output_biases)
    t, b, e = _dims(inputs, heads, 1)
    A.check(input_weights.shape == (3 * e, e) and output_weights.shape == (e, e), "weight shapes do not match the input")
    x = inputs.contiguous()
    w_in, w_out = input_weights.contiguous(), output_weights.contiguous()
    b_in = input_biases.contiguous() if input_biases is not None else None
    b_out = output_biases.contiguous() if output_biases is not None else None
    dev, dt = x.device, x.dtype
    km, kind = A.mask_arg(pad_mask, use_time_mask, b, t, t)
    bh = b * heads
    lin = torch.empty(t, b, 3 * e, dtype=dt, device=dev)
    keep_scores = A.scores_needed(is_training, dt, e // heads, t, need_backward)
    scores = torch.empty((bh, t, t) if keep_scores else (0,), dtype=dt, device=dev)
    keep_probs = want_probs or keep_scores
    dropped = torch.empty((bh, t, t) if keep_probs else (0,), dtype=dt, device=dev)
    ctx = torch.empty(t, b, e, dtype=dt, device=dev)
    out = torch.empty(t, b, e, dtype=dt, device=dev)
    dmask, mode, seed, offset = A.dropout_args(is_training, dropout_prob, (bh, t, t), dev, dropout_mask)
    if t == 0 or b == 0:        # an empty batch: the (empty) buffers are the result
        return [lin, scores, dropped, dmask, ctx, out]
    L.call("nmtg_self_attn_fwd", L.ptr(x), L.ptr(w_in), L.ptr(w_out), L.ptr(b_in), L.ptr(b_out), L.ptr(km), L.i32(kind),
           L.ptr(lin), L.ptr(scores if keep_scores else None), L.ptr(None), L.ptr(dropped if keep_probs else None), L.ptr(dmask if mode else None), L.i32(mode),
           L.f32(dropout_prob), A.u64(seed), A.u64(offset), L.ptr(ctx), L.ptr(out), L.i64(t), L.i64(b), L.i64(e),
           L.i32(heads), L.i32(L.dtype_code(x)), L.stream_of(x))
    return [lin, scores, dropped, dmask, ctx, out]


def forward_compact(use_time_mask, is_training, heads, input_lin_results, pad_mask, dropout_prob, *, dropout_mask=None):
    """input_lin_results [T, B, 3E] (projection done by the caller).
    -> [attn_scores, dropout_results, dropout_mask, matmul2_results]"""
    L.require_cuda(input_lin_results, pad_mask, dropout_mask)
    A.check_half(input_lin_results)
    t, b, e = _dims(input_lin_results, heads, 3)
    lin = input_lin_results.contiguous()
    dev, dt = lin.device, lin.dtype
    km, kind = A.mask_arg(pad_mask, use_time_mask, b, t, t)
    bh = b * heads
    scores = torch.empty(bh, t, t, dtype=dt, device=dev)
    dropped = torch.empty(bh, t, t, dtype=dt, device=dev)
    ctx = torch.empty(t, b, e, dtype=dt, device=dev)
    dmask, mode, seed, offset = A.dropout_args(is_training, dropout_prob, (bh, t, t), dev, dropout_mask)
    L.call("nmtg_self_attn_fwd", L.ptr(None), L.ptr(None), L.ptr(None), L.ptr(None), L.ptr(None), L.ptr(km), L.i32(kind),
           L.ptr(lin), L.ptr(scores), L.ptr(None), L.ptr(dropped), L.ptr(dmask if mode else None), L.i32(mode),
           L.f32(dropout_prob), A.u64(seed), A.u64(offset), L.ptr(ctx), L.ptr(None), L.i64(t), L.i64(b), L.i64(e),
           L.i32(heads), L.i32(L.dtype_code(lin)), L.stream_of(lin))
    return [scores, dropped, dmask, ctx]


def _bwd(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_results, inputs, input_weights,
         output_weights, dropout_mask, dropout_prob, want_weights=True, want_biases=True):
    L.require_cuda(output_grads, dropout_results, attn_scores, input_lin_results, inputs, input_weights, output_weights)
    A.check(output_grads.dim() == 3 and dropout_results.dim() == 3 and input_lin_results.dim() == 3, "expected 3D tensor")
    A.check_half(output_grads, dropout_results, attn_scores, input_lin_results, inputs, input_weights, output_weights)
    t, b, e = _dims(input_lin_results, heads, 3)
    dev, dt = output_grads.device, output_grads.dtype
    g = output_grads.contiguous()
    use_mask = dropout_mask is not None and dropout_mask.numel() > 0 and dropout_prob > 0.0
    if use_mask:
        A.check(dropout_mask.dtype == torch.uint8, "Only BYTE is supported")
    compact = output_weights is None
    dx = dw_in = dw_out = db_in = db_out = dlin = None
    if compact:
        dlin = torch.empty(t, b, 3 * e, dtype=dt, device=dev)
    else:
        dx = torch.empty(t, b, e, dtype=dt, device=dev)
        if want_weights:
            dw_in = torch.empty(3 * e, e, dtype=dt, device=dev)
            dw_out = torch.empty(e, e, dtype=dt, device=dev)
        if want_weights and want_biases:
            db_in = torch.empty(3 * e, dtype=dt, device=dev)
            db_out = torch.empty(e, dtype=dt, device=dev)
    if t == 0 or b == 0:        # an empty batch contributes zero gradients
        for z in (dx, dw_in, dw_out, db_in, db_out, dlin):
            if z is not None:
                z.zero_()
        return dx, dw_in, dw_out, db_in, db_out, dlin
    ws_bytes = L.load().nmtg_self_attn_bwd_workspace_bytes(L.i64(t), L.i64(b), L.i64(e), L.i32(heads))
    ws = A.workspace(ws_bytes, dev)
    # contiguous copies (if any) are bound to names: a temporary would be freed before the kernels read it
    c = lambda z: z.contiguous() if z is not None else None
    (matmul2_results, dropout_results, attn_scores, input_lin_results, inputs, input_weights, output_weights) = map(
        c, (matmul2_results, dropout_results, attn_scores, input_lin_results, inputs, input_weights, output_weights))
    dropout_mask = c(dropout_mask) if use_mask else None
    L.call("nmtg_self_attn_bwd", L.ptr(g), L.ptr(matmul2_results), L.ptr(dropout_results), L.ptr(attn_scores),
           L.ptr(input_lin_results), L.ptr(inputs), L.ptr(input_weights), L.ptr(output_weights),
           L.ptr(dropout_mask), L.f32(dropout_prob), L.ptr(dx), L.ptr(dw_in), L.ptr(dw_out),
           L.ptr(db_in), L.ptr(db_out), L.ptr(dlin), L.ptr(ws), L.i64(ws.numel()), L.i64(t), L.i64(b), L.i64(e),
           L.i32(heads), L.i32(L.dtype_code(g)), L.stream_of(g))
    return dx, dw_in, dw_out, db_in, db_out, dlin


def backward(use_time_mask, heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_results,
             inputs, input_weights, output_weights, dropout_mask, dropout_prob):
    """-> [input_grads, input_weight_grads, output_weight_grads, input_bias_grads, output_bias_grads]"""
    dx, dw_in, dw_out, db_in, db_out, _ = _bwd(heads, output_grads, matmul2_results, dropout_results, attn_scores,
                                               input_lin_results, inputs, input_weights, output_weights, dropout_mask,
                                               dropout_prob)
    return [dx, dw_in, dw_out, db_in, db_out]


def backward_input_only(use_time_mask, heads, output_grads, matmul2_results, dropout_results, attn_scores,
                        input_lin_results, inputs, input_weights, output_weights, dropout_mask, dropout_prob):
    """-> input_grads"""
    return _bwd(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_results, inputs,
                input_weights, output_weights, dropout_mask, dropout_prob, want_weights=False)[0]


def backward_compact(use_time_mask, heads, output_lin_grads, dropout_results, attn_scores, input_lin_results,
                     dropout_mask, dropout_prob):
    """output_lin_grads: gradient of the context [T, B, E]. -> [input_lin_grads [T, B, 3E]]"""
    return [_bwd(heads, output_lin_grads, None, dropout_results, attn_scores, input_lin_results, None, None, None,
                 dropout_mask, dropout_prob)[5]]


def backward_recompute(use_time_mask, heads, output_grads, inputs, input_weights, output_weights, input_biases,
                       output_biases, pad_mask, dropout_mask, dropout_prob):
    """Re-runs the forward from the inputs and the stored dropout mask, then the backward."""
    training = dropout_mask is not None and dropout_mask.numel() > 0 and dropout_prob > 0.0
    lin, scores, dropped, dmask, ctx, _ = forward(use_time_mask, training, heads, inputs, input_weights, output_weights,
                                                  input_biases, output_biases, pad_mask, dropout_prob,
                                                  dropout_mask=dropout_mask if training else None, need_backward=True)
    return backward(use_time_mask, heads, output_grads, ctx, dropped, scores, lin, inputs, input_weights, output_weights,
                    dmask, dropout_prob)
