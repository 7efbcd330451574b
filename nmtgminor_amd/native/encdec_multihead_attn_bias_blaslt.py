"""Stand-in for the reference module `encdec_multihead_attn_bias_blaslt`
(onmt/modules/extensions/multihead_attn_blaslt/encdec_multihead_attn_bias.cpp:124-475): forward,
backward, forward_compact, backward_compact, backward_recompute; plus backward_input_only of the
older `encdec_multihead_attn_bias_cuda` (multihead_attn/encdec_multihead_attn_bias.cpp:308-310).

Extras: any bias may be None (Whisper's key projection has none); fp16 and bf16; `forward` /
`forward_compact` take an optional keyword `dropout_mask` to replay an explicit keep-mask."""
import os

import torch

from .. import _lib as L
from . import _attn_common as A
from .linear_gemm import gemm

KEY_BLOCK = 64      # the GEMM main loops move whole 64-element steps of the reduction dimension with 16-byte accesses


def _shapes(q3, kv3, heads, kv_last):
    A.check(q3.dim() == 3 and kv3.dim() == 3, "expected 3D tensor")
    tq, b, e = q3.shape
    tk = kv3.shape[0]
    A.check(kv3.shape[1] == b and kv3.shape[2] == e * kv_last and e % heads == 0, "query / key-value shapes do not match")
    return tq, tk, b, e


def _fwd(is_training, heads, x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, q_lin, kv_lin, pad_mask, p, dropout_mask,
         tq, tk, b, e, dev, dt, softmax_out=None, want_probs=True, need_backward=None):
    km, kind = A.mask_arg(pad_mask, False, b, tq, tk)
    bh = b * heads
    if q_lin is None:
        q_lin = torch.empty(tq, b, e, dtype=dt, device=dev)
    if kv_lin is None:
        kv_lin = torch.empty(tk, b, 2 * e, dtype=dt, device=dev)
    keep_scores = softmax_out is not None or A.scores_needed(is_training, dt, e // heads, tk, need_backward)
    scores = torch.empty((bh, tq, tk) if keep_scores else (0,), dtype=dt, device=dev)
    keep_probs = want_probs or keep_scores
    dropped = torch.empty((bh, tq, tk) if keep_probs else (0,), dtype=dt, device=dev)
    ctx = torch.empty(tq, b, e, dtype=dt, device=dev)
    out = torch.empty(tq, b, e, dtype=dt, device=dev) if w_out is not None else None
    dmask, mode, seed, offset = A.dropout_args(is_training, p, (bh, tq, tk), dev, dropout_mask)
    if tq == 0 or b == 0:       # an empty batch / no query position: the (empty) buffers are the result
        return q_lin, kv_lin, scores, dropped, dmask, ctx, out
    L.call("nmtg_encdec_attn_fwd", L.ptr(x_q), L.ptr(x_kv), L.ptr(w_q), L.ptr(w_kv), L.ptr(w_out), L.ptr(b_q), L.ptr(b_kv),
           L.ptr(b_out), L.ptr(km), L.ptr(q_lin), L.ptr(kv_lin), L.ptr(scores if keep_scores else None), L.ptr(softmax_out),
           L.ptr(dropped if keep_probs else None),
           L.ptr(dmask if mode else None), L.i32(mode), L.f32(p), A.u64(seed), A.u64(offset), L.ptr(ctx), L.ptr(out),
           L.i64(tq), L.i64(tk), L.i64(b), L.i64(e), L.i32(heads), L.i32(L.dtype_code(ctx)), L.stream_of(ctx))
    return q_lin, kv_lin, scores, dropped, dmask, ctx, out


def _fwd_padded_keys(heads, x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, pad_mask, tq, tk, b, e):
    """Inference forward for a key length that is not a multiple of 64 (Whisper's 1500 encoder frames): the projected
    keys / values are written into a buffer of tk_pad = ceil(tk / 64) * 64 rows whose extra rows are zero and masked,
    so that the score / probability rows are 16-byte aligned and the per-head products run their fast main loops
    (with tk = 1500 every row of those tensors starts on an 8-byte boundary only, and the products over the keys end
    in a partial step). Masked keys have probability exactly 0, so the results for the real keys are the same numbers;
    the returned key/value projection, scores and probabilities are views of the padded buffers, cut back to tk."""
    dev, dt = x_q.device, x_q.dtype
    tk_pad = (tk + KEY_BLOCK - 1) // KEY_BLOCK * KEY_BLOCK
    kv_lin = torch.empty(tk_pad, b, 2 * e, dtype=dt, device=dev)
    kv_lin[tk:].zero_()
    gemm(x_kv.view(tk * b, e), w_kv, False, True, bias=b_kv, out=kv_lin[:tk].view(tk * b, 2 * e))
    q_lin = gemm(x_q.view(tq * b, e), w_q, False, True, bias=b_q).view(tq, b, e)
    mask = torch.ones(b, tk_pad, dtype=torch.uint8, device=dev)
    if pad_mask is not None and pad_mask.numel() > 0:
        mask[:, :tk] = pad_mask.reshape(b, tk).to(torch.uint8)
    else:
        mask[:, :tk] = 0
    r = _fwd(False, heads, None, None, None, None, None, None, None, None, q_lin, kv_lin, mask, 0.0, None, tq, tk_pad, b, e,
             dev, dt)
    scores, dropped, dmask, ctx = r[2], r[3], r[4], r[5]
    out = gemm(ctx.view(tq * b, e), w_out, False, True, bias=b_out).view(tq, b, e)
    return [q_lin, kv_lin[:tk], scores[:, :, :tk], dropped[:, :, :tk], dmask, ctx, out]


def forward(is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, input_biases_q,
            input_biases_kv, output_biases, pad_mask, dropout_prob, *, dropout_mask=None, want_probs=True,
            need_backward=None):
    """-> [input_lin_q_results, input_lin_kv_results, attn_scores, dropout_results, dropout_mask,
    matmul2_results, outputs]; attn_scores is empty for an inference call under torch.no_grad() (see
    _attn_common.scores_needed), and so is dropout_results when such a call says want_probs=False."""
    tensors = (inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, input_biases_q, input_biases_kv,
               output_biases)
    L.require_cuda(*tensors, pad_mask, dropout_mask)
    A.check_half(*tensors)
    tq, tk, b, e = _shapes(inputs_q, inputs_kv, heads, 1)
    A.check(input_weights_q.shape == (e, e) and input_weights_kv.shape == (2 * e, e) and output_weights.shape == (e, e),
            "weight shapes do not match the inputs")
    c = lambda z: z.contiguous() if z is not None else None
    # inference with a key length that is not a multiple of 64: keys / values padded with masked zero rows, so that every
    # tensor of the middle section is 16-byte aligned
    if (not is_training and tk % KEY_BLOCK != 0
            and A.scores_needed(False, inputs_q.dtype, e // heads, tk, need_backward)):
        return _fwd_padded_keys(heads, c(inputs_q), c(inputs_kv), c(input_weights_q), c(input_weights_kv), c(output_weights),
                                c(input_biases_q), c(input_biases_kv), c(output_biases), pad_mask, tq, tk, b, e)
    return list(_fwd(is_training, heads, c(inputs_q), c(inputs_kv), c(input_weights_q), c(input_weights_kv),
                     c(output_weights), c(input_biases_q), c(input_biases_kv), c(output_biases), None, None, pad_mask,
                     dropout_prob, dropout_mask, tq, tk, b, e, inputs_q.device, inputs_q.dtype, want_probs=want_probs,
                     need_backward=need_backward))


def forward_compact(is_training, heads, input_lin_q_results, input_lin_kv_results, pad_mask, dropout_prob, *,
                    dropout_mask=None, need_backward=None):
    """-> [attn_scores, dropout_results, dropout_mask, matmul2_results]"""
    L.require_cuda(input_lin_q_results, input_lin_kv_results, pad_mask, dropout_mask)
    A.check_half(input_lin_q_results, input_lin_kv_results)
    tq, tk, b, e = _shapes(input_lin_q_results, input_lin_kv_results, heads, 2)
    r = _fwd(is_training, heads, None, None, None, None, None, None, None, None, input_lin_q_results.contiguous(),
             input_lin_kv_results.contiguous(), pad_mask, dropout_prob, dropout_mask, tq, tk, b, e,
             input_lin_q_results.device, input_lin_q_results.dtype, need_backward=need_backward)
    return [r[2], r[3], r[4], r[5]]


def _bwd(heads, output_grads, matmul2_results, dropout_results, attn_scores, q_lin, kv_lin, inputs_q, inputs_kv, w_q, w_kv,
         w_out, dropout_mask, p, want_weights=True, want_biases=True, from_probs=False):
    """from_probs: `attn_scores` holds the softmax results (what the bias-free extension saves); no bias gradients."""
    want_biases = want_biases and not from_probs
    L.require_cuda(output_grads, dropout_results, attn_scores, q_lin, kv_lin, inputs_q, inputs_kv, w_q, w_kv, w_out)
    A.check_half(output_grads, dropout_results, attn_scores, q_lin, kv_lin, inputs_q, inputs_kv, w_q, w_kv, w_out)
    tq, tk, b, e = _shapes(q_lin, kv_lin, heads, 2)
    dev, dt = output_grads.device, output_grads.dtype
    g = output_grads.contiguous()
    use_mask = dropout_mask is not None and dropout_mask.numel() > 0 and p > 0.0
    compact = w_out is None
    n = {k: None for k in ("dxq", "dxkv", "dwq", "dwkv", "dwo", "dbq", "dbkv", "dbo", "dq", "dkv")}
    if compact:
        n["dq"] = torch.empty(tq, b, e, dtype=dt, device=dev)
        n["dkv"] = torch.empty(tk, b, 2 * e, dtype=dt, device=dev)
    else:
        n["dxq"] = torch.empty(tq, b, e, dtype=dt, device=dev)
        n["dxkv"] = torch.empty(tk, b, e, dtype=dt, device=dev)
        if want_weights:
            n["dwq"] = torch.empty(e, e, dtype=dt, device=dev)
            n["dwkv"] = torch.empty(2 * e, e, dtype=dt, device=dev)
            n["dwo"] = torch.empty(e, e, dtype=dt, device=dev)
            if want_biases:
                n["dbq"] = torch.empty(e, dtype=dt, device=dev)
                n["dbkv"] = torch.empty(2 * e, dtype=dt, device=dev)
                n["dbo"] = torch.empty(e, dtype=dt, device=dev)
    if tq == 0 or b == 0:       # an empty batch / no query position contributes zero gradients
        for z in n.values():
            if z is not None:
                z.zero_()
        return n
    ws_bytes = L.load().nmtg_encdec_attn_bwd_workspace_bytes(L.i64(tq), L.i64(tk), L.i64(b), L.i64(e), L.i32(heads))
    ws = A.workspace(ws_bytes, dev)
    # contiguous copies (if any) are bound to names: a temporary would be freed before the kernels read it
    c = lambda z: z.contiguous() if z is not None else None
    (matmul2_results, dropout_results, attn_scores, q_lin, kv_lin, inputs_q, inputs_kv, w_q, w_kv, w_out) = map(
        c, (matmul2_results, dropout_results, attn_scores, q_lin, kv_lin, inputs_q, inputs_kv, w_q, w_kv, w_out))
    dropout_mask = c(dropout_mask) if use_mask else None
    if from_probs:
        L.call("nmtg_encdec_attn_bwd_from_probs", L.ptr(g), L.ptr(matmul2_results), L.ptr(dropout_results), L.ptr(attn_scores),
               L.ptr(q_lin), L.ptr(kv_lin), L.ptr(inputs_q), L.ptr(inputs_kv), L.ptr(w_q), L.ptr(w_kv),
               L.ptr(w_out), L.ptr(dropout_mask), L.f32(p), L.ptr(n["dxq"]), L.ptr(n["dxkv"]),
               L.ptr(n["dwq"]), L.ptr(n["dwkv"]), L.ptr(n["dwo"]), L.ptr(n["dq"]), L.ptr(n["dkv"]), L.ptr(ws), L.i64(ws.numel()),
               L.i64(tq), L.i64(tk), L.i64(b), L.i64(e), L.i32(heads), L.i32(L.dtype_code(g)), L.stream_of(g))
        return n
    L.call("nmtg_encdec_attn_bwd", L.ptr(g), L.ptr(matmul2_results), L.ptr(dropout_results), L.ptr(attn_scores),
           L.ptr(q_lin), L.ptr(kv_lin), L.ptr(inputs_q), L.ptr(inputs_kv), L.ptr(w_q), L.ptr(w_kv),
           L.ptr(w_out), L.ptr(dropout_mask), L.f32(p), L.ptr(n["dxq"]), L.ptr(n["dxkv"]),
           L.ptr(n["dwq"]), L.ptr(n["dwkv"]), L.ptr(n["dwo"]), L.ptr(n["dbq"]), L.ptr(n["dbkv"]), L.ptr(n["dbo"]),
           L.ptr(n["dq"]), L.ptr(n["dkv"]), L.ptr(ws), L.i64(ws.numel()), L.i64(tq), L.i64(tk), L.i64(b), L.i64(e),
           L.i32(heads), L.i32(L.dtype_code(g)), L.stream_of(g))
    return n


def backward(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_q_results,
             input_lin_kv_results, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, dropout_mask,
             dropout_prob):
    """-> [input_q_grads, input_kv_grads, input_weight_q_grads, input_weight_kv_grads,
    output_weight_grads, input_bias_q_grads, input_bias_kv_grads, output_bias_grads]"""
    n = _bwd(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_q_results, input_lin_kv_results,
             inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, dropout_mask, dropout_prob)
    return [n[k] for k in ("dxq", "dxkv", "dwq", "dwkv", "dwo", "dbq", "dbkv", "dbo")]


def backward_input_only(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_q_results,
                        input_lin_kv_results, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights,
                        dropout_mask, dropout_prob):
    """-> [input_q_grads, input_kv_grads]"""
    n = _bwd(heads, output_grads, matmul2_results, dropout_results, attn_scores, input_lin_q_results, input_lin_kv_results,
             inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, dropout_mask, dropout_prob,
             want_weights=False)
    return [n["dxq"], n["dxkv"]]


def backward_compact(heads, output_lin_grads, dropout_results, attn_scores, input_lin_q_results, input_lin_kv_results,
                     dropout_mask, dropout_prob):
    """-> [input_lin_q_grads, input_lin_kv_grads]"""
    n = _bwd(heads, output_lin_grads, None, dropout_results, attn_scores, input_lin_q_results, input_lin_kv_results, None,
             None, None, None, None, dropout_mask, dropout_prob)
    return [n["dq"], n["dkv"]]


def backward_recompute(heads, output_grads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, input_biases_q,
                       input_biases_kv, output_weights, dropout_mask, pad_mask, dropout_prob):
    """Re-runs the forward from the inputs and the stored dropout mask, then the backward. The
    output bias does not enter any gradient, so it is not an argument (as in the reference)."""
    training = dropout_mask is not None and dropout_mask.numel() > 0 and dropout_prob > 0.0
    q_lin, kv_lin, scores, dropped, dmask, ctx, _ = forward(training, heads, inputs_q, inputs_kv, input_weights_q,
                                                            input_weights_kv, output_weights, input_biases_q,
                                                            input_biases_kv, None, pad_mask, dropout_prob,
                                                            dropout_mask=dropout_mask if training else None,
                                                            need_backward=True)
    return backward(heads, output_grads, ctx, dropped, scores, q_lin, kv_lin, inputs_q, inputs_kv, input_weights_q,
                    input_weights_kv, output_weights, dmask, dropout_prob)
