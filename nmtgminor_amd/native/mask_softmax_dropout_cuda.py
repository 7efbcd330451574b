"""Stand-in for the module `mask_softmax_dropout_cuda` that the reference's
AttentionSoftmaxDropout calls (onmt/modules/optimized/attention_softmax.py:32-33,58-59;
test/test_softmax.py:16-36). Its source is not in the reference tree; the signatures follow
those call sites: forward(is_training, heads, inputs, p) -> (dropout_mask, softmax, dropped);
backward(heads, grad, softmax, mask, p); backward_recompute(heads, grad, softmax, inputs, mask, p).

Extras (keyword only): `pad_mask` [batch, len_k] or `time_mask` [len_q, len_k] fused into the
softmax, and `dropout_mask` to replay an explicit keep-mask instead of drawing one."""
import ctypes

import torch

from .. import _lib as L
from .._rng import philox_seed_offset


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _mask_args(pad_mask, time_mask, inputs):
    if pad_mask is not None and time_mask is not None:
        raise RuntimeError("softmax: give a key-padding mask or a time mask, not both")
    len_q, len_k = inputs.shape[-2], inputs.shape[-1]
    if pad_mask is not None:
        m = pad_mask.reshape(-1, len_k).to(torch.uint8).contiguous()
        return m, 1
    if time_mask is not None:
        _check(time_mask.shape == (len_q, len_k), "softmax: time mask must be [len_q, len_k]")
        return time_mask.to(torch.uint8).contiguous(), 2
    return None, 0


def forward(is_training, heads, inputs, dropout_prob, *, pad_mask=None, time_mask=None, dropout_mask=None,
            want_softmax=True):
    """inputs [batch*heads, len_q, len_k] scores. -> (dropout_mask, softmax_results, dropout_results)."""
    L.require_cuda(inputs, pad_mask, time_mask, dropout_mask)
    _check(inputs.dim() == 3 and inputs.is_contiguous(), "softmax: inputs must be a contiguous [B*H, Tq, Tk] tensor")
    bh, len_q, len_k = inputs.shape
    km, kind = _mask_args(pad_mask, time_mask, inputs)
    if kind == 1:
        _check(km.shape[0] * heads == bh, "softmax: pad mask batch does not match inputs")
    rows = bh * len_q
    dropped = torch.empty_like(inputs)
    if is_training and dropout_prob > 0.0:
        softmax = torch.empty_like(inputs) if want_softmax else None
        if dropout_mask is not None:
            _check(dropout_mask.dtype == torch.uint8 and dropout_mask.numel() == inputs.numel(), "softmax: bad dropout mask")
            dropout_mask = dropout_mask.contiguous()
            mode, seed, offset = 1, 0, 0
        else:
            dropout_mask = torch.empty(inputs.shape, dtype=torch.uint8, device=inputs.device)
            mode = 2
            seed, offset = philox_seed_offset(inputs.device, inputs.numel())
    else:
        softmax, mode, seed, offset = None, 0, 0, 0
        dropout_mask = torch.empty(0, dtype=torch.uint8, device=inputs.device)
    L.call("nmtg_softmax_dropout_fwd", L.ptr(inputs), L.ptr(km), L.i32(kind), L.ptr(softmax), L.ptr(dropped),
           L.ptr(dropout_mask if mode else None), L.i32(mode), L.f32(dropout_prob), ctypes.c_uint64(seed),
           ctypes.c_uint64(offset), L.i64(rows), L.i64(len_k), L.i64(len_q), L.i64(heads), L.i32(L.dtype_code(inputs)),
           L.stream_of(inputs))
    if softmax is None:
        softmax = dropped
    return dropout_mask, softmax, dropped


def _bwd(grad, saved, saved_is_scores, heads, dropout_mask, dropout_prob, pad_mask, time_mask):
    L.require_cuda(grad, saved, dropout_mask, pad_mask, time_mask)
    grad = grad.contiguous()
    _check(saved.is_contiguous() and saved.shape == grad.shape and saved.dtype == grad.dtype,
           "softmax backward: saved tensor must match the gradient")
    bh, len_q, len_k = grad.shape
    km, kind = _mask_args(pad_mask, time_mask, grad) if saved_is_scores else (None, 0)
    use_mask = dropout_mask is not None and dropout_mask.numel() > 0 and dropout_prob > 0.0
    if use_mask:
        _check(dropout_mask.dtype == torch.uint8 and dropout_mask.numel() == grad.numel(), "softmax backward: bad dropout mask")
        dropout_mask = dropout_mask.contiguous()
    out = torch.empty_like(grad)
    L.call("nmtg_softmax_dropout_bwd", L.ptr(grad), L.ptr(saved), L.i32(1 if saved_is_scores else 0), L.ptr(km),
           L.i32(kind), L.ptr(dropout_mask if use_mask else None), L.i32(1 if use_mask else 0), L.f32(dropout_prob),
           L.ptr(out), L.i64(bh * len_q), L.i64(len_k), L.i64(len_q), L.i64(heads), L.i32(L.dtype_code(grad)),
           L.stream_of(grad))
    return out


def backward(heads, grad_outputs, softmax_results, dropout_mask, dropout_prob):
    """Gradient wrt the scores from the saved probabilities."""
    return _bwd(grad_outputs, softmax_results, False, heads, dropout_mask, dropout_prob, None, None)


def backward_recompute(heads, grad_outputs, softmax_results, inputs, dropout_mask, dropout_prob, *, pad_mask=None,
                       time_mask=None):
    """Gradient wrt the scores, recomputing the probabilities from the saved scores `inputs`
    (`softmax_results` is accepted for signature compatibility and not read)."""
    return _bwd(grad_outputs, inputs, True, heads, dropout_mask, dropout_prob, pad_mask, time_mask)
