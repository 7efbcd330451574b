"""Thin Python face of the elementwise kernels of self-attention with relative position encodings: the additions of
r_w_bias / r_r_bias to the queries, RelativeShift.forward fused with the sum of the two score terms, and
RelativeShift.backward (onmt/modules/optimized/relative_self_attention_func.py:26-76, :210-217, :246-253, :621-630); and
of the two kernels that run the shift inside the softmax + dropout pass and its adjoint inside that pass's backward."""
import ctypes
import os

import torch

from .. import _lib as L
from .._rng import philox_seed_offset


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def query_bias(queries, r_w_bias, r_r_bias, heads):
    """queries [len_q, batch*heads, head_dim], a view into the in-projection output (innermost stride 1, one uniform
    pitch from head row to head row); r_w_bias, r_r_bias [heads, head_dim]. -> (queries + r_w_bias, queries + r_r_bias),
    dense [len_q, batch*heads, head_dim]."""
    L.require_cuda(queries, r_w_bias, r_r_bias)
    _check(queries.dim() == 3 and queries.stride(2) == 1, "query_bias: queries must be [len_q, batch*heads, head_dim] with unit stride")
    t, bh, d = queries.shape
    ld = queries.stride(1)
    _check(t <= 1 or queries.stride(0) == bh * ld, "query_bias: rows of the queries must have one uniform pitch")
    _check(bh % heads == 0 and r_w_bias.numel() == heads * d and r_r_bias.numel() == heads * d,
           "query_bias: biases must be [heads, head_dim]")
    _check(r_w_bias.dtype == queries.dtype and r_r_bias.dtype == queries.dtype, "query_bias: dtypes differ")
    r_w_bias, r_r_bias = r_w_bias.contiguous(), r_r_bias.contiguous()
    rw = torch.empty(t, bh, d, dtype=queries.dtype, device=queries.device)
    rr = torch.empty_like(rw)
    L.call("nmtg_rel_query_bias", L.ptr(queries), L.i64(ld), L.ptr(r_w_bias), L.ptr(r_r_bias), L.ptr(rw), L.ptr(rr),
           L.i64(t * bh), L.i64(heads), L.i64(d), L.i32(L.dtype_code(queries)), L.stream_of(queries))
    return rw, rr


def shift_add_(scores, bd):
    """scores [batch, len_q, len_k] += RelativeShift.forward(bd)[:, :, :len_k] in place; bd [batch, len_q, len_r]."""
    L.require_cuda(scores, bd)
    _check(scores.dim() == 3 and bd.dim() == 3 and scores.is_contiguous() and bd.is_contiguous(),
           "shift_add: contiguous [batch, len_q, len_k] and [batch, len_q, len_r] tensors required")
    _check(scores.shape[:2] == bd.shape[:2] and scores.dtype == bd.dtype, "shift_add: shapes or dtypes differ")
    b, tq, tk = scores.shape
    L.call("nmtg_rel_shift_add", L.ptr(scores), L.ptr(bd), L.i64(b), L.i64(tq), L.i64(tk), L.i64(bd.shape[2]),
           L.i32(L.dtype_code(scores)), L.stream_of(scores))
    return scores


def shift_backward(grad_scores, len_r):
    """Gradient wrt bd [batch, len_q, len_r] of shift(bd)[:, :, :len_k], from grad_scores [batch, len_q, len_k]."""
    L.require_cuda(grad_scores)
    _check(grad_scores.dim() == 3, "shift_backward: [batch, len_q, len_k] gradient required")
    grad_scores = grad_scores.contiguous()
    b, tq, tk = grad_scores.shape
    out = torch.empty(b, tq, len_r, dtype=grad_scores.dtype, device=grad_scores.device)
    L.call("nmtg_rel_shift_bwd", L.ptr(grad_scores), L.ptr(out), L.i64(b), L.i64(tq), L.i64(tk), L.i64(len_r),
           L.i32(L.dtype_code(grad_scores)), L.stream_of(grad_scores))
    return out


def fused_ok(scores_shape, dtype, len_r):
    """Whether the softmax kernels can take the shift along (rel_softmax_dropout_*): rows of a multiple of 16 bytes, at
    most 4096 keys (2048 in fp32), 32-bit indices inside the kernel; NMTG_REL_FUSED=0 switches the route off."""
    if os.environ.get("NMTG_REL_FUSED", "1") == "0":
        return False
    b, tq, tk = scores_shape
    wide = 4 if dtype == torch.float32 else 8
    return (b > 0 and tq > 0 and tk > 0 and tk % wide == 0 and tk <= 512 * wide and len_r >= tk
            and tq * (len_r + 1) < 2 ** 31 and b * tq < 2 ** 31)


def shift_add_softmax_dropout(scores, bd, is_training, heads, dropout_prob, mask, mask_kind, dropout_mask=None):
    """scores [batch, len_q, len_k] (content term; replaced by the sum with the shifted position term bd
    [batch, len_q, len_r]) -> (dropout_mask, dropped probabilities). One pass instead of shift_add_ followed by the
    softmax; mask / mask_kind as the softmax kernels take them (uint8, 1 = pad mask [batch/heads, len_k], 2 = time mask)."""
    L.require_cuda(scores, bd, mask, dropout_mask)
    _check(scores.dim() == 3 and bd.dim() == 3 and scores.is_contiguous() and bd.is_contiguous()
           and scores.shape[:2] == bd.shape[:2] and scores.dtype == bd.dtype,
           "shift_add_softmax_dropout: contiguous [batch, len_q, len_k] and [batch, len_q, len_r] tensors of one dtype required")
    b, tq, tk = scores.shape
    dropped = torch.empty_like(scores)
    if is_training and dropout_prob > 0.0:
        if dropout_mask is not None:
            _check(dropout_mask.dtype == torch.uint8 and dropout_mask.numel() == scores.numel(), "shift_add_softmax_dropout: bad dropout mask")
            dropout_mask, mode, seed, offset = dropout_mask.contiguous(), 1, 0, 0
        else:
            dropout_mask, mode = torch.empty(scores.shape, dtype=torch.uint8, device=scores.device), 2
            seed, offset = philox_seed_offset(scores.device, scores.numel())
    else:
        mode, seed, offset = 0, 0, 0
        dropout_mask = torch.empty(0, dtype=torch.uint8, device=scores.device)
    L.call("nmtg_rel_softmax_dropout_fwd", L.ptr(scores), L.ptr(bd), L.i64(bd.shape[2]), L.ptr(mask), L.i32(mask_kind),
           L.ptr(dropped), L.ptr(dropout_mask if mode else None), L.i32(mode), L.f32(dropout_prob), ctypes.c_uint64(seed),
           ctypes.c_uint64(offset), L.i64(b), L.i64(tq), L.i64(tk), L.i64(heads), L.i32(L.dtype_code(scores)),
           L.stream_of(scores))
    return dropout_mask, dropped


def softmax_dropout_shift_backward(grad_dropped, scores, len_r, heads, dropout_mask, dropout_prob, mask, mask_kind, *,
                                   grad_bd=None):
    """-> (grad wrt the summed scores [batch, len_q, len_k], its shift adjoint [batch, len_q, len_r]) from the gradient of
    the dropped probabilities and the saved summed scores, in one pass. `grad_bd`: a buffer to write the adjoint to."""
    L.require_cuda(grad_dropped, scores, dropout_mask, mask)
    grad_dropped = grad_dropped.contiguous()
    _check(scores.is_contiguous() and scores.shape == grad_dropped.shape and scores.dtype == grad_dropped.dtype,
           "softmax_dropout_shift_backward: saved scores must match the gradient")
    b, tq, tk = scores.shape
    use_mask = dropout_mask is not None and dropout_mask.numel() > 0 and dropout_prob > 0.0
    if use_mask:
        _check(dropout_mask.dtype == torch.uint8 and dropout_mask.numel() == scores.numel(), "softmax_dropout_shift_backward: bad dropout mask")
        dropout_mask = dropout_mask.contiguous()
    grad_scores = torch.empty_like(scores)
    if grad_bd is None:
        grad_bd = torch.empty(b, tq, len_r, dtype=scores.dtype, device=scores.device)
    _check(grad_bd.shape == (b, tq, len_r) and grad_bd.dtype == scores.dtype and grad_bd.is_contiguous(),
           "softmax_dropout_shift_backward: grad_bd must be a contiguous [batch, len_q, len_r] tensor of the scores' dtype")
    L.require_cuda(grad_bd)
    L.call("nmtg_rel_softmax_dropout_bwd", L.ptr(grad_dropped), L.ptr(scores), L.ptr(mask), L.i32(mask_kind),
           L.ptr(dropout_mask if use_mask else None), L.i32(1 if use_mask else 0), L.f32(dropout_prob), L.ptr(grad_scores),
           L.ptr(grad_bd), L.i64(len_r), L.i64(b), L.i64(tq), L.i64(tk), L.i64(heads), L.i32(L.dtype_code(scores)),
           L.stream_of(scores))
    return grad_scores, grad_bd


def _rows_view(t, what):
    """(pointer tensor, rows, cols, pitch) of a tensor whose elements form rows of `cols` contiguous elements at one
    uniform pitch (a dense tensor, or a slice of the last-but-one dimension such as the queries inside the in-projection
    output)."""
    _check(t.dim() >= 2 and t.stride(-1) == 1, what + ": innermost stride must be 1")
    cols, ld = t.size(-1), t.stride(-2)
    rows = t.numel() // max(cols, 1)
    expect = ld
    for dim in range(t.dim() - 2, -1, -1):
        _check(t.size(dim) == 1 or t.stride(dim) == expect, what + ": rows must have one uniform pitch")
        expect *= t.size(dim)
    return rows, cols, ld


def add_rows(a, b, out=None):
    """out = a + b elementwise; the three tensors have equal shapes and each is a set of equally pitched rows (see
    _rows_view). out defaults to a new dense tensor and may be a or b."""
    L.require_cuda(a, b, out)
    if out is None:
        out = torch.empty(a.shape, dtype=a.dtype, device=a.device)
    _check(a.shape == b.shape == out.shape and a.dtype == b.dtype == out.dtype, "add_rows: shapes or dtypes differ")
    if a.numel() == 0:
        return out
    rows, cols, ld_a = _rows_view(a, "add_rows")
    _, _, ld_b = _rows_view(b, "add_rows")
    _, _, ld_o = _rows_view(out, "add_rows")
    L.call("nmtg_add_rows", L.ptr(out), L.i64(ld_o), L.ptr(a), L.i64(ld_a), L.ptr(b), L.i64(ld_b), L.i64(rows), L.i64(cols),
           L.i32(L.dtype_code(a)), L.stream_of(a))
    return out
