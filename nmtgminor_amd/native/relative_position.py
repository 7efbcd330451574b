"""Thin Python face of the elementwise kernels of self-attention with relative position encodings: the additions of
r_w_bias / r_r_bias to the queries, RelativeShift.forward fused with the sum of the two score terms, and
RelativeShift.backward (onmt/modules/optimized/relative_self_attention_func.py:26-76, :210-217, :246-253, :621-630)."""
import torch

from .. import _lib as L


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
