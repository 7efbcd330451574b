"""Stand-in for the reference module `xentropy_cuda`
(onmt/modules/extensions/xentropy/interface.cpp:24-61): forward, backward, __version__.

The logits may be a row-pitched view (stride(1) == 1, stride(0) >= classes), which is read in place; any other
layout is made contiguous first, as the reference does. `backward` takes an optional `out` of that kind.

Both functions take one optional extra keyword, `padding_idx`: rows whose label equals it get a
zero loss / zero gradient inside the kernel (the reference's Python wrapper does this afterwards
with masked_fill_). Left at None the behaviour is the reference module's."""
import torch

from .. import _lib as L

__version__ = "0.1"

_NO_PAD = -(1 << 63)


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _rows(t):
    """A 2-D tensor the kernels can read row by row: itself if its rows are dense, else a contiguous copy."""
    if t.dim() == 2 and t.size(0) > 0 and t.size(1) > 0 and t.stride(1) == 1 and t.stride(0) >= t.size(1):
        return t
    return t.contiguous()


def forward(logits, labels, smoothing, half_to_float=False, *, padding_idx=None, want_argmax=False):
    """-> [losses fp32 [N], max_log_sum_exp [N] (fp32 if half_to_float or fp32 logits)]; with want_argmax a third
    entry, int64 [N]: the index of each row's largest logit by torch.argmax's rule, from the same pass over the row."""
    L.require_cuda(logits, labels)
    if half_to_float:
        _check(logits.dtype in (torch.float16, torch.bfloat16), "conversion is supported for Half type only")
    _check(labels.dtype == torch.int64, "Label type should be CUDA Long")
    _check(logits.dim() == 2, "Currently only 2 dim input supported")
    _check(labels.dim() == 1, "Labels should be 1 dimensional")
    _check(logits.size(0) == labels.size(0), "Input and label should have same number of examples")
    _check(logits.numel() > 0, "Number of classes in input should not be 0")
    logits = _rows(logits)
    labels = labels.contiguous()
    n, v = logits.shape
    losses = torch.empty(n, dtype=torch.float32, device=logits.device)
    lse = torch.empty(n, dtype=torch.float32, device=logits.device)
    pad = L.i64(_NO_PAD if padding_idx is None else padding_idx)
    best = None
    if want_argmax:
        best = torch.empty(n, dtype=torch.int64, device=logits.device)
        L.call("nmtg_xentropy_fwd_argmax", L.ptr(logits), L.ptr(labels), L.ptr(losses), L.ptr(lse), L.ptr(best), L.i64(n), L.i64(v),
               L.i64(logits.stride(0)), L.f32(smoothing), pad, L.i32(L.dtype_code(logits)), L.stream_of(logits))
    else:
        L.call("nmtg_xentropy_fwd", L.ptr(logits), L.ptr(labels), L.ptr(losses), L.ptr(lse), L.i64(n), L.i64(v),
               L.i64(logits.stride(0)), L.f32(smoothing), pad, L.i32(L.dtype_code(logits)), L.stream_of(logits))
    if not half_to_float and logits.dtype != torch.float32:
        lse = lse.to(logits.dtype)
    return [losses, lse, best] if want_argmax else [losses, lse]


def backward(grad_loss, logits, max_log_sum_exp, labels, smoothing, *, padding_idx=None, out=None, class_offset=0,
             total_classes=None):
    """-> grad_logits (logits dtype and shape); written into `out` when given. With `class_offset` / `total_classes`
    the columns of `logits` are the slice [class_offset, class_offset + logits.size(1)) of that many classes (the
    backward is elementwise given the log-sum-exp of the whole row); labels stay global."""
    L.require_cuda(grad_loss, logits, max_log_sum_exp, labels)
    _check(labels.dtype == torch.int64, "Label type should be CUDA Long")
    _check(logits.dim() == 2 and labels.dim() == 1 and logits.size(0) == labels.size(0), "shape mismatch")
    _check(grad_loss.numel() == labels.numel() and max_log_sum_exp.numel() == labels.numel(), "shape mismatch")
    _check(logits.numel() > 0, "Number of classes in input should not be 0")      # as the reference (xentropy_kernel.cu:659)
    logits = _rows(logits)
    grad_loss = grad_loss.contiguous().float()
    lse = max_log_sum_exp.contiguous().float()
    n, v = logits.shape
    if out is None:
        grad_logits = torch.empty(n, v, dtype=logits.dtype, device=logits.device)
    else:
        L.require_cuda(out)
        _check(out.shape == logits.shape and out.dtype == logits.dtype and out.stride(1) == 1 and out.stride(0) >= v,
               "out must have the shape and dtype of the logits and dense rows")
        grad_logits = out
    labels = labels.contiguous()                          # bound to a name: a temporary would be freed before the kernel reads it
    L.call("nmtg_xentropy_bwd", L.ptr(grad_loss), L.ptr(logits), L.ptr(lse), L.ptr(labels),
           L.ptr(grad_logits), L.i64(n), L.i64(v), L.i64(logits.stride(0)), L.i64(grad_logits.stride(0)),
           L.i64(class_offset), L.i64(v if total_classes is None else total_classes), L.f32(smoothing),
           L.i64(_NO_PAD if padding_idx is None else padding_idx), L.i32(L.dtype_code(logits)), L.stream_of(logits))
    return grad_logits
