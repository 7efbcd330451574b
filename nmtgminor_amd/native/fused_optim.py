"""Stand-in for the reference's extension module `fused_optim` (onmt/modules/extensions/fused_optim/frontend.cpp:45-53):
multi_tensor_adam, multi_tensor_scale, multi_tensor_axpby, multi_tensor_l2norm and multi_tensor_l2norm_scale with the
reference's argument lists (chunk_size, noop_flag, tensor_lists, ...). `chunk_size` is accepted and not used: the kernels
work in chunks of 32768 elements."""
import ctypes

import torch

from .. import _lib as L


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _lists(tensor_lists, depth, what):
    _check(len(tensor_lists) == depth, "%s: expected %d tensor lists, got %d" % (what, depth, len(tensor_lists)))
    n = len(tensor_lists[0])
    for lst in tensor_lists:
        _check(len(lst) == n, what + ": tensor lists differ in length")
    for group in zip(*tensor_lists):
        for t in group:
            _check(t.is_contiguous() and t.numel() == group[0].numel(), what + ": tensors must be contiguous and of equal size across the lists")
    for lst in tensor_lists:
        _check(all(t.dtype == lst[0].dtype for t in lst), what + ": one dtype per list")
    L.require_cuda(*[t for lst in tensor_lists for t in lst])
    return n


def _ptr_array(tensors):
    return (ctypes.c_void_p * max(1, len(tensors)))(*[t.data_ptr() if t.numel() else None for t in tensors])


def _size_array(tensors):
    return (ctypes.c_int64 * max(1, len(tensors)))(*[t.numel() for t in tensors])


def multi_tensor_adam(chunk_size, noop_flag, tensor_lists, lr, beta1, beta2, epsilon, step, mode, bias_correction,
                      weight_decay):
    """tensor_lists = [grads, params, exp_avg, exp_avg_sq]; params and both moments are updated in place."""
    n = _lists(tensor_lists, 4, "multi_tensor_adam")
    if n == 0:
        return
    g, p, m, v = tensor_lists
    _check(g[0].dtype == p[0].dtype == m[0].dtype == v[0].dtype, "multi_tensor_adam: the four lists must share one dtype")
    L.call("nmtg_multi_tensor_adam", L.i32(n), _ptr_array(g), _ptr_array(p), _ptr_array(m), _ptr_array(v), _size_array(p),
           L.f32(lr), L.f32(beta1), L.f32(beta2), L.f32(epsilon), L.i32(step), L.i32(mode), L.i32(bias_correction),
           L.f32(weight_decay), L.i32(L.dtype_code(p[0])), L.stream_of(p[0]))


def multi_tensor_scale(chunk_size, noop_flag, tensor_lists, scale):
    """tensor_lists = [inputs, outputs]: out = in * scale; noop_flag (int32 device tensor) becomes 1 if an input element is
    inf or NaN."""
    n = _lists(tensor_lists, 2, "multi_tensor_scale")
    if n == 0:
        return
    src, dst = tensor_lists
    _check(noop_flag is None or (noop_flag.dtype == torch.int32 and noop_flag.numel() >= 1), "multi_tensor_scale: noop_flag must be an int32 tensor")
    L.require_cuda(noop_flag)
    L.call("nmtg_multi_tensor_scale", L.i32(n), _ptr_array(src), _ptr_array(dst), _size_array(src), L.f32(scale), L.ptr(noop_flag),
           L.i32(L.dtype_code(src[0])), L.i32(L.dtype_code(dst[0])), L.stream_of(src[0]))


def multi_tensor_l2norm(chunk_size, noop_flag, tensor_lists, per_tensor=False):
    """tensor_lists = [tensors] -> (norm over all of them, fp32 [1]; per-tensor norms, fp32 [n], or an empty tensor)."""
    n = _lists(tensor_lists, 1, "multi_tensor_l2norm")
    xs = tensor_lists[0]
    dev = xs[0].device if n else (noop_flag.device if noop_flag is not None else torch.device("cuda"))
    norm = torch.empty(1, dtype=torch.float32, device=dev)
    each = torch.empty(n if per_tensor else 0, dtype=torch.float32, device=dev)
    if n == 0:
        return norm.zero_(), each
    sizes = _size_array(xs)
    ws_bytes = int(L.load().nmtg_multi_tensor_l2norm_workspace_bytes(L.i32(n), sizes))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    L.call("nmtg_multi_tensor_l2norm", L.i32(n), _ptr_array(xs), sizes, L.ptr(norm), L.ptr(each if per_tensor else None), L.ptr(ws),
           L.i64(ws_bytes), L.i32(L.dtype_code(xs[0])), L.stream_of(xs[0]))
    return norm, each


def multi_tensor_axpby(chunk_size, noop_flag, tensor_lists, a, b, arg_to_check):
    """tensor_lists = [x, y, out]: out = a x + b y (y and out of one dtype); noop_flag becomes 1 if the checked operand
    (arg_to_check 0: x, 1: y, -1: both) holds an inf or NaN."""
    n = _lists(tensor_lists, 3, "multi_tensor_axpby")
    if n == 0:
        return
    x, y, out = tensor_lists
    _check(y[0].dtype == out[0].dtype, "multi_tensor_axpby: y and out must share one dtype")
    _check(noop_flag is None or (noop_flag.dtype == torch.int32 and noop_flag.numel() >= 1), "multi_tensor_axpby: noop_flag must be an int32 tensor")
    L.require_cuda(noop_flag)
    L.call("nmtg_multi_tensor_axpby", L.i32(n), _ptr_array(x), _ptr_array(y), _ptr_array(out), _size_array(x), L.f32(a), L.f32(b),
           L.i32(arg_to_check), L.ptr(noop_flag), L.i32(L.dtype_code(x[0])), L.i32(L.dtype_code(out[0])), L.stream_of(x[0]))


def multi_tensor_l2norm_scale(chunk_size, noop_flag, tensor_lists, scale, per_tensor=False):
    """tensor_lists = [inputs, outputs]: out = in * scale, and -> (norm of all inputs before scaling, fp32 [1]; per-tensor
    norms, fp32 [n], or an empty tensor), in one pass over the inputs."""
    n = _lists(tensor_lists, 2, "multi_tensor_l2norm_scale")
    src, dst = tensor_lists
    dev = src[0].device if n else (noop_flag.device if noop_flag is not None else torch.device("cuda"))
    norm = torch.empty(1, dtype=torch.float32, device=dev)
    each = torch.empty(n if per_tensor else 0, dtype=torch.float32, device=dev)
    if n == 0:
        return norm.zero_(), each
    sizes = _size_array(src)
    ws_bytes = int(L.load().nmtg_multi_tensor_l2norm_workspace_bytes(L.i32(n), sizes))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    L.call("nmtg_multi_tensor_l2norm_scale", L.i32(n), _ptr_array(src), _ptr_array(dst), sizes, L.f32(scale), L.ptr(norm),
           L.ptr(each if per_tensor else None), L.ptr(ws), L.i64(ws_bytes), L.i32(L.dtype_code(src[0])), L.i32(L.dtype_code(dst[0])),
           L.stream_of(src[0]))
    return norm, each
