"""Shared implementation of the fused-MLP stand-in modules (fused_mlp_gelu, fused_mlp_relu, ...).

Argument convention of the reference's native modules (onmt/modules/extensions/mlp/mlp_gelu.cpp:69-264):
`inputs` is the flat list [x, W_1..W_n, b_1..b_n]; forward returns
[out, reserved_space (dropped activations), reserved_activations (pre-activations), reserved_mask];
backward returns [dx, dW_1..dW_n, db_1..db_n]."""
import ctypes

import torch

from .. import _lib as L
from .._rng import philox_seed_offset


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _split_inputs(inputs):
    inputs = list(inputs)
    n = (len(inputs) - 1) // 2
    _check(n >= 1 and len(inputs) == 2 * n + 1, "mlp: inputs must be [x, W_1..W_n, b_1..b_n]")
    return inputs[0], inputs[1:1 + n], inputs[1 + n:]


def _ptr_array(tensors):
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr() if t is not None else None
    return arr


def _validate(x, weights, biases):
    L.require_cuda(x, *weights, *biases)
    _check(x.dtype in (torch.float16, torch.bfloat16, torch.float32),
           "mlp: fp32, fp16 and bf16 are supported (there is no fp64 kernel)")
    in_f = x.shape[-1]
    for w, b in zip(weights, biases):
        _check(w.dtype == x.dtype and w.dim() == 2 and w.shape[1] == in_f, "mlp: weight shape / dtype mismatch")
        _check(b is None or (b.dtype == x.dtype and b.numel() == w.shape[0]), "mlp: bias shape / dtype mismatch")
        in_f = w.shape[0]


def forward(act, p, inputs, mask=None, save_pre=True):
    x, weights, biases = _split_inputs(inputs)
    _validate(x, weights, biases)
    x2 = x.contiguous().view(-1, x.shape[-1])
    weights = [w.contiguous() for w in weights]
    biases = [b.contiguous() if b is not None else None for b in biases]
    batch, in_f = x2.shape
    n = len(weights)
    outs = [w.shape[0] for w in weights]
    hidden = sum(outs[:-1]) * batch
    dev = x.device
    out = torch.empty(*x.shape[:-1], outs[-1], dtype=x.dtype, device=dev)
    post = torch.empty(hidden, dtype=x.dtype, device=dev)
    pre = torch.empty(hidden if save_pre else 0, dtype=x.dtype, device=dev)
    seed = offset = 0
    if p > 0.0:
        if mask is not None:
            _check(mask.dtype == torch.uint8 and mask.numel() == hidden, "mlp: mask must be uint8 with one byte per hidden activation")
            mask = mask.contiguous().view(-1)
            mode = 1
        else:
            mask = torch.empty(hidden, dtype=torch.uint8, device=dev)
            mode = 2
            seed, offset = philox_seed_offset(dev, hidden)
    else:
        mask = torch.empty(0, dtype=torch.uint8, device=dev)
        mode = 0
    if batch == 0:          # nothing to compute (an empty shard): the buffers above are already the result
        return out, post, pre, mask
    of = (ctypes.c_int64 * n)(*outs)
    L.call("nmtg_mlp_fwd", L.i32(n), L.ptr(x2), _ptr_array(weights), _ptr_array(biases), of, L.i64(batch), L.i64(in_f),
           L.ptr(out), L.ptr(post if hidden else None), L.ptr(pre if (save_pre and hidden) else None),
           L.ptr(mask if mode else None), L.i32(mode), L.f32(p), ctypes.c_uint64(seed), ctypes.c_uint64(offset),
           L.i32(L.ACT_CODES[act]), L.i32(L.dtype_code(x)), L.stream_of(x))
    return out, post, pre, mask


def backward(act, p, grad_o, post, pre, mask, inputs, input_only=False, need_dx=None):
    x, weights, biases = _split_inputs(inputs)
    _validate(x, weights, biases)
    x2 = x.contiguous().view(-1, x.shape[-1])
    weights = [w.contiguous() for w in weights]
    batch, in_f = x2.shape
    n = len(weights)
    outs = [w.shape[0] for w in weights]
    dev = x.device
    g2 = grad_o.contiguous().view(-1, outs[-1])
    _check(g2.dtype == x.dtype and g2.shape[0] == batch, "mlp backward: grad_out shape / dtype mismatch")
    if need_dx is None:
        need_dx = x.requires_grad or input_only
    dx = torch.empty_like(x2) if need_dx else None
    if input_only:
        dws, dbs = [None] * n, [None] * n
    else:
        dws = [torch.empty_like(w) for w in weights]
        dbs = [torch.empty(o, dtype=x.dtype, device=dev) if b is not None else None for o, b in zip(outs, biases)]
    if batch == 0:          # an empty batch contributes zero gradients
        for t in dws + dbs:
            if t is not None:
                t.zero_()
        dx_empty = dx.view(x.shape) if dx is not None else None
        return [dx_empty] if input_only else [dx_empty] + dws + dbs
    of = (ctypes.c_int64 * n)(*outs)
    ws_bytes = int(L.load().nmtg_mlp_bwd_dtype_workspace_bytes(L.i32(n), of, L.i64(batch), L.i64(in_f), L.i32(L.dtype_code(x))))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    use_mask = mask is not None and mask.numel() > 0 and p > 0.0
    have_pre = pre is not None and pre.numel() > 0
    # the saved buffers are read as dense arrays: a strided view is copied (and the copy bound to a name, so that it
    # lives until the kernels have been queued)
    post = post.contiguous() if post is not None and post.numel() else None
    pre = pre.contiguous() if have_pre else None
    mask = mask.contiguous() if use_mask else None
    L.call("nmtg_mlp_bwd", L.i32(n), L.ptr(x2), _ptr_array(weights), of, L.i64(batch), L.i64(in_f), L.ptr(g2),
           L.ptr(post), L.ptr(pre), L.ptr(mask), L.f32(p), L.i32(L.ACT_CODES[act]), L.ptr(dx), _ptr_array(dws),
           _ptr_array(dbs), L.ptr(ws), L.i64(ws.numel()), L.i32(L.dtype_code(x)), L.stream_of(x))
    dx_out = dx.view(x.shape) if dx is not None else None
    if input_only:
        return [dx_out]
    return [dx_out] + dws + dbs
