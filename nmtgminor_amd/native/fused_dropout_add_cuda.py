"""Stand-in for the reference module `fused_dropout_add_cuda`
(onmt/modules/extensions/dropout_add/fused_dropout_add.cpp:28-66): forward, backward.

`forward` takes one optional extra argument, `mask`: an explicit uint8 keep-mask to replay
instead of drawing one (the reference always draws its own)."""
import torch

from .. import _lib as L
from .._rng import philox_seed_offset


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def forward(is_training, inputs, residuals, dropout_prob, mask=None):
    """-> (dropout_mask uint8 like inputs, outputs); outputs aliases `inputs` (in place)."""
    L.require_cuda(inputs, residuals, mask)
    _check(inputs.dtype == residuals.dtype, "fused_dropout_add: dtype mismatch")
    _check(inputs.is_contiguous() and residuals.is_contiguous(), "fused_dropout_add: tensors must be contiguous")
    _check(inputs.numel() == residuals.numel(), "fused_dropout_add: size mismatch")
    n = inputs.numel()
    if is_training and dropout_prob > 0.0:
        if mask is not None:
            _check(mask.dtype == torch.uint8 and mask.numel() == n and mask.is_contiguous(),
                   "fused_dropout_add: mask must be a contiguous uint8 tensor of the input's size")
            mode, seed, offset = 1, 0, 0
        else:
            mask = torch.empty(inputs.shape, dtype=torch.uint8, device=inputs.device)
            mode = 2
            seed, offset = philox_seed_offset(inputs.device, n)
    else:
        mask = torch.empty(inputs.shape, dtype=torch.uint8, device=inputs.device)  # unread, as in the reference
        mode, seed, offset = 0, 0, 0
    import ctypes
    L.call("nmtg_dropout_add_fwd", L.ptr(inputs), L.ptr(residuals), L.ptr(mask), L.i64(n), L.f32(dropout_prob),
           L.i32(mode), ctypes.c_uint64(seed), ctypes.c_uint64(offset), L.i32(L.dtype_code(inputs)), L.stream_of(inputs))
    return mask, inputs


def backward(output_grads, dropout_add_mask, dropout_prob):
    L.require_cuda(output_grads, dropout_add_mask)
    output_grads = output_grads.contiguous()
    if not dropout_prob > 0.0:
        return output_grads.clone()
    _check(dropout_add_mask.dtype == torch.uint8 and dropout_add_mask.numel() == output_grads.numel(),
           "fused_dropout_add: mask must be uint8 with the gradient's size")
    dx = torch.empty_like(output_grads)
    dropout_add_mask = dropout_add_mask.contiguous()      # bound to a name: a temporary would be freed before the kernel reads it
    L.call("nmtg_dropout_add_bwd", L.ptr(output_grads), L.ptr(dropout_add_mask), L.ptr(dx),
           L.i64(output_grads.numel()), L.f32(dropout_prob), L.i32(L.dtype_code(output_grads)), L.stream_of(output_grads))
    return dx
