"""Shared plumbing of the attention stand-in modules."""
import ctypes
import os

import torch

from .. import _lib as L
from .._rng import philox_seed_offset


def check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def check_half(*tensors):
    for t in tensors:
        if t is not None:
            check(t.dtype in (torch.float16, torch.bfloat16), "Only HALF / BFLOAT16 is supported")
    dts = {t.dtype for t in tensors if t is not None}
    check(len(dts) <= 1, "all tensors must share one dtype")


def mask_arg(mask, use_time_mask, batch, len_q, len_k):
    """Reference mask conventions: time mask [len_q, len_k]; key padding [B, len_k] or
    [B, 1, 1, len_k] (onmt/modules/optimized/self_attention_func.py:90-99). -> (uint8 tensor, kind)"""
    if mask is None or mask.numel() == 0:
        return None, 0
    if use_time_mask:
        check(mask.numel() == len_q * len_k, "time mask must be [len_q, len_k]")
        return _word_aligned(mask.reshape(len_q, len_k).to(torch.uint8).contiguous()), 2
    check(mask.numel() == batch * len_k, "key padding mask must be [batch, len_k]")
    return _word_aligned(mask.reshape(batch, len_k).to(torch.uint8).contiguous()), 1


def _word_aligned(mask):
    """The kernels read mask bytes four (or eight) at a time: a uint8 view that starts at an odd address is copied."""
    return mask if mask.data_ptr() % 8 == 0 else mask.clone()


def dropout_args(is_training, p, shape, device, dropout_mask):
    """-> (mask tensor, mode, seed, offset)"""
    if is_training and p > 0.0:
        if dropout_mask is not None:
            n = 1
            for s in shape:
                n *= s
            check(dropout_mask.dtype == torch.uint8 and dropout_mask.numel() == n, "dropout mask must be uint8 [B*H, Tq, Tk]")
            return dropout_mask.contiguous().view(shape), 1, 0, 0
        m = torch.empty(shape, dtype=torch.uint8, device=device)
        n = m.numel()
        seed, offset = philox_seed_offset(device, n)
        return m, 2, seed, offset
    return torch.empty(0, dtype=torch.uint8, device=device), 0, 0, 0


def scores_needed(is_training, dtype, head_dim, tk, need_backward=None):
    """Whether a forward call has to keep the pre-softmax scores. They exist for the backward; a call that is neither in
    training mode nor followed by a backward (inference under torch.no_grad()) leaves them out where the one-kernel
    inference path takes the shape (16-bit tensors, head dimension 64 or 128, a key count that is a multiple of 4), and
    the stand-in then returns an empty tensor in their place. NMTG_ATTN_PROBS=0 keeps them always.
    `need_backward`: what the caller knows about a backward to come. An autograd function passes
    any(ctx.needs_input_grad) (inside its forward the grad mode is always off, whatever the caller's was); None asks
    the grad mode, which is right for a direct call of the stand-in module."""
    if need_backward is None:
        need_backward = torch.is_grad_enabled()
    if is_training or need_backward or os.environ.get("NMTG_ATTN_PROBS", "1") == "0":
        return True
    return not (dtype in (torch.float16, torch.bfloat16) and head_dim in (64, 128) and tk >= 1 and tk % 4 == 0)


def u64(v):
    return ctypes.c_uint64(v)


def workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
