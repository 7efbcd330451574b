"""Gated feed-forward activation + dropout on the HIP kernels nmtg_glu_fwd / nmtg_glu_bwd: the element-wise middle of the
gated PositionWiseFeedForward, which the reference runs as PyTorch ops (onmt/modules/optimized/feed_forward.py:188-200)."""
import ctypes

import torch

from .. import _lib as L
from .._rng import philox_seed_offset

ACT_CODES = dict(L.ACT_CODES, swish=L.ACT_SILU, sigmoid=5)


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _rows(x):
    _check(x.dim() >= 2 and x.shape[-1] % 2 == 0, "glu: input must be [..., 2 * inner]")
    _check(x.dtype in (torch.float32, torch.float16, torch.bfloat16), "glu: fp32, fp16 or bf16 tensor required")
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    return x2, x.shape[-1] // 2


def forward(x, act, p, mask=None):
    """x [..., 2 * inner] -> (y [..., inner], mask). mask None with p > 0: one keep flag per output is drawn and returned
    (uint8 [rows, inner]); a given mask [mask_rows, inner] (uint8, mask_rows dividing the rows: row m uses mask row
    m % mask_rows) is replayed: [batch, inner] over a [time, batch, 2 * inner] input is the reference's variational dropout."""
    L.require_cuda(x, mask)
    x2, inner = _rows(x)
    rows = x2.shape[0]
    y = torch.empty(*x.shape[:-1], inner, dtype=x.dtype, device=x.device)
    mode, seed, offset, mask_rows = 0, 0, 0, rows
    if p > 0.0:
        if mask is not None:
            _check(mask.dtype == torch.uint8 and mask.dim() == 2 and mask.shape[1] == inner and mask.is_contiguous(),
                   "glu: mask must be contiguous uint8 [mask_rows, inner]")
            mask_rows = mask.shape[0]
            _check(mask_rows >= 1 and rows % mask_rows == 0, "glu: the mask rows must divide the input rows")
            mode = 1
        else:
            mask = torch.empty(rows, inner, dtype=torch.uint8, device=x.device)
            mode = 2
            seed, offset = philox_seed_offset(x.device, rows * inner)
    else:
        mask = None
    if rows:
        L.call("nmtg_glu_fwd", L.ptr(x2), L.i64(x2.stride(0)), L.ptr(y), L.ptr(mask), L.i64(mask_rows), L.i64(rows), L.i64(inner),
               L.i32(ACT_CODES[act]), L.i32(mode), L.f32(p), ctypes.c_uint64(seed), ctypes.c_uint64(offset),
               L.i32(L.dtype_code(x)), L.stream_of(x))
    return y, mask


def backward(grad_y, x, act, p, mask):
    """-> grad_x shaped like x."""
    L.require_cuda(grad_y, x, mask)
    x2, inner = _rows(x)
    rows = x2.shape[0]
    g2 = grad_y.reshape(rows, inner)
    if not g2.is_contiguous():
        g2 = g2.contiguous()
    _check(g2.dtype == x.dtype, "glu: gradient dtype differs from the input's")
    dx = torch.empty(rows, 2 * inner, dtype=x.dtype, device=x.device)
    mode = 1 if (p > 0.0 and mask is not None) else 0
    if rows:
        L.call("nmtg_glu_bwd", L.ptr(g2), L.ptr(x2), L.i64(x2.stride(0)), L.ptr(mask if mode else None),
               L.i64(mask.shape[0] if mode else rows), L.ptr(dx), L.i64(2 * inner), L.i64(rows), L.i64(inner),
               L.i32(ACT_CODES[act]), L.i32(mode), L.f32(p), L.i32(L.dtype_code(x)), L.stream_of(x))
    return dx.view(x.shape)
