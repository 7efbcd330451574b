"""Stand-in for the third-party module `flash_attn_cuda` (flash-attention 1.x) that the reference binds at
onmt/modules/optimized/flash_mha.py:32-75, on the HIP kernels nmtg_flash_attn_fwd / nmtg_flash_attn_bwd.

    fwd(q, k, v, out, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, zero_tensors,
        causal, return_softmax, num_splits, generator) -> [softmax_lse] (+ [S_dmask] with return_softmax)
    bwd(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
        softmax_scale, zero_tensors, causal, num_splits, generator) -> (dq, dk, dv, softmax_d)

q [total_q, H, D], k / v [total_k, H, D]: fp16 / bf16 views with a contiguous last dimension (the slots of a packed
[total, 3, H, D] projection are taken as they are), D = 64 or 128; cu_seqlens int32 [B + 1] on the device.

Differences from the CUDA module, all on the dropout side:
 * the keep-mask is a function of a Philox (seed, offset) pair; fwd draws the pair from the device's default generator
   (or `generator`) and remembers it in `last_rng`, bwd takes it from the keyword `rng` (the autograd functions of
   nmtgminor_amd/modules/flash_mha.py carry it from forward to backward) or, without it, replays `last_rng`; restoring
   the generator state before bwd, as the reference does, is harmless and not needed;
 * keyword `rng=(seed, offset)` on fwd fixes the Philox state instead of drawing one from the generator;
 * the kernels read the keep decisions as one bit per element from a workspace that a small kernel fills ahead of them;
   fwd allocates it and hands it on inside `last_rng` (a fifth entry), and a bwd that receives it runs no generator;
   a four-entry state makes bwd fill a workspace of its own from (seed, offset) or the mask;
 * return_softmax hands back the keep-mask (uint8 [B, H, max_seqlen_q, max_seqlen_k]) instead of the sign-encoded
   probability matrix, which exists nowhere in this kernel; keyword `dropout_mask` replays such a mask (tests);
 * num_splits is accepted and ignored: the kernels never accumulate across blocks, so results do not depend on it."""
import ctypes

import torch

from .. import _lib as L
from .._rng import philox_seed_offset

last_rng = None


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _view(t, name, heads=None, d=None):
    _check(t.dim() == 3, f"flash_attn: {name} must be [tokens, heads, head_dim]")
    _check(t.stride(2) == 1 or t.shape[2] == 1, f"flash_attn: the head dimension of {name} must be contiguous")
    if heads is not None:
        _check(t.shape[1] == heads and t.shape[2] == d, f"flash_attn: {name} has shape {tuple(t.shape)}, expected [*, {heads}, {d}]")
    return [L.i64(t.stride(0)), L.i64(t.stride(1))]


def _common(q, k, v, cu_q, cu_k):
    L.require_cuda(q, k, v, cu_q, cu_k)
    _check(q.dtype in (torch.float16, torch.bfloat16), "flash_attn: fp16 or bf16 tensors required")
    _check(k.dtype == q.dtype and v.dtype == q.dtype, "flash_attn: q, k and v must share a dtype")
    _check(cu_q.dtype == torch.int32 and cu_k.dtype == torch.int32 and cu_q.is_contiguous() and cu_k.is_contiguous(),
           "flash_attn: cu_seqlens must be contiguous int32 tensors")
    _check(cu_q.numel() == cu_k.numel() and cu_q.numel() >= 1, "flash_attn: cu_seqlens_q and cu_seqlens_k must both be [batch + 1]")
    _check(k.shape == v.shape and k.shape[1:] == q.shape[1:], "flash_attn: k and v must be [total_k, H, D] with q's H and D")
    return cu_q.numel() - 1, q.shape[1], q.shape[2]


def _draw(device, count, generator):
    if generator is None:
        return philox_seed_offset(device, count)
    seed, offset = generator.initial_seed() & 0xFFFFFFFFFFFFFFFF, generator.get_offset()
    generator.set_offset(offset + ((int(count) + 3) // 4) * 4)
    return seed, offset


def _bits(batch, heads, max_q, max_k, device):
    n = L.load().nmtg_flash_attn_dropout_bits_bytes(L.i64(batch), L.i64(heads), L.i64(max_q), L.i64(max_k))
    return torch.empty(max(int(n), 16) // 4, dtype=torch.int32, device=device)


def fwd(q, k, v, out, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, zero_tensors,
        causal, return_softmax, num_splits=0, generator=None, *, dropout_mask=None, rng=None):
    global last_rng
    batch, heads, d = _common(q, k, v, cu_seqlens_q, cu_seqlens_k)
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    _check(out.shape == q.shape and out.dtype == q.dtype, "flash_attn: out must look like q")
    if zero_tensors:
        out.zero_()
    lse = torch.zeros(batch, heads, max_seqlen_q, dtype=torch.float32, device=q.device)
    mode, seed, offset, mask_out, bits = 0, 0, 0, None, None
    if dropout_p > 0.0:
        bits = _bits(batch, heads, max_seqlen_q, max_seqlen_k, q.device)
        if dropout_mask is not None:
            _check(dropout_mask.dtype == torch.uint8 and tuple(dropout_mask.shape) == (batch, heads, max_seqlen_q, max_seqlen_k)
                   and dropout_mask.is_contiguous(), "flash_attn: dropout_mask must be contiguous uint8 [B, H, max_q, max_k]")
            L.require_cuda(dropout_mask)
            mode = 1
        else:
            mode = 2
            blocks = batch * heads * ((max_seqlen_q + 3) // 4) * ((max_seqlen_k + 3) // 4)
            # rng=(seed, offset): a Philox state fixed by the caller (a step that is captured into a graph cannot ask
            # the generator for one)
            seed, offset = rng if rng is not None else _draw(q.device, 4 * blocks, generator)
            if return_softmax:
                mask_out = torch.zeros(batch, heads, max_seqlen_q, max_seqlen_k, dtype=torch.uint8, device=q.device)
    last_rng = (mode, seed, offset, dropout_mask, bits)
    L.call("nmtg_flash_attn_fwd", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(out), L.ptr(cu_seqlens_q), L.ptr(cu_seqlens_k),
           L.ptr(lse), L.i64(batch), L.i64(heads), L.i64(d), L.i64(max_seqlen_q), L.i64(max_seqlen_k),
           *_view(q, "q"), *_view(k, "k", heads, d), *_view(v, "v", heads, d), *_view(out, "out", heads, d),
           L.f32(softmax_scale), L.i32(int(bool(causal))), L.i32(mode), L.f32(dropout_p), L.ptr(dropout_mask if mode == 1 else None),
           L.ptr(mask_out), L.ptr(bits), ctypes.c_uint64(seed), ctypes.c_uint64(offset), L.i32(L.dtype_code(q)), L.stream_of(q))
    if return_softmax:
        return [lse, dropout_mask if mode == 1 else mask_out]
    return [lse]


def bwd(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
        softmax_scale, zero_tensors, causal, num_splits=0, generator=None, *, rng=None):
    batch, heads, d = _common(q, k, v, cu_seqlens_q, cu_seqlens_k)
    L.require_cuda(dout, out, softmax_lse, dq, dk, dv)
    _check(dout.shape == q.shape and out.shape == q.shape and dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape,
           "flash_attn: dout, out and dq must look like q, dk like k, dv like v")
    _check(all(t.dtype == q.dtype for t in (dout, out, dq, dk, dv)), "flash_attn: every tensor must have q's dtype")
    _check(softmax_lse.dtype == torch.float32 and tuple(softmax_lse.shape) == (batch, heads, max_seqlen_q) and
           softmax_lse.is_contiguous(), "flash_attn: softmax_lse must be contiguous fp32 [B, H, max_seqlen_q]")
    if zero_tensors:
        dq.zero_(), dk.zero_(), dv.zero_()
    mode, seed, offset, mask, bits, ready = 0, 0, 0, None, None, 0
    if dropout_p > 0.0:
        state = rng if rng is not None else last_rng
        _check(state is not None and state[0] != 0, "flash_attn: backward with dropout needs the forward's generator state")
        mode, seed, offset, mask = state[:4]
        bits = state[4] if len(state) > 4 else None
        ready = int(bits is not None)
        if bits is None:
            bits = _bits(batch, heads, max_seqlen_q, max_seqlen_k, q.device)
        L.require_cuda(bits)
    softmax_d = torch.zeros(batch, heads, max_seqlen_q, dtype=torch.float32, device=q.device)
    L.call("nmtg_flash_attn_bwd", L.ptr(dout), L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(out), L.ptr(softmax_lse), L.ptr(dq),
           L.ptr(dk), L.ptr(dv), L.ptr(softmax_d), L.ptr(cu_seqlens_q), L.ptr(cu_seqlens_k), L.i64(batch), L.i64(heads),
           L.i64(d), L.i64(max_seqlen_q), L.i64(max_seqlen_k), *_view(dout, "dout", heads, d), *_view(q, "q"),
           *_view(k, "k", heads, d), *_view(v, "v", heads, d), *_view(out, "out", heads, d), *_view(dq, "dq", heads, d),
           *_view(dk, "dk", heads, d), *_view(dv, "dv", heads, d), L.f32(softmax_scale), L.i32(int(bool(causal))),
           L.i32(mode), L.f32(dropout_p), L.ptr(mask if mode == 1 else None), L.ptr(bits), L.i32(ready), ctypes.c_uint64(seed),
           ctypes.c_uint64(offset), L.i32(L.dtype_code(q)), L.stream_of(q))
    return dq, dk, dv, softmax_d


# ---------------------------------------------------------------------------------------------------------------------
# The same kernels over a padded batch (no counterpart in the CUDA module): what the training calls of self_attn_func /
# encdec_attn_func use when the caller does not return the coverage, so that no [B*H, len_q, len_k] tensor is written.
# ---------------------------------------------------------------------------------------------------------------------
def _view4(t, name, heads, d):
    _check(t.dim() == 4 and t.shape[2] == heads and t.shape[3] == d, f"flash_attn: {name} must be [len, batch, {heads}, {d}]")
    _check(t.stride(3) == 1, f"flash_attn: the head dimension of {name} must be contiguous")
    return [L.i64(t.stride(0)), L.i64(t.stride(1)), L.i64(t.stride(2))]


def _key_info(batch, len_k, device):
    n = L.load().nmtg_flash_attn_key_info_bytes(L.i64(batch), L.i64(len_k))
    return torch.empty(max(int(n), 4) // 4, dtype=torch.int32, device=device)


def _pad_mask(mask, batch, len_k):
    if mask is None:
        return None
    _check(mask.dtype == torch.uint8 and tuple(mask.shape) == (batch, len_k) and mask.is_contiguous(),
           "flash_attn: key_padding_mask must be contiguous uint8 [batch, len_k]")
    L.require_cuda(mask)
    return mask


def _time_mask(mask, len_q, len_k, device):
    """-> (mask, workspace) of a time mask uint8 [len_q, len_k] shared by every sequence and head, or (None, None)"""
    if mask is None:
        return None, None
    _check(mask.dtype == torch.uint8 and tuple(mask.shape) == (len_q, len_k) and mask.is_contiguous(),
           "flash_attn: time_mask must be contiguous uint8 [len_q, len_k]")
    L.require_cuda(mask)
    n = L.load().nmtg_flash_attn_time_info_bytes(L.i64(len_q), L.i64(len_k))
    return mask, torch.empty(max(int(n), 4) // 4, dtype=torch.int32, device=device)


def fwd_batched(q, k, v, key_padding_mask, dropout_p, softmax_scale, causal, *, dropout_mask=None, rng=None, want_mask=False,
                time_mask=None):
    """q [len_q, B, H, D], k / v [len_k, B, H, D] (views with a contiguous D), key_padding_mask uint8 [B, len_k] or None,
    time_mask uint8 [len_q, len_k] or None (one of the two at most)
    -> (out [len_q, B, H, D] contiguous, softmax_lse [B, H, len_q], state); `state` goes to bwd_batched as it is (dropout
    mode, Philox pair, explicit mask, keep bits, drawn mask when want_mask)."""
    L.require_cuda(q, k, v)
    _check(q.dtype in (torch.float16, torch.bfloat16) and k.dtype == q.dtype and v.dtype == q.dtype,
           "flash_attn: q, k and v must share a 16-bit dtype")
    _check(q.dim() == 4 and k.shape == v.shape, "flash_attn: q [len_q, B, H, D], k and v [len_k, B, H, D]")
    len_q, batch, heads, d = q.shape
    len_k = k.shape[0]
    _check(tuple(k.shape[1:]) == (batch, heads, d), "flash_attn: k and v must have q's batch, heads and head_dim")
    pad = _pad_mask(key_padding_mask, batch, len_k)
    kinfo = _key_info(batch, len_k, q.device) if pad is not None else None
    tmask, tinfo = _time_mask(time_mask, len_q, len_k, q.device)
    out = torch.empty(len_q, batch, heads, d, dtype=q.dtype, device=q.device)
    lse = torch.empty(batch, heads, len_q, dtype=torch.float32, device=q.device)
    mode, seed, offset, mask_out, bits = 0, 0, 0, None, None
    if dropout_p > 0.0:
        bits = _bits(batch, heads, len_q, len_k, q.device)
        if dropout_mask is not None:
            _check(dropout_mask.dtype == torch.uint8 and dropout_mask.numel() == batch * heads * len_q * len_k and
                   dropout_mask.is_contiguous(), "flash_attn: dropout_mask must be contiguous uint8 [B, H, len_q, len_k]")
            L.require_cuda(dropout_mask)
            mode = 1
        else:
            mode = 2
            blocks = batch * heads * ((len_q + 3) // 4) * ((len_k + 3) // 4)
            seed, offset = rng if rng is not None else philox_seed_offset(q.device, 4 * blocks)
            if want_mask:
                mask_out = torch.zeros(batch, heads, len_q, len_k, dtype=torch.uint8, device=q.device)
    L.call("nmtg_flash_attn_batched_fwd", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(out), L.ptr(pad), L.ptr(kinfo), L.ptr(tmask),
           L.ptr(tinfo), L.ptr(lse),
           L.i64(batch), L.i64(heads), L.i64(d), L.i64(len_q), L.i64(len_k), *_view4(q, "q", heads, d), *_view4(k, "k", heads, d),
           *_view4(v, "v", heads, d), *_view4(out, "out", heads, d), L.f32(softmax_scale), L.i32(int(bool(causal))), L.i32(mode),
           L.f32(dropout_p), L.ptr(dropout_mask if mode == 1 else None), L.ptr(mask_out), L.ptr(bits), ctypes.c_uint64(seed),
           ctypes.c_uint64(offset), L.i32(L.dtype_code(q)), L.stream_of(q))
    return out, lse, (mode, seed, offset, dropout_mask if mode == 1 else None, bits, mask_out)


def bwd_batched(dout, q, k, v, out, softmax_lse, dq, dk, dv, key_padding_mask, dropout_p, softmax_scale, causal, state, *,
                time_mask=None):
    """Writes dq, dk, dv (views with the strides of q, k, v: the slots of one projection-gradient buffer) -> softmax_d."""
    L.require_cuda(dout, q, k, v, out, softmax_lse, dq, dk, dv)
    len_q, batch, heads, d = q.shape
    len_k = k.shape[0]
    _check(all(t.dtype == q.dtype for t in (dout, k, v, out, dq, dk, dv)), "flash_attn: every tensor must have q's dtype")
    _check(dout.shape == q.shape and out.shape == q.shape and dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape,
           "flash_attn: dout, out and dq must look like q, dk like k, dv like v")
    _check(dout.stride() == out.stride() and dq.stride() == q.stride() and dk.stride() == k.stride() and dv.stride() == v.stride(),
           "flash_attn: dout must have the strides of out, and dq, dk, dv those of q, k, v")
    _check(softmax_lse.dtype == torch.float32 and tuple(softmax_lse.shape) == (batch, heads, len_q) and softmax_lse.is_contiguous(),
           "flash_attn: softmax_lse must be contiguous fp32 [B, H, len_q]")
    pad = _pad_mask(key_padding_mask, batch, len_k)
    kinfo = _key_info(batch, len_k, q.device) if pad is not None else None
    tmask, tinfo = _time_mask(time_mask, len_q, len_k, q.device)
    mode, seed, offset, mask, bits = state[:5]
    if dropout_p <= 0.0:
        mode, bits = 0, None
    ready = int(bits is not None)
    if mode != 0 and bits is None:
        bits = _bits(batch, heads, len_q, len_k, q.device)
    softmax_d = torch.empty(batch, heads, len_q, dtype=torch.float32, device=q.device)
    L.call("nmtg_flash_attn_batched_bwd", L.ptr(dout), L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(out), L.ptr(softmax_lse), L.ptr(dq),
           L.ptr(dk), L.ptr(dv), L.ptr(softmax_d), L.ptr(pad), L.ptr(kinfo), L.ptr(tmask), L.ptr(tinfo), L.i64(batch), L.i64(heads),
           L.i64(d), L.i64(len_q),
           L.i64(len_k), *_view4(q, "q", heads, d), *_view4(k, "k", heads, d), *_view4(v, "v", heads, d),
           *_view4(out, "out", heads, d), L.f32(softmax_scale), L.i32(int(bool(causal))), L.i32(mode), L.f32(dropout_p),
           L.ptr(mask if mode == 1 else None), L.ptr(bits), L.i32(ready), ctypes.c_uint64(seed), ctypes.c_uint64(offset),
           L.i32(L.dtype_code(q)), L.stream_of(q))
    return softmax_d
