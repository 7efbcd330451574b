"""Incremental (step by step) decoding for the two attention operators, on the HIP kernels.

What the reference does in the `incremental` branches of its attention functions
(onmt/modules/optimized/self_attention_func.py:162-174, encdec_attention_func_bias.py:181-213), with the same
cache entries so that the reference's beam search can reorder them (every entry is time-first [T, B, E] and is
re-indexed along dimension 1):
    self-attention     cache['k'], cache['v']      keys / values of all positions decoded so far (grow by one row,
                                                   inside a buffer with room to grow: see _append)
    cross-attention    cache['c_k'], cache['c_v']  keys / values of the encoder states (computed at the first step)
Inference only (no autograd graph, no dropout). The projections are GEMM calls of the library, the attention core is
the compact cross-attention entry point (queries and a [Tk, B*H, 2, D] key/value block come in, the context goes
out), which takes a key mask [B, Tk]: the mask of a one-position step (a time-mask row or a key-padding mask) is
handed over in that form. The cache bookkeeping (slices, concatenation, the interleave of keys and values) is tensor
movement on the device, exactly the reference's. A later step may carry one new position only: with more than one,
the new positions would need a causal mask among themselves, which the cross-attention core does not take.
"""
import os

import torch

from .. import _lib as L
from ..native import encdec_multihead_attn_bias_blaslt as ed_native
from ..native.linear_gemm import gemm


def _project(x, weight, bias):
    t, b, e = x.shape
    return gemm(x.reshape(t * b, e), weight, False, True, bias=bias).view(t, b, weight.shape[0])


def _decode_core(heads, q_lin, keys, values, pad_mask):
    """One query position: the cache-streaming kernel (nmtg_attn_decode) reads keys and values where they lie."""
    tk, b, e = keys.shape
    d = e // heads
    q_lin = q_lin.contiguous()
    km = None
    if pad_mask is not None:
        km = pad_mask.to(torch.uint8).contiguous()
        if km.shape != (b, tk):
            raise RuntimeError(f"incremental attention: key mask of shape {tuple(km.shape)}, expected {(b, tk)}")
    probs = torch.empty(b * heads, 1, tk, dtype=q_lin.dtype, device=q_lin.device)
    context = torch.empty(1, b, e, dtype=q_lin.dtype, device=q_lin.device)
    L.call("nmtg_attn_decode", L.ptr(q_lin), L.i64(e), L.ptr(keys), L.i64(keys.stride(0)), L.i64(keys.stride(1)), L.ptr(values),
           L.i64(values.stride(0)), L.i64(values.stride(1)), L.ptr(km), L.ptr(probs), L.ptr(context), L.i64(e), L.i64(b),
           L.i64(heads), L.i64(d), L.i64(tk), L.f32(d ** -0.5), L.i32(L.dtype_code(q_lin)), L.stream_of(q_lin))
    return context, probs


def _decode_ok(q_lin, keys, values, heads):
    """NMTG_ATTN_DECODE=0 keeps one-position steps on the GEMM path (the plainer of the two validated paths)."""
    e = keys.shape[2]
    return (q_lin.shape[0] == 1 and os.environ.get("NMTG_ATTN_DECODE", "1") != "0" and e // heads in (32, 64, 128)
            and 0 < keys.shape[0] <= 16384 and q_lin.dtype in (torch.float16, torch.bfloat16)
            and keys.stride(2) == 1 and values.stride(2) == 1 and all(s % 8 == 0 for s in keys.stride()[:2] + values.stride()[:2])
            and keys.data_ptr() % 16 == 0 and values.data_ptr() % 16 == 0)


def _core(heads, q_lin, keys, values, pad_mask):
    """q_lin [Tq, B, E]; keys, values [Tk, B, E] -> (context [Tq, B, E], probabilities [B*H, Tq, Tk])."""
    if _decode_ok(q_lin, keys, values, heads):
        return _decode_core(heads, q_lin, keys, values, pad_mask)
    tk, b, e = keys.shape
    d = e // heads
    kv = torch.stack([keys.view(tk, b * heads, d), values.view(tk, b * heads, d)], dim=-2).view(tk, b, 2 * e)
    scores, probs, _, context = ed_native.forward_compact(False, heads, q_lin.contiguous(), kv, pad_mask, 0.0)
    return context, probs


def _key_mask(mask, use_time_mask, b, tk, device):
    """The mask of a one-position step as a key mask [B, Tk] (True = masked), or None. The reference fills the scores
    [B*H, 1, Tk] with -inf where the mask is set (self_attention_func.py:203-215): a time mask is 2-D and broadcasts
    over the batch (its one row, or the last row of a [T, Tk] mask, is the new position's), a key-padding mask is
    [B, Tk]."""
    if mask is None:
        return None
    mask = mask.to(device=device, dtype=torch.bool)
    if use_time_mask:
        if mask.dim() == 1:
            mask = mask.unsqueeze(0)
        if mask.dim() != 2 or mask.size(-1) != tk or mask.size(0) not in (1, tk):
            raise RuntimeError(f"incremental self-attention: time mask of shape {tuple(mask.shape)}, expected [1, {tk}] (the new "
                               f"position's row) or [{tk}, {tk}] (whose last row it is)")
        return mask[-1:].expand(b, tk).contiguous()
    if mask.dim() == 3:
        mask = mask.squeeze(1)
    if mask.shape != (b, tk):
        raise RuntimeError(f"incremental self-attention: key-padding mask of shape {tuple(mask.shape)}, expected {(b, tk)}")
    return mask.contiguous()


def _append(cache, name, row):
    """cache[name] [T, B, E] with `row` (the B * E values of one position) behind it. The reference concatenates (a copy of the whole cache per
    step, self_attention_func.py:165-169). Here the rows live in a buffer with room to grow and cache[name] is its
    leading slice, which carries the buffer as an attribute (the dict keeps exactly the reference's entries): while the
    caller leaves that tensor in place, a step writes one row. A caller that replaces cache[name] (beam search re-indexes
    every entry along dimension 1, which yields new tensors) gets a fresh buffer filled from it: the reference's copy,
    with room for the steps that follow."""
    old = cache[name]
    n = old.shape[0]
    buf = getattr(old, "_nmtg_buffer", None)
    in_place = (buf is not None and buf.shape[0] > n and buf.shape[1:] == old.shape[1:] and buf.dtype == old.dtype
                and buf.device == old.device and old.is_contiguous() and old.data_ptr() == buf.data_ptr())
    if not in_place:
        buf = old.new_empty((max(2 * n, n + 64),) + tuple(old.shape[1:]))
        buf[:n].copy_(old)
    buf[n:n + 1].view(row.shape).copy_(row)       # `row` may be the strided [1, B*H, D] slice of the projection
    grown = buf[:n + 1]
    grown._nmtg_buffer = buf
    return grown


@torch.no_grad()
def self_attn_step(heads, inputs, input_weights, output_weights, input_biases, output_biases, mask, cache,
                   use_time_mask=True):
    """inputs [T_new, B, E]: all positions at the first call (no 'k' in the cache), one new position afterwards.
    mask: a time mask (use_time_mask: [T_new, T_total], True = masked) or a key-padding mask [B, T_total]; both are
    applied as the reference applies them. -> (outputs [T_new, B, E], probabilities [B*H, T_new, T_total])."""
    t_new, b, e = inputs.shape
    d = e // heads
    lin = _project(inputs, input_weights, input_biases).view(t_new, b * heads, 3, d)
    queries = lin[:, :, 0, :].reshape(t_new, b, e)
    first = not ("k" in cache and "v" in cache)
    if not first:
        if t_new != 1:
            raise NotImplementedError("incremental self-attention: one new position per step once the cache is filled")
        # the new row goes from the interleaved projection straight into the cache (one copy each)
        keys = _append(cache, "k", lin[:, :, 1, :])
        values = _append(cache, "v", lin[:, :, 2, :])
    else:
        keys = lin[:, :, 1, :].reshape(t_new, b, e)
        values = lin[:, :, 2, :].reshape(t_new, b, e)
    cache["k"], cache["v"] = keys, values
    if first and t_new > 1:
        # a prefix of several positions: the full-sequence kernel with its mask, fed with the same projection
        from ..native import self_multihead_attn_blaslt as sa_native
        if mask is not None:
            mask = mask.to(torch.bool)
        _, probs, _, context = sa_native.forward_compact(use_time_mask and mask is not None, False, heads,
                                                         lin.view(t_new, b, 3 * e), mask, 0.0)
    else:
        context, probs = _core(heads, queries, keys, values, _key_mask(mask, use_time_mask, b, keys.shape[0], inputs.device))
    return _project(context, output_weights, output_biases), probs


@torch.no_grad()
def encdec_attn_step(heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, input_bias_q,
                     input_bias_kv, output_bias, mask, cache):
    """inputs_q [Tq, B, E]; inputs_kv [Tk, B, E] is read at the first call only. mask: key padding [B, Tk]."""
    tq, b, e = inputs_q.shape
    d = e // heads
    if "c_k" in cache and "c_v" in cache:
        keys, values = cache["c_k"], cache["c_v"]
    else:
        tk = inputs_kv.shape[0]
        kv = _project(inputs_kv, input_weights_kv, input_bias_kv).view(tk, b * heads, 2, d)
        keys = kv[:, :, 0, :].reshape(tk, b, e)
        values = kv[:, :, 1, :].reshape(tk, b, e)
        cache["c_k"], cache["c_v"] = keys, values
    q_lin = _project(inputs_q, input_weights_q, input_bias_q)
    context, probs = _core(heads, q_lin, keys, values, mask)
    return _project(context, output_weights, output_bias), probs
