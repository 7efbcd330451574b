"""CPU restatement of the reference's rotary position encoding and of self / encoder-decoder attention with it.
Test infrastructure only: nothing under nmtgminor_amd/ imports this.

Reference: rotate_half, apply_rotary_pos_emb, rotate_backward (onmt/modules/optimized/self_attention_func.py:25-48),
applied to the query / key views of the in-projection output (:178-184) with the gradient rule of :467-469; the
one-operand form of onmt/modules/optimized/encdec_attention_func.py:21-34, queries with the query positions' table and
keys with the key positions' (:173-180). Everything here is differentiable PyTorch in `ctype` (fp64 in the tests), so
gradients come from autograd; rotate_backward is restated only to be pinned as the transpose of the forward."""
import torch

from .attention import _core_fwd, _linear, _r


def rotate_half(x):
    """cat(-x[D/2:], x[:D/2]) over the last dimension (self_attention_func.py:25-28)."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary(x, cos, sin):
    """x [T, N, D], cos / sin [T, 1, D] -> x cos + rotate_half(x) sin (self_attention_func.py:31-42)."""
    return x * cos + rotate_half(x) * sin


def rotate_backward(dx):
    """cat(dx[D/2:], -dx[:D/2]) (self_attention_func.py:45-47): the transpose of rotate_half."""
    h = dx.shape[-1] // 2
    return torch.cat((dx[..., h:], -dx[..., :h]), dim=-1)


def apply_rotary_transposed(g, cos, sin):
    """g cos + rotate_backward(sin g) (self_attention_func.py:467-469)."""
    return g * cos + rotate_backward(sin * g)


def tables(positions, dim, base=10000.0, dtype=torch.float64):
    """(cos, sin), each [T, 1, dim], of the usual rotary angles pos * base^(-2i/dim), duplicated over the two halves."""
    inv = base ** (-torch.arange(0, dim, 2, dtype=dtype) / dim)
    ang = torch.as_tensor(positions, dtype=dtype)[:, None] * inv[None, :]
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos()[:, None, :], ang.sin()[:, None, :]


def self_attn_rotary(x, w_in, w_out, b_in, b_out, heads, pad_mask, time_mask, cos, sin, p=0.0, dropout_mask=None,
                     ctype=torch.float64, round_to=None):
    """-> (outputs [T, B, E], dropout_results [B*H, T, T]); differentiable. round_to: the 16-bit type every tensor that
    the kernels store is rounded to on the way (projection, rotated slots, scores, probabilities, context); the rounding
    passes gradients through unchanged."""
    t, b, e = x.shape
    d = e // heads
    lin = _r(_linear(x.reshape(t * b, e).to(ctype), w_in.to(ctype), None if b_in is None else b_in.to(ctype)), round_to)
    lin = lin.view(t, b * heads, 3, d)
    q = _r(apply_rotary(lin[:, :, 0, :], cos.to(ctype), sin.to(ctype)), round_to)
    k = _r(apply_rotary(lin[:, :, 1, :], cos.to(ctype), sin.to(ctype)), round_to)
    v = lin[:, :, 2, :]
    _, _, dr, ctx = _core_fwd(q, k, v, heads, pad_mask, time_mask, p, dropout_mask, ctype, round_to)
    out = _linear(ctx.reshape(t * b, e), w_out.to(ctype), None if b_out is None else b_out.to(ctype)).view(t, b, e)
    return out, dr


def encdec_attn_rotary(x_q, x_kv, w_q, w_kv, w_out, heads, pad_mask, cos_q, sin_q, cos_k, sin_k, p=0.0, dropout_mask=None,
                       ctype=torch.float64, round_to=None):
    tq, b, e = x_q.shape
    tk = x_kv.shape[0]
    d = e // heads
    q = _r(_linear(x_q.reshape(tq * b, e).to(ctype), w_q.to(ctype), None), round_to).view(tq, b * heads, d)
    kv = _r(_linear(x_kv.reshape(tk * b, e).to(ctype), w_kv.to(ctype), None), round_to).view(tk, b * heads, 2, d)
    q = _r(apply_rotary(q, cos_q.to(ctype), sin_q.to(ctype)), round_to)
    k = _r(apply_rotary(kv[:, :, 0, :], cos_k.to(ctype), sin_k.to(ctype)), round_to)
    _, _, dr, ctx = _core_fwd(q, k, kv[:, :, 1, :], heads, pad_mask, None, p, dropout_mask, ctype, round_to)
    out = _linear(ctx.reshape(tq * b, e), w_out.to(ctype), None).view(tq, b, e)
    return out, dr
