"""Rotary position encoding on the HIP kernel (nmtg_rotary): what apply_rotary_pos_emb / rotate_backward of the
reference do with PyTorch ops (onmt/modules/optimized/self_attention_func.py:25-48), in place on strided head slots."""
import torch

from .. import _lib as L


def _table(t, rows, d, like):
    """cos / sin as the reference passes them ([T, 1, D] or [T, D]) -> contiguous [T, D] in the dtype of `like`."""
    t = t.reshape(-1, t.shape[-1])
    if t.shape != (rows, d):
        raise RuntimeError(f"rotary: position table of shape {tuple(t.shape)}, expected {(rows, d)}")
    return t.to(device=like.device, dtype=like.dtype).contiguous()


def rotate_(x, cos, sin, heads_total, head_dim, parts, stride_n, stride_part, inverse=False):
    """Rotates, in place, `parts` slots of `head_dim` elements in every one of `heads_total` heads of every position of
    x [T, ...] (x.stride(0) elements between positions, stride_n between heads, stride_part between the slots)."""
    L.require_cuda(x, cos, sin)
    if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise RuntimeError("rotary: fp32, fp16 or bf16 tensor required")
    if head_dim % 2:
        raise RuntimeError("rotary: the head dimension must be even")
    t = x.shape[0]
    if x.numel() == 0:
        return x
    if x[0].numel() > 1 and not x[0].is_contiguous():
        raise RuntimeError("rotary: positions must be contiguous blocks")
    cos, sin = _table(cos, t, head_dim, x), _table(sin, t, head_dim, x)
    L.call("nmtg_rotary", L.ptr(x), L.ptr(cos), L.ptr(sin), L.i64(t), L.i64(heads_total), L.i64(head_dim), L.i64(parts),
           L.i64(x.stride(0)), L.i64(stride_n), L.i64(stride_part), L.i32(int(inverse)), L.i32(L.dtype_code(x)), L.stream_of(x))
    return x


def rotate_qk_(lin, cos, sin, batch_heads, head_dim, inverse=False):
    """lin [T, B, 3E] viewed as [T, B*H, 3, D]: the query and key slots."""
    return rotate_(lin, cos, sin, batch_heads, head_dim, 2, 3 * head_dim, head_dim, inverse)


def rotate_q_(q_lin, cos, sin, batch_heads, head_dim, inverse=False):
    """q_lin [Tq, B, E] viewed as [Tq, B*H, D]."""
    return rotate_(q_lin, cos, sin, batch_heads, head_dim, 1, head_dim, head_dim, inverse)


def rotate_k_(kv_lin, cos, sin, batch_heads, head_dim, inverse=False):
    """kv_lin [Tk, B, 2E] viewed as [Tk, B*H, 2, D]: the key slot."""
    return rotate_(kv_lin, cos, sin, batch_heads, head_dim, 1, 2 * head_dim, head_dim, inverse)
