"""Projection-weight layouts on either side of the attention operators.

Checkpoints in the common layout (Hugging Face Whisper / BART / MBart, torch.nn.MultiheadAttention) keep separate
q, k, v projections, each [E, E] with rows ordered (head, head_dim). The fused operators take one in-projection whose
rows are ordered (head, {q, k, v}, head_dim), so that the projected activations viewed as [T, B*H, 3, D] yield
queries, keys and values without a copy; the cross-attention key/value projection likewise is (head, {k, v},
head_dim). These are the conversions the reference performs when it switches a loaded model to its fast attention
(onmt/models/whisper/whisper_encoder.py:246-274, whisper_decoder.py:43-70), in both directions, for weights
([E, E] -> [3E, E]) and biases ([E] -> [3E]) alike. Pure index permutations: no arithmetic, any dtype or device.
"""
import torch


def _interleave(parts, heads):
    e = parts[0].shape[0]
    if e % heads:
        raise ValueError(f"{e} rows do not split into {heads} heads")
    if any(p.shape != parts[0].shape for p in parts):
        raise ValueError("projections must have equal shapes")
    d = e // heads
    rest = parts[0].shape[1:]
    stacked = torch.stack([p.reshape(heads, d, *rest) for p in parts], dim=1)        # [H, n, D, ...]
    return stacked.reshape(len(parts) * e, *rest).contiguous()


def _deinterleave(fused, heads, n):
    rows = fused.shape[0]
    if rows % (n * heads):
        raise ValueError(f"{rows} rows do not split into {n} projections of {heads} heads")
    d = rows // (n * heads)
    rest = fused.shape[1:]
    v = fused.reshape(heads, n, d, *rest)
    return tuple(v[:, i].reshape(heads * d, *rest).contiguous() for i in range(n))


def interleave_qkv(q, k, v, heads):
    """Separate q / k / v weights [E, E] (or biases [E]) -> in_proj_weight [3E, E] (in_proj_bias [3E])."""
    return _interleave([q, k, v], heads)


def deinterleave_qkv(in_proj, heads):
    """in_proj_weight [3E, E] (or in_proj_bias [3E]) -> (q, k, v)."""
    return _deinterleave(in_proj, heads, 3)


def interleave_kv(k, v, heads):
    """Separate k / v weights -> in_proj_weight_kv [2E, E] of the cross-attention."""
    return _interleave([k, v], heads)


def deinterleave_kv(in_proj_kv, heads):
    return _deinterleave(in_proj_kv, heads, 2)


def from_packed_qkv(packed, heads):
    """torch.nn.MultiheadAttention's in_proj_weight / in_proj_bias (q rows, then k rows, then v rows) -> fused layout."""
    e = packed.shape[0] // 3
    return interleave_qkv(packed[:e], packed[e:2 * e], packed[2 * e:], heads)


def to_packed_qkv(in_proj, heads):
    return torch.cat(deinterleave_qkv(in_proj, heads), dim=0)
