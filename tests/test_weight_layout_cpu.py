"""The q/k/v weight-layout converters (nmtgminor_amd/modules/weight_layout.py): round trips, agreement with the
permutation the reference applies to Hugging Face checkpoints (onmt/models/whisper/whisper_encoder.py:246-274:
cat(q, k, v) viewed [3, H, D, E], transposed to [H, 3, D, E]), and the property that makes the layout useful — the
fused projection's output viewed [T, B*H, 3, D] is exactly the separate projections' outputs split per head."""
import pytest
import torch

from nmtgminor_amd.modules import weight_layout as wl


def test_matches_the_checkpoint_conversion_and_round_trips():
    e, h = 24, 4
    d = e // h
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(e, e, generator=g) for _ in range(3))
    fused = wl.interleave_qkv(q, k, v, h)
    want = torch.cat([q, k, v], 0).view(3, h, d, e).transpose(0, 1).reshape(-1, e)
    assert torch.equal(fused, want)
    for a, b in zip(wl.deinterleave_qkv(fused, h), (q, k, v)):
        assert torch.equal(a, b)
    kv = wl.interleave_kv(k, v, h)
    assert torch.equal(kv, torch.cat([k, v], 0).view(2, h, d, e).transpose(0, 1).reshape(-1, e))
    for a, b in zip(wl.deinterleave_kv(kv, h), (k, v)):
        assert torch.equal(a, b)
    bq, bk, bv = (torch.randn(e, generator=g) for _ in range(3))
    fb = wl.interleave_qkv(bq, bk, bv, h)
    assert fb.shape == (3 * e,) and torch.equal(wl.deinterleave_qkv(fb, h)[1], bk)
    packed = torch.cat([q, k, v], 0)
    assert torch.equal(wl.from_packed_qkv(packed, h), fused) and torch.equal(wl.to_packed_qkv(fused, h), packed)
    with pytest.raises(ValueError):
        wl.interleave_qkv(q, k, v, 5)
    with pytest.raises(ValueError):
        wl.interleave_qkv(q, k[:-1], v, h)


def test_fused_projection_yields_per_head_queries_keys_values():
    t, b, e, h = 5, 2, 16, 4
    d = e // h
    g = torch.Generator().manual_seed(2)
    x = torch.randn(t, b, e, generator=g, dtype=torch.float64)
    q, k, v = (torch.randn(e, e, generator=g, dtype=torch.float64) for _ in range(3))
    lin = (x.view(t * b, e) @ wl.interleave_qkv(q, k, v, h).t()).view(t, b * h, 3, d)
    for i, w in enumerate((q, k, v)):
        sep = (x.view(t * b, e) @ w.t()).view(t, b * h, d)
        torch.testing.assert_close(lin[:, :, i, :], sep)
    mha = torch.nn.MultiheadAttention(e, h, bias=True, dtype=torch.float64)
    from oracle import attention
    fused_w = wl.from_packed_qkv(mha.in_proj_weight.detach(), h)
    fused_b = wl.from_packed_qkv(mha.in_proj_bias.detach(), h)
    out = attention.self_attn_fwd(x, fused_w, mha.out_proj.weight.detach(), fused_b, mha.out_proj.bias.detach(), h, ctype=torch.float64)
    ref, _ = mha(x, x, x, need_weights=False)
    torch.testing.assert_close(out["outputs"], ref.detach(), rtol=1e-10, atol=1e-11)
