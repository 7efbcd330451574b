"""Incremental decoding (one position per step, keys / values cached) against the CPU oracle's full-sequence rows.

Decoding position by position with the cache must reproduce, row by row, what the attention computes for the whole
sequence under a causal mask: the property the reference's translator relies on
(onmt/modules/optimized/self_attention_func.py:162-174, encdec_attention_func_bias.py:181-213). Every decoded row is
compared with the oracle (fp64 on the rounded operands) at the 16-bit tolerance, and, as a secondary check, with the
library's own full-sequence result. The cache entries
('k', 'v', 'c_k', 'c_v': time-first [T, B, E]) can be re-indexed along the batch dimension between steps, as beam
search does.
"""
from types import SimpleNamespace

import pytest
import torch

from nmtgminor_amd.modules.encdec_attention import EncdecMultiheadAttn
from nmtgminor_amd.modules.self_attention import SelfMultiheadAttn
from nmtgminor_amd.modules.transformer_layers import DecoderLayer
from oracle import attention as oat, inputs, transformer_layers as otl
from util import assert_close

D = torch.float64

pytestmark = pytest.mark.gpu


def _randomise(module, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for p in module.parameters():
            p.add_((0.1 if p.dim() == 1 else 0.02) * torch.randn(p.shape, generator=g))
    return module


def close(a, b, dtype, what):
    # secondary check, library against library: the same products, accumulated by different kernels (a [1, T] row
    # instead of a [T, T] tile), each rounded to 16 bits on its own
    assert_close(a, b.float().cpu(), dtype, what, rtol=2e-2, atol=4e-3 if dtype == torch.float16 else 3e-2)


def _cpu(module, *names):
    return [getattr(module, n).detach().cpu() for n in names]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("prefix", [1, 3])
def test_self_attention_step_by_step(dev, dtype, prefix):
    t, b, e, h = 11, 3, 128, 4
    attn = _randomise(SelfMultiheadAttn(e, h, 0.1), 91).to(dev).to(dtype).eval()
    x = torch.randn(t, b, e, generator=torch.Generator().manual_seed(92)).to(dtype).to(dev)
    causal = torch.triu(torch.ones(t, t, device=dev), 1).bool()
    with torch.no_grad():
        full, _ = attn(x, None, None, causal)
    cache = {}
    rows = []
    with torch.no_grad():
        out, cov = attn(x[:prefix], None, None, causal[:prefix, :prefix], incremental=True, incremental_cache=cache)
        rows.append(out)
        assert cov.shape == (b * h, prefix, prefix)
        homes = set()
        for i in range(prefix, t):
            out, cov = attn(x[i:i + 1], None, None, causal[i:i + 1, :i + 1], incremental=True, incremental_cache=cache)
            rows.append(out)
            assert cache["k"].shape == (i + 1, b, e) and cache["v"].shape == (i + 1, b, e)
            homes.add((cache["k"].data_ptr(), cache["v"].data_ptr()))
            assert cov.shape == (b * h, 1, i + 1)
            assert_close(cov.float().sum(-1), torch.ones(b * h, 1), dtype, "probabilities sum to one", atol=2e-2)
        assert len(homes) == 1                 # the cache grows inside one buffer: a step writes a row, it copies nothing
    w_in, w_out, b_in, b_out = _cpu(attn, "in_proj_weight", "out_proj_weight", "in_proj_bias", "out_proj_bias")
    want = oat.self_attn_fwd(x.cpu(), w_in, w_out, b_in, b_out, h, None, causal.cpu(), 0.0, None, D, round_to=dtype)
    assert_close(torch.cat(rows), want["outputs"], dtype, "stepwise self-attention vs oracle")
    assert_close(cov, want["dropout_results"][:, t - 1:t], dtype, "last step's probabilities vs oracle")
    close(torch.cat(rows), full, dtype, "stepwise self-attention")
    with pytest.raises(NotImplementedError):
        attn(x[:2], None, None, None, incremental=True, incremental_cache=cache)       # two positions onto a filled cache
    with pytest.raises(RuntimeError):
        attn(x[:1], None, None, None, incremental=True, incremental_cache=None)
    # a time mask for a step is the new position's row, or the square mask whose last row that is: other row counts are
    # refused (filled caches are copied: the refused call must not have grown them)
    keys = cache["k"].shape[0]
    with pytest.raises(RuntimeError, match="time mask"):
        attn(x[:1], None, None, causal[:3, :keys + 1], incremental=True, incremental_cache=dict(cache))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_self_attention_steps_honour_a_key_padding_mask(dev, dtype):
    # a batch whose prefixes start with padding: the padded keys must stay out of every step's softmax
    # (reference: masked_fill_ of the scores for either mask kind, self_attention_func.py:203-215)
    t, b, e, h = 9, 3, 128, 4
    attn = _randomise(SelfMultiheadAttn(e, h, 0.1), 97).to(dev).to(dtype).eval()
    x = torch.randn(t, b, e, generator=torch.Generator().manual_seed(98)).to(dtype).to(dev)
    pads = torch.tensor([0, 2, 4])                                   # leading pad positions per batch entry
    pad_mask = (torch.arange(t)[None, :] < pads[:, None])           # [B, T], True = pad
    w_in, w_out, b_in, b_out = _cpu(attn, "in_proj_weight", "out_proj_weight", "in_proj_bias", "out_proj_bias")
    cache = {}
    with torch.no_grad():
        for i in range(4, t):                                        # first call: a prefix of 5 positions, then one by one
            lo = 0 if i == 4 else i
            out, cov = attn(x[lo:i + 1], None, pad_mask[:, :i + 1].to(dev), None, incremental=True, incremental_cache=cache)
            want = oat.self_attn_fwd(x[:i + 1].cpu(), w_in, w_out, b_in, b_out, h, pad_mask[:, :i + 1], None, 0.0, None, D,
                                     round_to=dtype)
            assert_close(out, want["outputs"][lo:], dtype, f"step {i}: outputs vs oracle")
            assert_close(cov, want["dropout_results"][:, lo:], dtype, f"step {i}: probabilities vs oracle")
            # exact zeros on the padded keys
            for bi in range(b):
                assert (cov[bi * h:(bi + 1) * h, :, :pads[bi]] == 0).all()


def test_one_position_against_the_longest_cache_at_head_dimension_128(dev):
    """16384 cached keys of head dimension 128: the score row plus the partial contexts take more than 64 KB of LDS, the
    launch that has to ask for the larger allocation. One query position, a key mask on the second sequence; probabilities
    and context against the softmax of the same row in fp64 (scores rounded to the tensors' type, as the kernel stores them)."""
    from nmtgminor_amd.modules import incremental
    tk, b, h, d, dtype = 16384, 2, 2, 128, torch.bfloat16
    e = h * d
    g = torch.Generator().manual_seed(97)
    q = torch.randn(1, b, e, generator=g).to(dtype)
    keys = torch.randn(tk, b, e, generator=g).to(dtype)
    values = torch.randn(tk, b, e, generator=g).to(dtype)
    pad = torch.zeros(b, tk, dtype=torch.bool)
    pad[1, 16000:] = True
    pad[1, 5] = True
    assert incremental._decode_ok(q.to(dev), keys.to(dev), values.to(dev), h)
    ctx, probs = incremental._decode_core(h, q.to(dev), keys.to(dev), values.to(dev), pad.to(dev))
    q4, k4, v4 = q.view(b, h, d).to(D), keys.view(tk, b, h, d).to(D), values.view(tk, b, h, d).to(D)
    s = (torch.einsum("bhd,tbhd->bht", q4, k4) * d ** -0.5).to(dtype).to(D)
    s = s.masked_fill(pad.view(b, 1, tk), float("-inf"))
    pr = torch.softmax(s, -1)
    assert_close(probs.view(b, h, tk), pr, dtype, "probabilities", atol=1e-5)
    assert (probs.view(b, h, tk).cpu()[1, :, 16000:] == 0).all() and (probs.view(b, h, tk).cpu()[1, :, 5] == 0).all()
    assert_close(ctx.view(b, h, d), torch.einsum("bht,tbhd->bhd", pr.to(dtype).to(D), v4), dtype, "context")


@pytest.mark.parametrize("d", [32, 64, 128])
def test_one_position_does_not_read_the_cache_behind_a_sentences_last_live_key(dev, d):
    """Key masks of every kind in one batch: padding at the end, a hole in the middle, both, a sentence without any live
    key, a sentence with every key live. The cache rows behind each sentence's last live key hold NaN: the kernel must
    not read them (their probability is zero whatever they hold), and the row still equals the masked softmax in fp64."""
    from nmtgminor_amd.modules import incremental
    tk, b, h, dtype = 700, 5, 2, torch.bfloat16
    e = h * d
    g = torch.Generator().manual_seed(98)
    q = torch.randn(1, b, e, generator=g).to(dtype)
    keys = torch.randn(tk, b, e, generator=g).to(dtype)
    values = torch.randn(tk, b, e, generator=g).to(dtype)
    pad = torch.zeros(b, tk, dtype=torch.bool)
    pad[0, 333:] = True
    pad[1, 100:164] = True
    pad[2, 7] = True
    pad[2, 699] = True
    pad[3, :] = True
    live = [333, tk, 699, 0, tk]
    kd, vd = keys.clone(), values.clone()
    for bi, n in enumerate(live):
        kd[n:, bi] = float("nan")
        vd[n:, bi] = float("nan")
    assert incremental._decode_ok(q.to(dev), kd.to(dev), vd.to(dev), h)
    ctx, probs = incremental._decode_core(h, q.to(dev), kd.to(dev), vd.to(dev), pad.to(dev))
    q4, k4, v4 = q.view(b, h, d).to(D), keys.view(tk, b, h, d).to(D), values.view(tk, b, h, d).to(D)
    s = (torch.einsum("bhd,tbhd->bht", q4, k4) * d ** -0.5).to(dtype).to(D)
    s = s.masked_fill(pad.view(b, 1, tk), float("-inf"))
    pr = torch.softmax(s, -1)
    pr[3] = 0.0                                     # no live key: zeros, not the NaN of an empty softmax
    assert_close(probs.view(b, h, tk), pr, dtype, "probabilities", atol=1e-5)
    assert (probs.view(b, h, tk).cpu()[pad.view(b, 1, tk).expand(b, h, tk)] == 0).all()
    assert_close(ctx.view(b, h, d), torch.einsum("bht,tbhd->bhd", pr.to(dtype).to(D), v4), dtype, "context")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cross_attention_with_cached_encoder_states(dev, dtype):
    tq, tk, b, e, h = 7, 37, 3, 128, 4
    g = torch.Generator().manual_seed(93)
    attn = _randomise(EncdecMultiheadAttn(h, e, 0.1), 94).to(dev).to(dtype).eval()
    q = torch.randn(tq, b, e, generator=g).to(dtype).to(dev)
    ctxt = torch.randn(tk, b, e, generator=g).to(dtype).to(dev)
    pad, _ = inputs.lengths_mask(b, tk, tk // 2, tk, g)
    pad = pad.to(dev)
    with torch.no_grad():
        full, full_cov = attn(q, ctxt, ctxt, pad)
        cache = {}
        rows = []
        for i in range(tq):
            # after the first step the encoder states are not read again
            kv = ctxt if i == 0 else torch.full_like(ctxt, float("nan"))
            out, cov = attn(q[i:i + 1], kv, kv, pad, incremental=True, incremental_cache=cache)
            rows.append(out)
            close(cov, full_cov[:, i:i + 1], dtype, "stepwise coverage")
        assert cache["c_k"].shape == (tk, b, e) and cache["c_v"].shape == (tk, b, e)
    w_q, w_kv, w_out = _cpu(attn, "in_proj_weight_q", "in_proj_weight_kv", "out_proj_weight")
    want = oat.encdec_attn_fwd(q.cpu(), ctxt.cpu(), w_q, w_kv, w_out, None, None, None, h, pad.cpu(), 0.0, None, D,
                               round_to=dtype)
    assert_close(torch.cat(rows), want["outputs"], dtype, "stepwise cross-attention vs oracle")
    close(torch.cat(rows), full, dtype, "stepwise cross-attention")


def test_decoder_layer_step_by_step_with_beam_reordering(dev):
    dtype = torch.bfloat16
    opt = SimpleNamespace(model_size=128, inner_size=256, n_heads=4, dropout=0.1, attn_dropout=0.1, variational_dropout=False,
                          macaron=False, rezero=False, ffn_activation="gelu", ffn_glu=False, fast_self_attention=True,
                          fast_xattention=True, fast_feed_forward=True, ignore_source=False)
    tq, tk, b = 6, 20, 4
    g = torch.Generator().manual_seed(95)
    layer = _randomise(DecoderLayer(opt), 96).to(dev).to(dtype).eval()
    x = torch.randn(tq, b, 128, generator=g).to(dtype).to(dev)
    ctxt = torch.randn(tk, b, 128, generator=g).to(dtype).to(dev)
    src_pad, _ = inputs.lengths_mask(b, tk, tk // 2, tk, g)
    src_pad = src_pad.to(dev)
    causal = torch.triu(torch.ones(tq, tq, device=dev), 1).bool()
    perm = torch.tensor([2, 0, 3, 1], device=dev)
    with torch.no_grad():
        full, _, _ = layer(x, ctxt, causal, src_pad)
        # the hypotheses are re-ordered after step 2: from then on batch entry j continues hypothesis perm[j]
        x_after = x[:, perm]
        full_after, _, _ = layer(torch.cat([x[:3][:, perm], x_after[3:]]), ctxt[:, perm], causal, src_pad[perm])
        cache = None
        rows = []
        for i in range(tq):
            if i == 3:
                for key in cache:
                    cache[key] = cache[key].index_select(1, perm)
            cur_x = x[i:i + 1] if i < 3 else x_after[i:i + 1]
            cur_ctxt, cur_pad = (ctxt, src_pad) if i < 3 else (ctxt[:, perm], src_pad[perm])
            out, _, cache = layer(cur_x, cur_ctxt, causal[i:i + 1, :i + 1], cur_pad, incremental=True, incremental_cache=cache)
            rows.append(out)
        assert sorted(cache) == ["c_k", "c_v", "k", "v"]
    # against the layer oracle (fp64, the weights the kernels saw): a whole layer rounds to 16 bits at every operator
    # boundary and the oracle nowhere, hence the layer tolerance of tests/test_zy_layers_gpu.py
    p64 = {k: v.detach().cpu().to(dtype).to(D) for k, v in layer.state_dict().items()}
    want, _ = otl.decoder_layer(x.cpu().to(D), ctxt.cpu().to(D), p64, opt.n_heads, causal.cpu(), src_pad.cpu(), act="gelu",
                                training=False)
    x_mixed = torch.cat([x[:3][:, perm], x_after[3:]])
    want_after, _ = otl.decoder_layer(x_mixed.cpu().to(D), ctxt[:, perm].cpu().to(D), p64, opt.n_heads, causal.cpu(),
                                      src_pad[perm].cpu(), act="gelu", training=False)
    tol = 2.5e-2 * max(1.0, float(want.abs().max()))
    assert_close(torch.cat(rows[:3]), want[:3], dtype, "steps before the re-ordering vs oracle", rtol=3e-2, atol=tol)
    assert_close(torch.cat(rows[3:]), want_after[3:], dtype, "steps after the re-ordering vs oracle", rtol=3e-2, atol=tol)
    close(torch.cat(rows[:3]), full[:3], dtype, "steps before the re-ordering")
    close(torch.cat(rows[3:]), full_after[3:], dtype, "steps after the re-ordering")
