"""Attention over packed variable-length sequences (nmtg_flash_attn_fwd / _bwd through the flash_attn_cuda stand-in and
the autograd functions of nmtgminor_amd/modules/flash_mha.py) against the per-sequence oracle
(oracle/flash_attention.py, pinned against torch's scaled_dot_product_attention in tests/test_oracle_pins.py).

What the reference computes here: flash_attn_cuda.fwd / .bwd as called from onmt/modules/optimized/flash_mha.py:43-183.
Tolerance: the one every 16-bit comparison here uses (util.assert_close: 2e-2 relative, 1e-3 absolute, the gradients'
absolute part scaled by their largest expected magnitude). The oracle is given round_to = the tensors' type and then rounds
where the kernels do: the unnormalised probabilities as matrix-core operands against the kernel's reference point, dS and
the kept probabilities in the backward, each result once. The log-sum-exp, an fp32 result of 16-bit inputs, to 2e-3
absolute; rowsum(dO * O) to fp32 accuracy against the same sum over the output the kernel itself stored.
"""
import pytest
import torch

from nmtgminor_amd._rng import philox4x32_10
from nmtgminor_amd.modules import flash_mha
from nmtgminor_amd.native import flash_attn_cuda
from oracle import flash_attention as ofa
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64


def _cu(lengths):
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.as_tensor(lengths), 0)
    return cu


def _inputs(lq, lk, heads, d, dtype, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(sum(lq), heads, d, generator=g) * std).to(dtype)
    k = (torch.randn(sum(lk), heads, d, generator=g) * std).to(dtype)
    v = torch.randn(sum(lk), heads, d, generator=g).to(dtype)
    do = torch.randn(sum(lq), heads, d, generator=g).to(dtype)
    return q, k, v, do


def _check_fwd_bwd(dev, q, k, v, do, lq, lk, causal, p=0.0, mask=None, scale=None, philox=False):
    dtype, (heads, d) = q.dtype, q.shape[1:]
    cu_q, cu_k = _cu(lq), _cu(lk)
    mq, mk = max(lq), max(lk)
    scale = d ** -0.5 if scale is None else scale
    qd, kd, vd, dod = (t.to(dev) for t in (q, k, v, do))
    out = torch.full_like(qd, float("nan"))
    res = flash_attn_cuda.fwd(qd, kd, vd, out, cu_q.to(dev), cu_k.to(dev), mq, mk, p, scale, False, causal, philox, 0, None,
                              dropout_mask=None if mask is None else mask.to(dev))
    lse = res[0]
    rng = flash_attn_cuda.last_rng
    p_eff = p
    if philox:                                        # the drawn mask comes back; its scale is 256 / round(256 (1 - p))
        mask = res[1].cpu()
        p_eff = 1.0 - round(256 * (1.0 - p)) / 256.0
    want_out, want_lse = ofa.flash_attn_fwd(q, k, v, cu_q, cu_k, mq, scale, causal, p_eff, mask, D, round_to=dtype)
    assert_close(out, want_out, dtype, "out")
    for b in range(len(lq)):
        if lk[b] == 0:
            assert bool(torch.isinf(lse[b, :, :lq[b]]).all())
            continue
        assert_close(lse[b, :, :lq[b]], want_lse[b, :, :lq[b]], torch.float32, f"lse[{b}]", rtol=1e-3, atol=2e-3)
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (qd, kd, vd))
    _, _, _, sd = flash_attn_cuda.bwd(dod, qd, kd, vd, out, lse, dq, dk, dv, cu_q.to(dev), cu_k.to(dev), mq, mk, p, scale,
                                      False, causal, 0, None, rng=rng)
    if p:
        # the backward above read the forward's keep bits; one that only gets the generator state (or the mask) fills a
        # workspace of its own and must arrive at the same numbers
        assert len(rng) == 5 and rng[4] is not None
        dq2, dk2, dv2 = (torch.full_like(t, float("nan")) for t in (qd, kd, vd))
        flash_attn_cuda.bwd(dod, qd, kd, vd, out, lse, dq2, dk2, dv2, cu_q.to(dev), cu_k.to(dev), mq, mk, p, scale, False, causal,
                            0, None, rng=rng[:4])
        assert torch.equal(dq2, dq) and torch.equal(dk2, dk) and torch.equal(dv2, dv)
    # the backward is a function of the output it is handed: the oracle's gets the same one (D = rowsum(dO * O) feels a
    # last-place difference of O wherever dS = P (dP - D) cancels)
    wdq, wdk, wdv, wsd = ofa.flash_attn_bwd(do, q, k, v, cu_q, cu_k, mq, scale, causal, p_eff, mask, D, round_to=dtype, out=out.cpu())
    assert_close(dq, wdq, dtype, "dq", scale_atol=True)
    assert_close(dk, wdk, dtype, "dk", scale_atol=True)
    assert_close(dv, wdv, dtype, "dv", scale_atol=True)
    rows = (do.to(D) * out.cpu().to(D)).sum(-1)                                    # [total_q, H]
    for b in range(len(lq)):
        assert_close(sd[b, :, :lq[b]], rows[cu_q[b]:cu_q[b + 1]].t(), torch.float32, f"softmax_d[{b}]", rtol=1e-4, atol=1e-4)
        assert_close(sd[b, :, :lq[b]], wsd[b, :, :lq[b]], torch.float32, f"softmax_d[{b}] against the oracle", rtol=5e-2, atol=1e-1)
    return mask


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_ragged_self_attention_matches_the_oracle(dev, dtype, d, causal):
    lens = [5, 64, 131, 1, 70]
    q, k, v, do = _inputs(lens, lens, 2, d, dtype, seed=d + causal)
    _check_fwd_bwd(dev, q, k, v, do, lens, lens, causal)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_different_query_and_key_lengths_and_an_empty_sequence(dev, dtype):
    lq, lk = [3, 140, 0, 17, 9], [200, 65, 12, 0, 129]
    q, k, v, do = _inputs(lq, lk, 3, 64, dtype, seed=11)
    _check_fwd_bwd(dev, q, k, v, do, lq, lk, False, scale=0.2)


@pytest.mark.parametrize("causal", [False, True])
def test_large_scores_do_not_overflow_the_online_softmax(dev, causal):
    lens = [150, 66]
    q, k, v, do = _inputs(lens, lens, 2, 64, torch.bfloat16, seed=5, std=6.0)     # scores of a few hundred before scaling
    _check_fwd_bwd(dev, q, k, v, do, lens, lens, causal, scale=1.0)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_dropout_with_a_replayed_mask(dev, dtype, d, causal):
    lq, lk = [70, 33, 129], [70, 140, 5]
    q, k, v, do = _inputs(lq, lk, 2, d, dtype, seed=21)
    g = torch.Generator().manual_seed(3)
    mask = (torch.rand(len(lq), 2, max(lq), max(lk), generator=g) < 0.75).to(torch.uint8)
    _check_fwd_bwd(dev, q, k, v, do, lq, lk, causal, p=0.25, mask=mask)


@pytest.mark.parametrize("dtype,d", [(torch.float16, 64), (torch.bfloat16, 128)])
def test_dropout_drawn_on_the_device_is_the_documented_philox_stream_in_both_passes(dev, dtype, d):
    lq, lk = [70, 33, 129], [70, 140, 5]
    heads, p = 2, 0.3
    q, k, v, do = _inputs(lq, lk, heads, d, dtype, seed=23)
    torch.cuda.manual_seed(1234)
    mask = _check_fwd_bwd(dev, q, k, v, do, lq, lk, False, p=p, philox=True)      # forward and backward agree with the mask
    mode, seed, offset = flash_attn_cuda.last_rng[:3]
    assert mode == 2
    thr = round(256 * (1 - p))
    q4, k4 = (max(lq) + 3) // 4, (max(lk) + 3) // 4
    for b, h, i, j in [(0, 0, 0, 0), (0, 1, 69, 69), (1, 0, 32, 139), (2, 1, 128, 4), (2, 0, 77, 3), (1, 1, 5, 66)]:
        block = ((b * heads + h) * q4 + i // 4) * k4 + j // 4
        words = philox4x32_10([offset, offset >> 32, block, block >> 32], [seed, seed >> 32])
        byte = (words[i % 4] >> (8 * (j % 4))) & 0xFF
        assert int(mask[b, h, i, j]) == int(byte < thr), (b, h, i, j)
    kept = torch.cat([mask[b, :, :lq[b], :lk[b]].reshape(-1) for b in range(3)]).double().mean()
    assert abs(float(kept) - thr / 256) < 0.02
    for b in range(3):                                                           # nothing outside the sequences is written
        assert int(mask[b, :, lq[b]:, :].sum()) == 0 and int(mask[b, :, :, lk[b]:].sum()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_packed_qkv_function_takes_strided_slots_and_fills_one_gradient_tensor(dev, dtype):
    lens, heads, d = [37, 128, 66], 4, 64
    g = torch.Generator().manual_seed(31)
    qkv = torch.randn(sum(lens), 3, heads, d, generator=g).to(dtype)
    do = torch.randn(sum(lens), heads, d, generator=g).to(dtype)
    cu = _cu(lens)
    x = qkv.to(dev).requires_grad_()
    out = flash_mha.flash_bert_mha(x, cu.to(dev), max(lens), 0.0, None, True, False)
    out.backward(do.to(dev))
    want, _ = ofa.flash_attn_fwd(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, max(lens), None, True, ctype=D, round_to=dtype)
    wdq, wdk, wdv, _ = ofa.flash_attn_bwd(do, qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, max(lens), None, True, ctype=D, round_to=dtype)
    assert_close(out, want, dtype, "out")
    assert x.grad.shape == qkv.shape
    for slot, w, name in ((0, wdq, "dq"), (1, wdk, "dk"), (2, wdv, "dv")):
        assert_close(x.grad[:, slot], w, dtype, name, scale_atol=True)


def test_packed_kv_function_with_dropout_repeats_its_mask_in_the_backward(dev):
    lq, lk, heads, d, dtype, p = [20, 90], [130, 64], 2, 64, torch.bfloat16, 0.2
    g = torch.Generator().manual_seed(37)
    q = torch.randn(sum(lq), heads, d, generator=g).to(dtype)
    kv = torch.randn(sum(lk), 2, heads, d, generator=g).to(dtype)
    do = torch.randn(sum(lq), heads, d, generator=g).to(dtype)
    cu_q, cu_k = _cu(lq), _cu(lk)
    qd, kvd = q.to(dev).requires_grad_(), kv.to(dev).requires_grad_()
    out, lse, mask = flash_mha.flash_encdec_mha(qd, kvd, cu_q.to(dev), cu_k.to(dev), max(lq), max(lk), p, None, False, True)
    torch.cuda.manual_seed(999)                       # the generator moves on between the passes; the context carries the state
    out.backward(do.to(dev))
    p_eff = 1.0 - round(256 * (1 - p)) / 256.0
    want, _ = ofa.flash_attn_fwd(q, kv[:, 0], kv[:, 1], cu_q, cu_k, max(lq), None, False, p_eff, mask.cpu(), D, round_to=dtype)
    wdq, wdk, wdv, _ = ofa.flash_attn_bwd(do, q, kv[:, 0], kv[:, 1], cu_q, cu_k, max(lq), None, False, p_eff, mask.cpu(), D,
                                          round_to=dtype)
    assert_close(out, want, dtype, "out")
    assert_close(qd.grad, wdq, dtype, "dq", scale_atol=True)
    assert_close(kvd.grad[:, 0], wdk, dtype, "dk", scale_atol=True)
    assert_close(kvd.grad[:, 1], wdv, dtype, "dv", scale_atol=True)


@pytest.mark.parametrize("seed", range(3000, 3010))
def test_randomly_drawn_shapes(dev, seed):
    """Lengths around the tile sizes (64 keys, 128 queries), head counts, both head dimensions, causal or not, dropout
    replayed, drawn or off, query and key lengths equal or independent, scale drawn too."""
    import random
    rnd = random.Random(seed)
    batch, heads, d = rnd.randint(1, 5), rnd.randint(1, 4), rnd.choice([64, 128])
    pick = lambda: rnd.choice([0, 1, 2, 63, 64, 65, 127, 128, 129, rnd.randint(1, 200), rnd.randint(1, 200)])
    lq = [pick() for _ in range(batch)]
    lk = lq if rnd.random() < 0.5 else [pick() for _ in range(batch)]
    if max(lq) == 0:
        lq = [7] + lq[1:]
        lk = lq if lk is lq else lk
    if max(lk) == 0:
        lk = [9] + lk[1:]
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    causal = rnd.random() < 0.5
    mode = rnd.choice(["none", "replay", "philox"])
    p = 0.0 if mode == "none" else rnd.choice([0.1, 0.3, 0.5])
    q, k, v, do = _inputs(lq, lk, heads, d, dtype, seed)
    mask = None
    if mode == "replay":
        mask = (torch.rand(batch, heads, max(lq), max(lk), generator=torch.Generator().manual_seed(seed)) >= p).to(torch.uint8)
    _check_fwd_bwd(dev, q, k, v, do, lq, lk, causal, p=p, mask=mask, scale=rnd.choice([None, 0.05, 0.3]), philox=mode == "philox")


def test_unsupported_inputs_are_refused(dev):
    cu = _cu([4]).to(dev)
    q = torch.zeros(4, 2, 64, device=dev)
    with pytest.raises(RuntimeError, match="fp16 or bf16"):
        flash_attn_cuda.fwd(q, q, q, None, cu, cu, 4, 4, 0.0, 1.0, False, False, False)
    q = torch.zeros(4, 2, 48, device=dev, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="head dimension 48"):
        flash_attn_cuda.fwd(q, q, q, None, cu, cu, 4, 4, 0.0, 1.0, False, False, False)
    q = torch.zeros(4, 2, 72, device=dev, dtype=torch.float16)[:, :, 4:68]          # 8-byte aligned view
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        flash_attn_cuda.fwd(q, q, q, torch.empty(4, 2, 64, device=dev, dtype=torch.float16), cu, cu, 4, 4, 0.0, 1.0, False, False, False)
