"""Parity of the bandwidth-bound ops — dropout+add, masked softmax(+dropout), label-smoothed
cross-entropy — HIP (through the C ABI) vs the CPU oracle on identical seeded inputs.

Shapes follow the reference's tests where it has them: softmax with a row length that is not a
multiple of 4 (test/test_softmax.py:1-58), cross-entropy with padding on a fraction of rows and a
256 000-class vocabulary (onmt/modules/test_label_smoothing.py:76-118,
extensions/xentropy/test_xentropy.py:127-170), dropout-add at p = 0 (optimized/dropout_add.py:93-142).
"""
import pytest
import torch

from nmtgminor_amd._rng import philox_keep_mask_reference
from nmtgminor_amd.modules.attention_softmax import AttentionSoftmaxDropout
from nmtgminor_amd.modules.dropout_add import fused_dropout_add
from nmtgminor_amd.modules.softmax_xentropy import SoftmaxCrossEntropyLoss
from nmtgminor_amd.native import fused_dropout_add_cuda, mask_softmax_dropout_cuda, xentropy_cuda
from oracle import dropout_add as oda, inputs, softmax_dropout as osd, xentropy as oxe
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64
DTYPES = [torch.float32, torch.float16, torch.bfloat16]


# ----------------------------------------------------------------------------- dropout + add
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 7, 4096, 512 * 32 * 64 + 3])
def test_dropout_add_replayed_mask(dev, dtype, n):
    g = torch.Generator().manual_seed(31)
    x = torch.randn(n, generator=g).to(dtype)
    r = torch.randn(n, generator=g).to(dtype)
    m = inputs.bernoulli_mask((n,), 0.9, g)
    go = torch.randn(n, generator=g).to(dtype)
    xd = x.to(dev)
    mask, out = fused_dropout_add_cuda.forward(True, xd, r.to(dev), 0.1, m.to(dev))
    assert out.data_ptr() == xd.data_ptr()                       # in place, as the reference
    assert_close(out, oda.dropout_add_fwd(x, r, m, 0.1, D), dtype, "out")
    dx = fused_dropout_add_cuda.backward(go.to(dev), mask, 0.1)
    assert_close(dx, oda.dropout_add_bwd(go, m, 0.1, D)[0], dtype, "dx")
    assert (dx[m.to(dev) == 0] == 0).all()                        # dropped positions: exact zeros


@pytest.mark.parametrize("dtype", DTYPES)
def test_dropout_add_eval_and_p0(dev, dtype):
    g = torch.Generator().manual_seed(32)
    x = torch.randn(33, 40, generator=g).to(dtype)
    r = torch.randn(33, 40, generator=g).to(dtype)
    for training, p in ((False, 0.3), (True, 0.0)):
        _, out = fused_dropout_add_cuda.forward(training, x.to(dev), r.to(dev), p)
        assert_close(out, oda.dropout_add_fwd(x, r, None, 0.0, D), dtype, "eval out")


def test_dropout_add_philox_mask_is_reproducible_and_fair(dev):
    n = 1 << 20
    x = torch.ones(n, device=dev, dtype=torch.bfloat16)
    r = torch.zeros(n, device=dev, dtype=torch.bfloat16)
    torch.cuda.manual_seed(1234)
    m1, o1 = fused_dropout_add_cuda.forward(True, x.clone(), r, 0.25)
    m2, _ = fused_dropout_add_cuda.forward(True, x.clone(), r, 0.25)
    torch.cuda.manual_seed(1234)
    m3, _ = fused_dropout_add_cuda.forward(True, x.clone(), r, 0.25)
    assert torch.equal(m1, m3) and not torch.equal(m1, m2)        # same seed+offset -> same mask; offset advances
    keep = m1.float().mean().item()
    assert abs(keep - 0.75) < 5e-3
    assert_close(o1, m1.float().cpu() / 0.75, torch.bfloat16, "rng out")
    # bit-exact against the Python restatement of Philox4x32-10 on a few windows
    seed = torch.cuda.default_generators[0].initial_seed()
    for first in (0, 4, 1000, n - 16):
        want = philox_keep_mask_reference(seed, 0, first, 16, 0.75)
        assert m1[first:first + 16].cpu().tolist() == want


def test_dropout_add_autograd_wrapper(dev):
    g = torch.Generator().manual_seed(33)
    x = torch.randn(8, 4, 64, generator=g).to(torch.bfloat16)
    r = torch.randn(8, 4, 64, generator=g).to(torch.bfloat16)
    m = inputs.bernoulli_mask((8, 4, 64), 0.8, g)
    go = torch.randn(8, 4, 64, generator=g).to(torch.bfloat16)
    xin = x.to(dev).requires_grad_()
    rin = r.to(dev).requires_grad_()
    out = fused_dropout_add(xin * 1.0, rin, 0.2, True, m.to(dev))
    out.backward(go.to(dev))
    assert_close(out, oda.dropout_add_fwd(x, r, m, 0.2, D), torch.bfloat16, "out")
    assert_close(xin.grad, oda.dropout_add_bwd(go, m, 0.2, D)[0], torch.bfloat16, "dx")
    assert torch.equal(rin.grad.cpu(), go)


# ----------------------------------------------------------------------------- masked softmax
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bh,tq,tk", [(8, 75, 56), (6, 5, 1), (4, 64, 512), (4, 17, 1500), (2, 128, 128),
                                      (2, 9, 2048), (4, 7, 333), (2, 3, 4096)])
def test_softmax_dropout_fwd_bwd(dev, dtype, bh, tq, tk):
    if tk == 4096 and dtype == torch.float32:
        pytest.skip("4096 keys is the 16-bit limit")
    g = torch.Generator().manual_seed(41)
    heads = 2
    s = (torch.randn(bh, tq, tk, generator=g) * 3).to(dtype)
    pad, _ = inputs.lengths_mask(bh // heads, tk, max(1, tk // 2), tk, g)
    dm = inputs.bernoulli_mask((bh, tq, tk), 0.9, g)
    go = torch.randn(bh, tq, tk, generator=g).to(dtype)
    masked = osd.masked_scores(s.to(D), pad_mask=pad, heads=heads)
    sm_o, dr_o = osd.softmax_dropout_fwd(masked, dm, 0.1, D)
    ds_o = osd.softmax_dropout_bwd(go, sm_o, dm, 0.1, D)
    # fused key-padding mask + replayed dropout mask
    _, sm, dr = mask_softmax_dropout_cuda.forward(True, heads, s.to(dev), 0.1, pad_mask=pad.to(dev), dropout_mask=dm.to(dev))
    assert_close(sm, sm_o, dtype, "softmax")
    assert_close(dr, dr_o, dtype, "dropped")
    padk = pad.view(bh // heads, 1, 1, tk).expand(bh // heads, heads, tq, tk).reshape(bh, tq, tk)
    assert (sm.cpu()[padk] == 0).all() and (dr.cpu()[dm == 0] == 0).all()      # exact zeros
    rs = sm.float().sum(-1).cpu()
    assert (rs - 1).abs().max() < (1e-5 if dtype == torch.float32 else 2e-2)
    # backward, recomputing the probabilities from the saved scores
    ds = mask_softmax_dropout_cuda.backward_recompute(heads, go.to(dev), None, s.to(dev), dm.to(dev), 0.1, pad_mask=pad.to(dev))
    assert_close(ds, ds_o, dtype, "dscores(recompute)")
    assert (ds.cpu()[padk] == 0).all()
    # backward from saved probabilities (as stored, i.e. rounded to dtype)
    ds2 = mask_softmax_dropout_cuda.backward(heads, go.to(dev), sm, dm.to(dev), 0.1)
    assert_close(ds2, osd.softmax_dropout_bwd(go, sm.cpu(), dm, 0.1, D), dtype, "dscores(saved)")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_softmax_time_mask_premasked_scores_and_empty_rows(dev, dtype):
    g = torch.Generator().manual_seed(42)
    bh, t = 6, 96
    s = torch.randn(bh, t, t, generator=g).to(dtype)
    tm = torch.triu(torch.ones(t, t), 1).bool()
    want, _ = osd.softmax_dropout_fwd(osd.masked_scores(s.to(D), time_mask=tm), None, 0.0, D)
    _, sm, dr = mask_softmax_dropout_cuda.forward(False, 3, s.to(dev), 0.0, time_mask=tm.to(dev))
    assert sm.data_ptr() == dr.data_ptr()
    assert_close(dr, want, dtype, "causal")
    # -inf already in the scores (what the attention path hands over), incl. fully masked rows
    pre = s.clone()
    pre.masked_fill_(tm.unsqueeze(0), float("-inf"))
    pre[1, 5, :] = float("-inf")
    _, _, dr2 = mask_softmax_dropout_cuda.forward(False, 3, pre.to(dev), 0.0)
    want2, _ = osd.softmax_dropout_fwd(pre.to(D), None, 0.0, D)
    assert_close(dr2, want2, dtype, "premasked")
    assert (dr2[1, 5] == 0).all() and not torch.isnan(dr2).any()
    go = torch.randn(bh, t, t, generator=g).to(dtype)
    ds = mask_softmax_dropout_cuda.backward_recompute(3, go.to(dev), None, pre.to(dev), None, 0.0)
    assert_close(ds, osd.softmax_dropout_bwd(go, want2, None, 0.0, D), dtype, "premasked bwd")
    assert not torch.isnan(ds).any()


def test_softmax_rng_dropout_and_wrapper(dev):
    s = torch.randn(4, 32, 256, device=dev, dtype=torch.bfloat16)
    torch.cuda.manual_seed(7)
    mask, sm, dr = AttentionSoftmaxDropout.forward(s, False, 0.3, True, 2)
    assert mask.dtype == torch.uint8 and mask.shape == s.shape
    assert abs(mask.float().mean().item() - 0.7) < 2e-2
    assert_close(dr, sm.float().cpu() * mask.float().cpu() / 0.7, torch.bfloat16, "rng dropped")
    seed = torch.cuda.default_generators[0].initial_seed()
    assert mask.view(-1)[:12].cpu().tolist() == philox_keep_mask_reference(seed, 0, 0, 12, 0.7)
    go = torch.randn_like(s)
    ds = AttentionSoftmaxDropout.backward(go, sm, torch.tensor([0.3]), torch.tensor([2]), mask)
    assert_close(ds, osd.softmax_dropout_bwd(go.cpu(), sm.cpu(), mask.cpu(), 0.3, D), torch.bfloat16, "wrapper bwd")


def test_softmax_errors(dev):
    with pytest.raises(RuntimeError):
        mask_softmax_dropout_cuda.forward(False, 1, torch.randn(1, 2, 5000, device=dev), 0.0)     # row too long
    with pytest.raises(RuntimeError):
        mask_softmax_dropout_cuda.forward(False, 1, torch.randn(2, 2, 8), 0.0)                    # CPU tensor
    with pytest.raises(RuntimeError):
        mask_softmax_dropout_cuda.forward(True, 1, torch.randn(2, 2, 8, device=dev), 1.0)         # p = 1


# ----------------------------------------------------------------------------- cross-entropy
def _xent_case(dev, n, v, dtype, eps, pad, seed=51, misalign=0):
    d = inputs.xentropy_inputs(n, v, dtype, eps, padding_idx=pad, pad_fraction=1 / 6, seed=seed)
    logits = d["logits"]
    if misalign:                                   # rows that start off a 16-byte boundary
        buf = torch.empty(n * v + misalign, dtype=dtype, device=dev)
        ld = buf[misalign:].view(n, v)
        ld.copy_(logits)
    else:
        ld = logits.to(dev)
    labels = d["labels"].to(dev)
    losses, lse = xentropy_cuda.forward(ld, labels, eps, dtype != torch.float32, padding_idx=pad)
    lo, lseo = oxe.xentropy_fwd(logits, d["labels"], eps, pad, D)
    assert losses.dtype == torch.float32 and lse.dtype == torch.float32
    assert_close(losses, lo, torch.float32, "losses", rtol=2e-5, atol=2e-5)
    assert_close(lse, lseo, torch.float32, "lse", rtol=2e-6, atol=2e-5)
    gl = (torch.rand(n, generator=torch.Generator().manual_seed(seed)) + 0.5)
    dx = xentropy_cuda.backward(gl.to(dev), ld, lse, labels, eps, padding_idx=pad)
    dxo = oxe.xentropy_bwd(gl, logits, lseo, d["labels"], eps, pad, D)
    assert dx.dtype == dtype and dx.shape == (n, v)
    assert_close(dx, dxo, dtype, "dlogits", atol=1e-6 if dtype == torch.float32 else None)
    padrows = (d["labels"] == pad)
    assert padrows.any()
    assert (losses.cpu()[padrows] == 0).all() and (dx.cpu()[padrows] == 0).all()       # bit-exact zeros on padding
    # the gradients are O(1/V), far below the absolute tolerance: check them relatively as well
    big = dxo.abs() > 1e-4
    if big.any() and dtype != torch.float32:
        rel = ((dx.cpu().to(D) - dxo).abs() / dxo.abs())[big].max().item()
        assert rel < 2e-2, rel
    if (~padrows).any():
        rows = dx.cpu().to(D)[~padrows].sum(1).abs().max().item()
        assert rows < (1e-5 if dtype == torch.float32 else 5e-2)                        # each row sums to ~0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,v", [(128 * 74 // 8, 32320), (5, 7), (3, 1), (64, 250054 // 8 + 1), (17, 4099)])
def test_xentropy_shapes(dev, dtype, n, v):
    _xent_case(dev, n, v, dtype, 0.1, pad=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_xentropy_large_vocabulary(dev, dtype):
    _xent_case(dev, 64, 256000, dtype, 0.1, pad=1)
    _xent_case(dev, 24, 250054, dtype, 0.1, pad=1)         # row stride 500108 B: rows cycle through 4 alignments


@pytest.mark.parametrize("misalign", [1, 3, 5])
def test_xentropy_misaligned_base(dev, misalign):
    _xent_case(dev, 9, 1001, torch.bfloat16, 0.1, pad=0, misalign=misalign)


def test_xentropy_no_smoothing_and_module_parity(dev):
    _xent_case(dev, 40, 1000, torch.float32, 0.0, pad=3)
    # reference module contract: without padding_idx the rows are NOT zeroed (the wrapper does it)
    d = inputs.xentropy_inputs(32, 500, torch.float32, 0.1, padding_idx=1, pad_fraction=0.25, seed=52)
    losses, lse = xentropy_cuda.forward(d["logits"].to(dev), d["labels"].to(dev), 0.1, False)
    lo, _ = oxe.xentropy_fwd(d["logits"], d["labels"], 0.1, -100, D)
    assert_close(losses, lo, torch.float32, "unpadded losses", rtol=2e-5, atol=2e-5)
    h = xentropy_cuda.forward(d["logits"].half().to(dev), d["labels"].to(dev), 0.1, False)[1]
    assert h.dtype == torch.float16                           # lse in the input dtype unless half_to_float


def test_xentropy_autograd_function(dev):
    d = inputs.xentropy_inputs(48, 3000, torch.bfloat16, 0.1, padding_idx=1, pad_fraction=0.2, seed=53)
    x = d["logits"].to(dev).requires_grad_()
    losses = SoftmaxCrossEntropyLoss.apply(x, d["labels"].to(dev), 0.1, 1, True)
    losses.sum().backward()
    lo, lseo = oxe.xentropy_fwd(d["logits"], d["labels"], 0.1, 1, D)
    assert_close(losses, lo, torch.float32, "fn losses", rtol=2e-5, atol=2e-5)
    assert_close(x.grad, oxe.xentropy_bwd(torch.ones(48), d["logits"], lseo, d["labels"], 0.1, 1, D), torch.bfloat16, "fn grad")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,v", [(33, 4099), (7, 1), (5, 250054 // 4 + 3), (64, 32320)])
def test_xentropy_argmax_follows_torch_argmax_bit_for_bit(dev, dtype, n, v):
    # coarse values: every row holds its maximum several times, so the lowest-index rule decides (onmt/modules/loss.py:293-311
    # takes torch.argmax of the logits); rows 1 and 2 hold NaN, which torch.argmax treats as the largest value
    g = torch.Generator().manual_seed(41)
    logits = torch.randint(-4, 5, (n, v), generator=g).to(dtype)
    if n > 2 and v > 40:
        logits[1, 37] = float("nan")
        logits[2, 5] = float("nan")
        logits[2, 31] = float("nan")
        logits[0, :16] = float("-inf")
    labels = torch.randint(0, v, (n,), generator=g)
    x = logits.to(dev)
    losses, lse, best = xentropy_cuda.forward(x, labels.to(dev), 0.0, dtype != torch.float32, padding_idx=-1, want_argmax=True)
    assert best.dtype == torch.int64
    assert torch.equal(best.cpu(), torch.argmax(logits.float(), dim=1))
    assert torch.equal(best, torch.argmax(x, dim=1))
    plain, lse2 = xentropy_cuda.forward(x, labels.to(dev), 0.0, dtype != torch.float32, padding_idx=-1)
    assert torch.equal(plain.isnan(), losses.isnan()) and torch.equal(plain[~plain.isnan()], losses[~losses.isnan()])


@pytest.mark.parametrize("dtype", DTYPES)
def test_xentropy_leading_block_of_minus_infinity(dev, dtype):
    # a masked vocabulary block: lanes that have only seen -inf must not produce NaN (the reference takes the row maximum
    # first, xentropy_kernel.cu:382-474, so such a row has a finite loss there)
    n, v = 9, 5000
    d = inputs.xentropy_inputs(n, v, dtype, 0.0, padding_idx=1, pad_fraction=0.0, seed=43)
    logits = d["logits"].clone()
    logits[:, :2048] = float("-inf")
    logits[3, 2048:] = float("-inf")
    logits[3, 77] = 1.5                                       # one finite class inside the block
    labels = torch.randint(2048, v, (n,), generator=torch.Generator().manual_seed(44))
    labels[3] = 77
    losses, lse = xentropy_cuda.forward(logits.to(dev), labels.to(dev), 0.0, dtype != torch.float32, padding_idx=1)
    want, want_lse = oxe.xentropy_fwd(logits, labels, 0.0, 1, torch.float64)
    assert torch.isfinite(losses).all()
    assert_close(losses, want, torch.float32, "losses with a -inf block", rtol=2e-5, atol=2e-5)
    assert_close(lse.float(), want_lse, torch.float32, "lse with a -inf block", rtol=2e-5, atol=2e-5)
    grad = xentropy_cuda.backward(torch.ones(n, device=dev), logits.to(dev), lse, labels.to(dev), 0.0, padding_idx=1)
    assert (grad[:, :2048].cpu()[torch.arange(n) != 3] == 0).all()
    assert_close(grad, oxe.xentropy_bwd(torch.ones(n), logits, want_lse, labels, 0.0, 1, torch.float64), dtype, "gradient with a -inf block")


def test_xentropy_errors(dev):
    x = torch.randn(4, 10, device=dev)
    with pytest.raises(RuntimeError):
        xentropy_cuda.forward(x, torch.zeros(4, device=dev, dtype=torch.int32), 0.1, False)   # labels must be int64
    with pytest.raises(RuntimeError):
        xentropy_cuda.forward(x.view(2, 2, 10), torch.zeros(4, device=dev, dtype=torch.long), 0.1, False)
    with pytest.raises(RuntimeError):
        xentropy_cuda.forward(x, torch.zeros(5, device=dev, dtype=torch.long), 0.1, False)
    with pytest.raises(RuntimeError):
        xentropy_cuda.forward(x, torch.zeros(4, device=dev, dtype=torch.long), 0.1, True)     # half_to_float on fp32


@pytest.mark.parametrize("nbytes", [16, 4096 * 16 + 48, 1 << 20])
def test_streaming_probes_move_what_they_say(dev, nbytes):
    """The bench's streaming probes (nmtg_stream_probe) are kernels like any other: copy, fp32 add and per-block sums of a
    buffer whose size is not a multiple of a block's chunk (16 KiB) are exact (sums: small integers, exact in fp32)."""
    from nmtgminor_amd import _lib as L
    n = nbytes // 4
    g = torch.Generator().manual_seed(nbytes)
    a = torch.randint(-8, 9, (n,), generator=g).float().to(dev)
    b = torch.randint(-8, 9, (n,), generator=g).float().to(dev)
    out = torch.full((n + 4,), 7.0, device=dev)
    for mode, want in ((0, a), (1, a + b)):
        out.fill_(7.0)
        L.call("nmtg_stream_probe", L.ptr(a), L.ptr(b), L.ptr(out), L.i64(nbytes), L.i32(mode), L.stream_of(a))
        assert torch.equal(out[:n], want) and (out[n:] == 7.0).all()
    blocks = L.load().nmtg_stream_probe_blocks(L.i64(nbytes))
    assert blocks == (nbytes + 16383) // 16384
    sums = torch.full((blocks + 1,), 7.0, device=dev)
    L.call("nmtg_stream_probe", L.ptr(a), L.ptr(None), L.ptr(sums), L.i64(nbytes), L.i32(2), L.stream_of(a))
    pad = torch.zeros(blocks * 4096, device=dev)
    pad[:n] = a
    assert torch.equal(sums[:blocks], pad.view(blocks, 4096).sum(1)) and sums[blocks] == 7.0
    with pytest.raises(RuntimeError, match="multiple of 16"):
        L.call("nmtg_stream_probe", L.ptr(a), L.ptr(b), L.ptr(out), L.i64(24), L.i32(0), L.stream_of(a))
