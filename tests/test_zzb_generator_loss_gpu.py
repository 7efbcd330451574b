"""Output projection + label-smoothed cross-entropy in row chunks (no [N, V] logits tensor) against the unchunked pair
of operators it replaces and against the fp32 oracle.

What the reference computes here: Generator.forward (onmt/modules/base_seq2seq.py:26-47) then
CrossEntropyLossBase._compute_loss (onmt/modules/loss.py:60-109). Losses on rows whose label is the padding index are
exactly zero, and so are their gradients; the validation argmax is an index and is compared exactly.
"""
import pytest
import torch

from nmtgminor_amd.modules.generator_loss import GeneratorLoss, LinearSoftmaxCrossEntropy, linear_cross_entropy_eval
from nmtgminor_amd.modules.softmax_xentropy import SoftmaxCrossEntropyLoss
from nmtgminor_amd.native import linear_gemm
from oracle import generator_loss as og
from util import assert_close

pytestmark = pytest.mark.gpu
PAD = 1


def _case(n, e, v, dtype, bias, seed):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(n, e, generator=g).to(dtype)
    w = (torch.randn(v, e, generator=g) / e ** 0.5).to(dtype)
    b = (0.1 * torch.randn(v, generator=g)).to(dtype) if bias else None
    y = torch.randint(0, v, (n,), generator=g)
    y[torch.rand(n, generator=g) < 0.2] = PAD
    gl = torch.rand(n, generator=g) + 0.5
    return h, w, b, y, gl


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,e,v,chunk,bias,eps", [(80, 64, 1000, 32, True, 0.1),      # 32 + 32 + 16 rows
                                                  (64, 128, 517, 64, False, 0.0),     # one chunk, odd vocabulary
                                                  (33, 64, 2048, 8, True, 0.3)])      # ragged last chunk of one row
@pytest.mark.parametrize("kept", [True, False])
def test_chunked_projection_loss_matches_oracle_and_unchunked_operators(dev, dtype, n, e, v, chunk, bias, eps, kept):
    """kept: the logits fit the memory budget and stay for the backward (one projection, the gradient written over them);
    otherwise they are never whole (rows in chunks forward, class slices recomputed backward). Same oracle, same tolerance."""
    h, w, b, y, gl = _case(n, e, v, dtype, bias, 100 + n)
    hd, wd, yd, gd = h.to(dev).requires_grad_(), w.to(dev).requires_grad_(), y.to(dev), gl.to(dev)
    bd = b.to(dev).requires_grad_() if bias else None
    loss = LinearSoftmaxCrossEntropy.apply(hd, wd, bd, yd, eps, PAD, chunk, (16 << 30) if kept else 0)
    loss.backward(gd, retain_graph=kept)
    # the fp32 oracle with the logits rounded where the reference stores them
    want, _, _ = og.generator_loss_fwd(h, w, b, y, eps, PAD, dtype)
    dh, dw, db = og.generator_loss_bwd(gl, h, w, b, y, eps, PAD, dtype)
    assert loss.dtype == torch.float32
    assert_close(loss, want, dtype, "losses", atol=2e-3)
    assert_close(hd.grad, dh, dtype, "grad of the states")
    assert_close(wd.grad, dw, dtype, "grad of the weight", scale_atol=True)
    if bias:
        assert_close(bd.grad, db, dtype, "grad of the bias", scale_atol=True)
    pad = y == PAD
    assert pad.any() and (loss.cpu()[pad] == 0).all() and (hd.grad.cpu()[pad] == 0).all()     # exact zeros on padding
    if kept:
        # the first backward turned the kept logits into their gradient: a second one over the same graph recomputes
        first = [t.grad.clone() for t in (hd, wd)]
        hd.grad = wd.grad = None
        loss.backward(gd)
        assert_close(hd.grad, first[0].float().cpu(), dtype, "second backward, states")
        assert_close(wd.grad, first[1].float().cpu(), dtype, "second backward, weight", scale_atol=True)
    # the unchunked operators on the same device (the GEMM may pick another main loop for the dense, odd-pitched logits
    # tensor than for the 64-element-pitched chunk, so the two agree to rounding, not bit for bit)
    z = linear_gemm.gemm(h.to(dev), w.to(dev), trans_b=True, bias=None if b is None else b.to(dev))
    z.requires_grad_()
    ref = SoftmaxCrossEntropyLoss.apply(z, yd, eps, PAD, True)
    ref.backward(gd)
    assert_close(loss, ref.detach().cpu(), dtype, "losses against the unchunked operators", atol=2e-3)
    assert_close(hd.grad, linear_gemm.gemm(z.grad, w.to(dev)).float().cpu(), dtype, "grad of the states against the unchunked operators")


def test_per_row_weights_and_no_gradient_for_frozen_weights(dev):
    dtype = torch.bfloat16
    h, w, b, y, gl = _case(48, 64, 300, dtype, True, 7)
    gl[::3] = 0.0                                                     # rows switched off by their loss weight
    hd = h.to(dev).requires_grad_()
    wd, bd = w.to(dev), b.to(dev)                                     # frozen output layer
    loss = LinearSoftmaxCrossEntropy.apply(hd, wd, bd, y.to(dev), 0.1, PAD, 20)
    (loss * gl.to(dev)).sum().backward()
    dh, _, _ = og.generator_loss_bwd(gl, h, w, b, y, 0.1, PAD, dtype)
    assert_close(hd.grad, dh, dtype, "grad of the states")
    assert (hd.grad.cpu()[::3] == 0).all()


def test_validation_pass_counts_correct_predictions(dev):
    dtype = torch.float16
    h, w, b, y, _ = _case(70, 64, 900, dtype, True, 9)
    want, _, am = og.generator_loss_fwd(h, w, b, y, 0.0, PAD, dtype)
    y[:10] = am[:10]                                                  # some rows the model gets right
    y[3] = PAD
    want, _, am = og.generator_loss_fwd(h, w, b, y, 0.0, PAD, dtype)
    losses, preds = linear_cross_entropy_eval(h.to(dev), w.to(dev), b.to(dev), y.to(dev), PAD, 32)
    assert_close(losses, want, dtype, "validation losses", atol=2e-3)
    # an index: exact wherever the two best logits are not within rounding of each other
    z = (h.float() @ w.float().t() + b.float())
    top2 = z.topk(2, dim=1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2e-2 * top2[:, 0].abs().clamp_min(1.0)
    assert clear.sum() > 50 and torch.equal(preds.cpu()[clear], am[clear])
    mod = GeneratorLoss(64, 900, label_smoothing=0.1, padding_idx=PAD, chunk_rows=32).to(dev).to(dtype)
    with torch.no_grad():
        mod.linear.weight.copy_(w.to(dev))
        mod.linear.bias.copy_(b.to(dev))
    mod.eval()
    out = mod(h.to(dev).view(7, 10, 64), y.to(dev).view(7, 10), eval=True)
    real = y != PAD
    assert out["total"] == int(real.sum())
    assert out["correct"] == int(((preds.cpu() == y) & real).sum()) and out["correct"] >= 9
    assert abs(out["data"] - float(want.sum())) < 2e-2 * float(want.sum())


def test_module_matches_the_reference_loss_assembly(dev):
    dtype = torch.bfloat16
    h, w, b, y, gl = _case(60, 64, 400, dtype, True, 11)
    mod = GeneratorLoss(64, 400, label_smoothing=0.1, padding_idx=PAD, chunk_rows=25).to(dev).to(dtype)
    with torch.no_grad():
        mod.linear.weight.copy_(w.to(dev))
        mod.linear.bias.copy_(b.to(dev))
    mod.train()
    hd = h.to(dev).view(6, 10, 64).requires_grad_()
    out = mod(hd, y.to(dev).view(6, 10), loss_weights=gl.to(dev).view(6, 10), loss_constraint=0.25)
    out["loss"].backward()
    rows, _, _ = og.generator_loss_fwd(h, w, b, y, 0.1, PAD, dtype)
    real = (y != PAD).float()
    want = ((rows - 0.25 * real) * gl).sum()
    assert abs(float(out["loss"].detach()) - float(want)) < 2e-2 * abs(float(want))
    assert abs(out["data"] - float(rows.sum())) < 2e-2 * float(rows.sum())
    dh, dw, db = og.generator_loss_bwd(gl, h, w, b, y, 0.1, PAD, dtype)
    assert_close(hd.grad.view(60, 64), dh, dtype, "grad of the states")
    assert_close(mod.linear.weight.grad, dw, dtype, "grad of the weight", scale_atol=True)
    assert_close(mod.linear.bias.grad, db, dtype, "grad of the bias", scale_atol=True)
    # label smoothing is a training-time setting (onmt/modules/loss.py:74)
    mod.eval()
    plain = mod(h.to(dev), y.to(dev))
    rows0, _, _ = og.generator_loss_fwd(h, w, b, y, 0.0, PAD, dtype)
    assert abs(plain["data"] - float(rows0.sum())) < 2e-2 * float(rows0.sum())


def test_argument_checks_and_empty_batch(dev):
    h, w, b, y, _ = _case(8, 64, 100, torch.float16, True, 13)
    with pytest.raises(RuntimeError):
        LinearSoftmaxCrossEntropy.apply(h.to(dev), w.to(dev)[:, :32], None, y.to(dev))           # model dimensions differ
    with pytest.raises(RuntimeError):
        LinearSoftmaxCrossEntropy.apply(h.to(dev), w.to(dev), None, y.to(dev).int())             # labels must be int64
    with pytest.raises(RuntimeError):
        LinearSoftmaxCrossEntropy.apply(h.to(dev), w.to(dev).float(), None, y.to(dev))           # one dtype
    with pytest.raises(RuntimeError):
        LinearSoftmaxCrossEntropy.apply(h.to(dev), w.to(dev), None, y.to(dev), 0.0, PAD, 0)      # chunk_rows
    hd = h.to(dev)[:0].requires_grad_()
    wd = w.to(dev).requires_grad_()
    loss = LinearSoftmaxCrossEntropy.apply(hd, wd, None, y.to(dev)[:0], 0.1, PAD, 4)
    assert loss.shape == (0,)
    loss.sum().backward()
    assert hd.grad.shape == (0, 64) and float(wd.grad.abs().sum()) == 0.0
