"""Empty inputs (a shard without sentences, a batch without rows): every operator returns empty results and zero
parameter gradients, or refuses exactly where the reference refuses (the cross-entropy: xentropy_kernel.cu:590, 659).
The autograd modules must also survive them, so that a training step over an empty shard is a no-op."""
import pytest
import torch

from nmtgminor_amd.modules.feed_forward import PositionWiseFeedForward
from nmtgminor_amd.modules.self_attention import SelfMultiheadAttn
from nmtgminor_amd.native import (encdec_multihead_attn_bias_blaslt as ed, fast_layer_norm_cuda as ln, fused_dropout_add_cuda as da,
                                  fused_mlp_gelu, mask_softmax_dropout_cuda as sm, self_multihead_attn_blaslt as sa, xentropy_cuda as xe)
from nmtgminor_amd.native.linear_gemm import gemm

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def test_attention_with_an_empty_batch_or_no_positions(dev):
    e, h = 128, 2
    r = lambda *s: torch.randn(*s).to(BF).to(dev)
    w_in, w_out, b_in, b_out = r(3 * e, e), r(e, e), r(3 * e), r(e)
    for t, b in ((0, 2), (5, 0)):
        x = r(t, b, e)
        lin, sc, dr, dm, ctx, out = sa.forward(False, True, h, x, w_in, w_out, b_in, b_out, None, 0.1)
        assert lin.shape == (t, b, 3 * e) and sc.shape == (b * h, t, t) and out.shape == (t, b, e)
        dx, dw_in, dw_out, db_in, db_out = sa.backward(False, h, out, ctx, dr, sc, lin, x, w_in, w_out, dm, 0.1)
        assert dx.shape == x.shape and not dw_in.any() and not dw_out.any() and not db_in.any() and not db_out.any()
    wq, wkv = r(e, e), r(2 * e, e)
    x_kv = r(7, 0, e)
    res = ed.forward(True, h, r(3, 0, e), x_kv, wq, wkv, w_out, None, None, None, None, 0.0)
    assert res[-1].shape == (3, 0, e)
    g = ed.backward(h, res[-1], res[5], res[3], res[2], res[0], res[1], r(3, 0, e), x_kv, wq, wkv, w_out, res[4], 0.0)
    assert g[0].shape == (3, 0, e) and g[1].shape == (7, 0, e) and not g[2].any() and not g[3].any() and not g[4].any()
    # one query position over one key is the smallest non-empty case
    res = ed.forward(False, h, r(1, 1, e), r(1, 1, e), wq, wkv, w_out, None, None, None, None, 0.0)
    assert torch.equal(res[3], torch.ones_like(res[3]))                   # a single key takes all the probability


def test_mlp_gemm_and_elementwise_with_empty_inputs(dev):
    e = 128
    r = lambda *s: (0.1 * torch.randn(*s)).to(BF).to(dev)
    x = r(0, e).requires_grad_()
    ins = [x, r(256, e), r(e, 256), r(256), r(e)]
    out = fused_mlp_gelu.forward(0.1, ins)
    assert out[0].shape == (0, e)
    g = fused_mlp_gelu.backward(0.1, r(0, e), out, ins)
    assert g[0].shape == (0, e) and [tuple(t.shape) for t in g[1:]] == [(256, e), (e, 256), (256,), (e,)] and not any(t.any() for t in g[1:])
    assert gemm(r(0, 64), r(32, 64), False, True).shape == (0, 32)
    bias = r(32)
    assert torch.equal(gemm(r(8, 0), r(32, 0), False, True, bias=bias), bias.expand(8, 32))     # an empty sum, plus the bias
    assert da.forward(True, r(0), r(0), 0.1)[1].numel() == 0 and da.backward(r(0), torch.zeros(0, dtype=torch.uint8, device=dev), 0.1).numel() == 0
    assert sm.forward(False, 1, r(0, 4, 16), 0.0)[2].shape == (0, 4, 16) and sm.forward(False, 1, r(2, 0, 16), 0.0)[2].shape == (2, 0, 16)
    z, mu, rs = ln.ln_fwd(torch.randn(0, 64, device=dev), torch.ones(64, device=dev), torch.zeros(64, device=dev), 1e-5)
    assert z.shape == (0, 64) and mu.numel() == 0
    labels = torch.zeros(0, dtype=torch.int64, device=dev)
    with pytest.raises(RuntimeError, match="should not be 0"):
        xe.forward(r(0, 100), labels, 0.1, True)
    with pytest.raises(RuntimeError, match="should not be 0"):
        xe.backward(torch.ones(0, device=dev), r(0, 100), torch.zeros(0, device=dev), labels, 0.1)


def test_modules_train_through_an_empty_batch(dev):
    attn = SelfMultiheadAttn(128, 2, 0.1).to(dev).to(BF).train()
    ffn = PositionWiseFeedForward(128, 256, 0.1, activation="gelu").to(dev).to(BF).train()
    x = torch.randn(6, 0, 128).to(BF).to(dev).requires_grad_()
    y, _ = attn(x, None, torch.zeros(0, 6, dtype=torch.bool, device=dev), None)
    z = ffn(y)
    z.float().sum().backward()
    assert x.grad.shape == x.shape
    for p in list(attn.parameters()) + list(ffn.parameters()):
        assert p.grad is not None and not p.grad.any()
