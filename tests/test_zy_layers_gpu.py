"""Layer glue — PrePostProcessing, EncoderLayer, DecoderLayer — on the HIP operators against the layer oracle
(oracle/transformer_layers.py: the same composition in fp64, gradients by autograd).

The layers draw their own dropout masks, so value parity is checked with dropout off (evaluation mode, and
training mode with p = 0, which takes the training code paths); with dropout on, the checks are structural
(the fused dropout + add is exactly residual + keep * x / (1 - p), gradients are finite, the keep rate is right).
Composition follows onmt/models/transformer_layers.py:145-185, 283-343 and onmt/modules/pre_post_processing.py:53-82.
"""
from types import SimpleNamespace

import pytest
import torch

from nmtgminor_amd.modules.pre_post_processing import PrePostProcessing
from nmtgminor_amd.modules.transformer_layers import DecoderLayer, EncoderLayer
from oracle import inputs, layer_norm as oln, transformer_layers as otl
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64


# gelu throughout: relu's step derivative flips on pre-activations within rounding of zero, which moves whole rows of dx
# by more than any tolerance that would still catch a mistake (the relu kernels are checked per operator)
def options(**kw):
    base = dict(model_size=128, inner_size=256, n_heads=4, dropout=0.0, attn_dropout=0.0, variational_dropout=False,
                macaron=False, rezero=False, ffn_activation="gelu", ffn_glu=False, fast_self_attention=True,
                fast_xattention=True, fast_feed_forward=True, ignore_source=False)
    base.update(kw)
    return SimpleNamespace(**base)


def randomise(module, seed):
    """Every parameter away from its initial value (biases 0, LayerNorm 1 hide mistakes)."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for p in module.parameters():
            p.add_((0.1 if p.dim() == 1 else 0.02) * torch.randn(p.shape, generator=g))
    return module


def layer_close(actual, expected, dtype, what, summed=False):
    """The oracle rounds to `dtype` where the layer does (every operator boundary, the operators' stored tensors, the
    stored gradients), so nearly every element meets the comparison every 16-bit result gets: 2e-2 relative, 1e-3 of the
    largest magnitude absolute. What remains are last-place flips: where the fp32-accumulating kernel and the fp64 oracle
    land on opposite sides of a rounding boundary of an intermediate of magnitude M, a residual sum that cancels to a
    small value inherits one unit in the last place of M. Such elements are few (under 1 %) and bounded by one unit in
    the last place of the largest magnitude (eps * max); a wrong term or a missing rounding point shows as many elements,
    or as a larger error. summed: a parameter gradient, a sum over all tokens of such elements, so that a flip in any one
    of its hundred-odd terms shows in it: the bound alone."""
    a, e = actual.detach().to("cpu", D), expected.detach().to("cpu", D)
    peak = max(1.0, float(e.abs().max()))
    outside = ((a - e).abs() > 1e-3 * peak + 2e-2 * e.abs()).double().mean().item()
    assert summed or outside < 0.01, f"{what}: {100 * outside:.2f} % of the elements beyond the 16-bit tolerance"
    assert_close(actual, expected, dtype, what, atol=torch.finfo(dtype).eps * peak)


def attn_core(opt, training):
    """Which attention kernels the layer's self-attention runs, hence which rounding points the oracle models: the tiled
    core in training where it takes the head dimension, the extension's stored-tensor chain otherwise."""
    return "tiled" if training and opt.model_size // opt.n_heads in (64, 128) else "stored"


def params64(module):
    return {k: v.detach().cpu().to(D).requires_grad_() for k, v in module.state_dict().items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pre_post_processing_sequences(dev, dtype):
    g = torch.Generator().manual_seed(81)
    t, b, e = 12, 3, 128
    x = torch.randn(t, b, e, generator=g).to(dtype)
    r = torch.randn(t, b, e, generator=g).to(dtype)
    # "n": LayerNorm with the reference's state_dict keys
    n = randomise(PrePostProcessing(e, 0.1, sequence="n"), 82).to(dev).to(dtype)
    assert sorted(n.state_dict()) == ["layer_norm.function.bias", "layer_norm.function.weight"]
    want, _, _ = oln.ln_fwd(x.view(t * b, e), n.layer_norm.function.weight.cpu(), n.layer_norm.function.bias.cpu(), 1e-5, D)
    assert_close(n(x.to(dev)).view(t * b, e), want, dtype, "n")
    # "da" in evaluation mode: residual add only, and the input of the step is reused as the output buffer
    da = PrePostProcessing(e, 0.25, sequence="da").to(dev).eval()
    assert_close(da(x.to(dev), r.to(dev)), x.to(D) + r.to(D), dtype, "da eval")
    # "da" in training: out = residual + keep * x / (1 - p), keep rate 1 - p, gradient = keep / (1 - p)
    da.train()
    xin = x.to(dev).requires_grad_()
    rin = r.to(dev).requires_grad_()
    out = da(xin * 1.0, rin)
    out.sum().backward()
    keep = (xin.grad != 0)
    assert abs(keep.float().mean().item() - 0.75) < 0.03
    assert_close(xin.grad, keep.cpu().to(D) / 0.75, dtype, "da grad")
    assert torch.equal(rin.grad.cpu(), torch.ones_like(r))
    assert_close(out, r.to(D) + keep.cpu().to(D) * x.to(D) / 0.75, dtype, "da train")
    # "nda": the three steps chained; "z": ReZero starts as the identity on the residual
    nda = randomise(PrePostProcessing(e, 0.0, sequence="nda"), 83).to(dev).to(dtype).eval()
    want, _, _ = oln.ln_fwd(x.view(t * b, e), nda.layer_norm.function.weight.cpu(), nda.layer_norm.function.bias.cpu(), 1e-5, D)
    got = nda(x.to(dev), r.to(dev)).view(t * b, e)
    if dtype == torch.float32:
        assert_close(got, want + r.to(D).view(t * b, e), dtype, "nda")
    else:
        layer_close(got, want.to(dtype).to(D) + r.to(D).view(t * b, e), dtype, "nda")      # "n" stores its result in `dtype`
    z = PrePostProcessing(e, 0.0, sequence="z").to(dev)
    assert_close(z(x.to(dev), r.to(dev)), r.to(D), dtype, "z")
    # variational dropout: one mask per (batch, feature), shared over time
    v = PrePostProcessing(e, 0.5, sequence="d", variational=True).to(dev).train()
    y = v(torch.ones(t, b, e, device=dev))
    assert torch.equal(y[0], y[-1]) and set(y.unique().tolist()) <= {0.0, 2.0}
    # multilingual: the affine pair of language `factor`; the gradient lands in that row only
    ml = PrePostProcessing(e, 0.0, sequence="n", multilingual=True, n_languages=3)
    assert sorted(ml.state_dict()) == ["layer_norm.bias", "layer_norm.weight"] and ml.layer_norm.weight.shape == (3, e)
    ml = randomise(ml, 85).to(dev).to(dtype)
    factor = torch.tensor([2], device=dev)
    xin = x.to(dev).requires_grad_()
    out = ml(xin, factor=factor)
    dy = torch.randn(t, b, e, generator=g).to(dtype)
    out.backward(dy.to(dev))
    w, bb = ml.layer_norm.weight.detach().cpu(), ml.layer_norm.bias.detach().cpu()
    want, mu, rs = oln.ln_fwd(x.view(t * b, e), w[2], bb[2], 1e-5, D)
    dxo, dgo, dbo = oln.ln_bwd(dy.view(t * b, e), x.view(t * b, e), mu, rs, w[2], D)
    assert_close(out.view(t * b, e), want, dtype, "multilingual n")
    assert_close(xin.grad.view(t * b, e), dxo, dtype, "multilingual dx", atol=1e-5 if dtype == torch.float32 else None)
    assert_close(ml.layer_norm.weight.grad[2], dgo, dtype, "multilingual dgamma", scale_atol=True, atol=1e-5 if dtype == torch.float32 else None)
    assert_close(ml.layer_norm.bias.grad[2], dbo, dtype, "multilingual dbeta", scale_atol=True, atol=1e-5 if dtype == torch.float32 else None)
    assert (ml.layer_norm.weight.grad[:2] == 0).all() and (ml.layer_norm.bias.grad[:2] == 0).all()
    with pytest.raises(RuntimeError, match="factor"):
        ml(x.to(dev))


def _encoder_case(dev, dtype, macaron, training, death_rate=0.0, seed=84, **more):
    opt = options(macaron=macaron, **more)
    t, b = 40, 3
    g = torch.Generator().manual_seed(seed)
    layer = randomise(EncoderLayer(opt, death_rate=death_rate), seed + 1)
    p64 = params64(layer)
    layer = layer.to(dev).to(dtype).train(training)
    x = torch.randn(t, b, opt.model_size, generator=g).to(dtype)
    pad, _ = inputs.lengths_mask(b, t, t // 2, t, g)
    dy = torch.randn(t, b, opt.model_size, generator=g).to(dtype)
    xin = x.to(dev).requires_grad_()
    torch.manual_seed(0)                       # the stochastic-depth coin: rand(1) = 0.4963 >= death_rate 0.3 -> the layer runs
    y = layer(xin, pad.to(dev))
    y.backward(dy.to(dev))
    x64 = x.to(D).requires_grad_()
    p64r = {k: v.detach().to(dtype).to(D).requires_grad_() for k, v in p64.items()}     # the weights the kernels saw
    want = otl.encoder_layer(x64, p64r, opt.n_heads, pad, act="gelu", macaron=macaron, death_rate=death_rate, training=training,
                             round_to=dtype, attn_core=attn_core(opt, training))
    want.backward(dy.to(D))
    layer_close(y, want.detach(), dtype, "encoder output")
    layer_close(xin.grad, x64.grad, dtype, "encoder dx")
    for name, prm in layer.named_parameters():
        layer_close(prm.grad, p64r[name].grad, dtype, "d " + name, summed=True)
    return layer


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("macaron,training", [(False, False), (False, True), (True, True)])
def test_encoder_layer_matches_the_oracle(dev, dtype, macaron, training):
    layer = _encoder_case(dev, dtype, macaron, training)
    names = {"preprocess_attn.layer_norm.function.weight", "preprocess_attn.layer_norm.function.bias", "multihead.in_proj_weight",
             "multihead.out_proj_weight", "multihead.in_proj_bias", "multihead.out_proj_bias",
             "preprocess_ffn.layer_norm.function.weight", "preprocess_ffn.layer_norm.function.bias", "feedforward.in_proj_weight",
             "feedforward.out_proj_weight", "feedforward.in_proj_bias", "feedforward.out_proj_bias"}
    if macaron:
        names |= {"preprocess_mcr_ffn.layer_norm.function.weight", "preprocess_mcr_ffn.layer_norm.function.bias",
                  "mcr_feedforward.in_proj_weight", "mcr_feedforward.out_proj_weight", "mcr_feedforward.in_proj_bias",
                  "mcr_feedforward.out_proj_bias"}
    assert set(layer.state_dict()) == names


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_encoder_layer_with_head_dimension_64_drops_the_coverage_and_runs_the_tiled_core(dev, dtype, monkeypatch):
    """The layer drops the coverage, so in training its self-attention writes no [B*H, T, T] tensor where the tiled core
    takes the shape (head dimension 64 or 128; the other layer tests run heads of 32). Same oracle, same tolerance."""
    from nmtgminor_amd.native import flash_attn_cuda
    calls = []
    real = flash_attn_cuda.fwd_batched
    monkeypatch.setattr(flash_attn_cuda, "fwd_batched", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    _encoder_case(dev, dtype, False, True, model_size=256, inner_size=512, seed=86)
    assert calls == [1]


def test_encoder_layer_stochastic_depth(dev):
    # a surviving layer scales its branches by 1 / (1 - death_rate); a dropped layer is the identity
    _encoder_case(dev, torch.float16, False, True, death_rate=0.3)
    layer = EncoderLayer(options(), death_rate=1.0).to(dev).half().train()
    x = torch.randn(8, 2, 128, device=dev).half()
    assert torch.equal(layer(x, torch.zeros(2, 8, dtype=torch.bool, device=dev)), x)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ignore_source", [False, True])
def test_decoder_layer_matches_the_oracle(dev, dtype, ignore_source):
    _decoder_case(dev, dtype, ignore_source)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decoder_layer_with_head_dimension_64_runs_its_self_attention_on_the_tiled_core(dev, dtype, monkeypatch):
    """The layer drops the coverage of its self-attention (the cross-attention's is returned), so in training the time-masked
    self-attention writes no [B*H, T, T] tensor where the tiled core takes the shape. Same oracle, same tolerance."""
    from nmtgminor_amd.native import flash_attn_cuda
    calls = []
    real = flash_attn_cuda.fwd_batched
    monkeypatch.setattr(flash_attn_cuda, "fwd_batched", lambda *a, **k: (calls.append(k.get("time_mask") is not None), real(*a, **k))[1])
    _decoder_case(dev, dtype, False, model_size=256, inner_size=512)
    assert calls == [True]


def _decoder_case(dev, dtype, ignore_source, **more):
    opt = options(ignore_source=ignore_source, **more)
    tq, tk, b = 24, 50, 2
    g = torch.Generator().manual_seed(86)
    layer = randomise(DecoderLayer(opt), 87)
    p64 = params64(layer)
    layer = layer.to(dev).to(dtype).train()
    x = torch.randn(tq, b, opt.model_size, generator=g).to(dtype)
    ctxt = torch.randn(tk, b, opt.model_size, generator=g).to(dtype)
    src_pad, _ = inputs.lengths_mask(b, tk, tk // 2, tk, g)
    causal = torch.triu(torch.ones(tq, tq), 1).bool()
    dy = torch.randn(tq, b, opt.model_size, generator=g).to(dtype)
    xin, cin = x.to(dev).requires_grad_(), ctxt.to(dev).requires_grad_()
    y, coverage, cache = layer(xin, cin, causal.to(dev), src_pad.to(dev))
    y.backward(dy.to(dev))
    x64, c64 = x.to(D).requires_grad_(), ctxt.to(D).requires_grad_()
    p64r = {k: v.detach().to(dtype).to(D).requires_grad_() for k, v in p64.items()}
    want, cov = otl.decoder_layer(x64, c64, p64r, opt.n_heads, causal, src_pad, act="gelu", ignore_source=ignore_source, training=True,
                                  round_to=dtype, attn_core=attn_core(opt, True))
    want.backward(dy.to(D))
    layer_close(y, want.detach(), dtype, "decoder output")
    layer_close(xin.grad, x64.grad, dtype, "decoder dx")
    assert cache is None
    if ignore_source:
        assert coverage is None and cin.grad is None
        assert not any(n.startswith("multihead_src") or n.startswith("preprocess_src_attn") for n in layer.state_dict())
    else:
        layer_close(cin.grad, c64.grad, dtype, "decoder dcontext")
        assert_close(coverage, cov.detach(), dtype, "coverage")
    for name, prm in layer.named_parameters():
        layer_close(prm.grad, p64r[name].grad, dtype, "d " + name, summed=True)


def test_layers_with_dropout_and_unsupported_options(dev):
    opt = options(dropout=0.1, attn_dropout=0.1)
    layer = randomise(EncoderLayer(opt), 88).to(dev).bfloat16().train()
    x = torch.randn(32, 2, 128, device=dev).bfloat16().requires_grad_()
    pad = torch.zeros(2, 32, dtype=torch.bool, device=dev)
    torch.cuda.manual_seed(5)
    y1 = layer(x, pad)
    torch.cuda.manual_seed(5)
    y2 = layer(x, pad)
    y3 = layer(x, pad)
    assert torch.equal(y1, y2) and not torch.equal(y1, y3)          # masks follow the device generator
    y1.float().sum().backward()
    assert torch.isfinite(x.grad.float()).all() and all(torch.isfinite(p.grad.float()).all() for p in layer.parameters())
    assert not torch.equal(layer.eval()(x, pad), y1)
    # an inf in the outgoing stream is clamped to the largest finite value minus a margin (the reference's guard for
    # fp16 training); shown on a layer that stochastic depth skips, so that the stream is the input itself
    skipped = EncoderLayer(opt, death_rate=1.0).to(dev).half().train()
    bad = torch.ones(4, 2, 128, device=dev).half()
    bad[0, 0, 0], bad[1, 0, 0] = float("inf"), float("-inf")
    out = skipped(bad, pad[:, :4])
    assert out[0, 0, 0].item() == 65504.0 - 1000 + 8 and out[1, 0, 0].item() == -(65504.0 - 1000 + 8)   # fp16 spacing 32 at 64504
    assert torch.equal(out[2:], bad[2:])
    for field in ("fast_self_attention", "fast_feed_forward"):
        with pytest.raises(NotImplementedError):
            EncoderLayer(options(**{field: False}))
    with pytest.raises(NotImplementedError):
        DecoderLayer(options(fast_xattention=False))
    gated = EncoderLayer(options(ffn_glu=True)).to(dev).bfloat16().train()          # the gated feed-forward block is built and runs
    assert gated.feedforward.in_proj_weight.shape[0] == 2 * gated.feedforward.inner_size
    xg = x.detach().clone().requires_grad_()
    gated(xg, pad).float().sum().backward()
    assert torch.isfinite(xg.grad.float()).all()
