"""LayerNorm parity: HIP kernels (through the C ABI) vs the CPU oracle on identical seeded inputs.

Mirrors the reference's test plan: forward / backward against the PyTorch result for several
hidden sizes and dtype pairs, plus the memory-efficient backward
(extensions/layer_norm/test_layer_norm.py:91-158,236-303; onmt/modules/test_layer_norm.py:130-240).
"""
import pytest
import torch

from nmtgminor_amd.modules.layer_norm import LayerNorm, fast_layer_norm_affine
from nmtgminor_amd.native import fast_layer_norm_cuda
from oracle import inputs, layer_norm as oln
from util import assert_close

pytestmark = pytest.mark.gpu

D = torch.float64


def _run(rows, hidden, dtype, wdtype, dev, memeff=False, seed=21):
    d = inputs.layer_norm_inputs(rows, hidden, dtype, wdtype, seed=seed)
    x, g, b, dy = (d[k].to(dev) for k in ("x", "gamma", "beta", "dy"))
    z, mu, rs = fast_layer_norm_cuda.ln_fwd(x, g, b, d["eps"])
    zo, muo, rso = oln.ln_fwd(d["x"], d["gamma"], d["beta"], d["eps"], D)
    assert z.dtype == wdtype and mu.dtype == torch.float32
    assert_close(z, zo, wdtype, "z")
    assert_close(mu, muo, torch.float32, "mu", atol=1e-6)
    assert_close(rs, rso, torch.float32, "rsigma")
    if memeff:
        dx, dg, db, dgp, dbp = fast_layer_norm_cuda.ln_bwd(dy, z, None, rs, g, b, True)
        dxo, dgo, dbo = oln.ln_bwd_memory_efficient(d["dy"], z.cpu(), rs.cpu(), d["gamma"], d["beta"], D)
    else:
        dx, dg, db, dgp, dbp = fast_layer_norm_cuda.ln_bwd(dy, x, mu, rs, g, None, False)
        dxo, dgo, dbo = oln.ln_bwd(d["dy"], d["x"], muo, rso, d["gamma"], D)
    assert dx.dtype == dtype and dg.dtype == wdtype
    assert dgp.shape[1] == hidden and dgp.dtype == torch.float32
    assert_close(dx, dxo, dtype, "dx", atol=1e-5 if dtype == torch.float32 else None)
    # column sums over `rows` terms: absolute error grows with sqrt(rows)
    assert_close(dg, dgo, wdtype, "dgamma", scale_atol=True, atol=1e-5 if wdtype == torch.float32 else None)
    assert_close(db, dbo, wdtype, "dbeta", scale_atol=True, atol=1e-5 if wdtype == torch.float32 else None)
    # the partial buffers are an output too: their column sums are the gradients
    assert_close(dgp.sum(0), dgo, torch.float32, "dgamma_part", scale_atol=True, atol=1e-5)
    assert_close(dbp.sum(0), dbo, torch.float32, "dbeta_part", scale_atol=True, atol=1e-5)


def test_workload_shape_fp32(dev):
    _run(4096, 512, torch.float32, torch.float32, dev, seed=1001)


@pytest.mark.parametrize("hidden", [64, 256, 768, 1024, 1280, 1536, 2048, 3072, 4096, 8192])
def test_hidden_sizes_fp32(dev, hidden):
    _run(257, hidden, torch.float32, torch.float32, dev)


@pytest.mark.parametrize("dtype,wdtype", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                          (torch.float16, torch.float32), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("hidden", [512, 1024, 4096, 16384])
def test_dtype_pairs(dev, dtype, wdtype, hidden):
    _run(130, hidden, dtype, wdtype, dev)


@pytest.mark.parametrize("hidden", [2, 3, 100, 513, 1000, 20000])
def test_odd_hidden_sizes_take_the_generic_kernel(dev, hidden):
    _run(37, hidden, torch.float32, torch.float32, dev)
    _run(37, hidden, torch.bfloat16, torch.bfloat16, dev)


@pytest.mark.parametrize("rows", [1, 2, 3, 5, 4097])
def test_ragged_row_counts(dev, rows):
    _run(rows, 512, torch.float32, torch.float32, dev)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [512, 1024, 8192])
def test_memory_efficient_backward(dev, dtype, hidden):
    _run(300, hidden, dtype, dtype, dev, memeff=True)


def test_empty_input(dev):
    x = torch.empty(0, 512, device=dev)
    g = torch.ones(512, device=dev)
    z, mu, rs = fast_layer_norm_cuda.ln_fwd(x, g, g, 1e-5)
    assert z.shape == (0, 512) and mu.numel() == 0
    dx, dg, db, _, _ = fast_layer_norm_cuda.ln_bwd(x, x, mu, rs, g, None, False)
    assert dx.shape == (0, 512) and (dg == 0).all() and (db == 0).all()


def test_argument_errors_raise(dev):
    g = torch.ones(512, device=dev)
    with pytest.raises(RuntimeError):
        fast_layer_norm_cuda.ln_fwd(torch.randn(4, 4, 512, device=dev), g, g, 1e-5)   # not 2-D
    with pytest.raises(RuntimeError):
        fast_layer_norm_cuda.ln_fwd(torch.randn(4, 256, device=dev), g, g, 1e-5)      # hidden mismatch
    with pytest.raises(RuntimeError):
        fast_layer_norm_cuda.ln_fwd(torch.randn(4, 1024, device=dev)[:, ::2], g, g, 1e-5)  # non-contiguous
    with pytest.raises(RuntimeError):
        fast_layer_norm_cuda.ln_fwd(torch.randn(4, 512, device=dev), g, g, -1.0)
    with pytest.raises(RuntimeError):
        fast_layer_norm_cuda.ln_fwd(torch.randn(4, 512), torch.ones(512), torch.ones(512), 1e-5)  # CPU tensors
    with pytest.raises(RuntimeError):
        fast_layer_norm_cuda.ln_fwd(torch.randn(4, 512, device=dev), g.half(), g.half(), 1e-5)  # fp32 x, fp16 w


def test_module_and_autograd(dev):
    d = inputs.layer_norm_inputs(96, 1024, torch.float32, seed=22)
    for me in (False, True):
        ln = LayerNorm(1024, memory_efficient=me).to(dev)
        with torch.no_grad():
            ln.weight.copy_(d["gamma"])
            ln.bias.copy_(d["beta"])
        x = d["x"].view(12, 8, 1024).to(dev).requires_grad_()
        y = ln(x)
        y.backward(d["dy"].view(12, 8, 1024).to(dev))
        zo, muo, rso = oln.ln_fwd(d["x"], d["gamma"], d["beta"], 1e-5, D)
        dxo, dgo, dbo = oln.ln_bwd(d["dy"], d["x"], muo, rso, d["gamma"], D)
        assert_close(y.view(96, 1024), zo, torch.float32, "module y")
        assert_close(x.grad.view(96, 1024), dxo, torch.float32, "module dx", atol=2e-5)
        assert_close(ln.weight.grad, dgo, torch.float32, "module dgamma", atol=2e-5, scale_atol=True)
        assert_close(ln.bias.grad, dbo, torch.float32, "module dbeta", atol=2e-5, scale_atol=True)
    assert sorted(n for n, _ in ln.named_parameters()) == ["bias", "weight"]


def test_autocast_casts_inputs(dev):
    d = inputs.layer_norm_inputs(64, 512, torch.float32, seed=23)
    x, g, b = (d[k].to(dev) for k in ("x", "gamma", "beta"))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = fast_layer_norm_affine(x, g, b, (512,), 1e-5)
    assert y.dtype == torch.bfloat16
    zo, _, _ = oln.ln_fwd(d["x"].bfloat16(), d["gamma"].bfloat16(), d["beta"].bfloat16(), 1e-5, D)
    assert_close(y, zo, torch.bfloat16, "autocast y")
