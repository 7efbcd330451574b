"""The multi-tensor optimizer passes (Adam / AdamW update, scale with overflow flag, L2 norm) against the oracle
(oracle/fused_optim.py) and FusedAdam against torch.optim.AdamW stepping a copy of the same parameters.

What the reference computes here: fused_optim.multi_tensor_adam / multi_tensor_scale / multi_tensor_axpby /
multi_tensor_l2norm / multi_tensor_l2norm_scale
(onmt/modules/extensions/fused_optim/frontend.cpp:45-53) under FusedAdam.step (onmt/modules/optimized/fused_adam.py:113-191).
fp32 to 1e-5 relative; 16-bit parameters to the 16-bit tolerance (one rounding of p, m, v per step); the overflow flag and
which elements change are exact.
"""
import random

import pytest
import torch

from nmtgminor_amd.modules.fused_adam import FusedAdam, multi_tensor_applier
from nmtgminor_amd.modules.fused_clip_norm import fused_clip_grad_norm
from nmtgminor_amd.native import fused_optim
from oracle import fused_optim as ofo
from util import assert_close, load_golden

pytestmark = pytest.mark.gpu
D = torch.float64
# sizes around the 16-byte vector width, around one 8192-element chunk, an empty tensor, and more tensors than any
# launch's table holds (84 to 160, by the number of lists)
SIZES = [1, 7, 64, 1000, 65536, 65537, 0, 200003, 8191, 8192, 8193] + [33 + i for i in range(170)]


def _tensors(sizes, dtype, seed, scale=1.0, positive=False):
    g = torch.Generator().manual_seed(seed)
    out = []
    for n in sizes:
        t = scale * torch.randn(n, generator=g)
        out.append((t.abs() if positive else t).to(dtype))
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mode,bias_correction,wd", [(1, 1, 0.01), (0, 1, 0.01), (1, 0, 0.0)])
def test_adam_update_of_a_list_of_tensors(dev, dtype, mode, bias_correction, wd):
    sizes = SIZES if dtype == torch.float32 else SIZES[:8] + SIZES[8:12]
    g, p = _tensors(sizes, dtype, 1), _tensors(sizes, dtype, 2)
    m, v = _tensors(sizes, dtype, 3, 0.1), _tensors(sizes, dtype, 4, 0.01, positive=True)
    gd, pd, md, vd = ([t.to(dev) for t in lst] for lst in (g, p, m, v))
    misaligned = torch.zeros(1001, dtype=dtype, device=dev)[1:]                  # a tensor that starts off a 16-byte boundary
    gd.append(torch.ones_like(misaligned)); pd.append(misaligned); md.append(torch.zeros_like(misaligned)); vd.append(torch.zeros_like(misaligned))
    g.append(torch.ones(1000, dtype=dtype)); p.append(torch.zeros(1000, dtype=dtype)); m.append(torch.zeros(1000, dtype=dtype)); v.append(torch.zeros(1000, dtype=dtype))
    g_before = [t.clone() for t in gd]
    multi_tensor_applier(fused_optim.multi_tensor_adam, None, [gd, pd, md, vd], 3e-3, 0.9, 0.98, 1e-8, 3, mode, bias_correction, wd)
    for i in range(len(g)):
        want = ofo.adam_step(g[i], p[i], m[i], v[i], 3e-3, 0.9, 0.98, 1e-8, 3, mode, bool(bias_correction), wd, D)
        for got, exp, what in zip((pd[i], md[i], vd[i]), want, ("p", "m", "v")):
            assert_close(got, exp, dtype, f"{what} of tensor {i} ({g[i].numel()} elements)", atol=1e-6 if dtype == torch.float32 else None)
        assert torch.equal(gd[i], g_before[i])                                     # gradients are read only


def test_adam_argument_checks(dev):
    t = lambda n=8: torch.zeros(n, device=dev)
    with pytest.raises(RuntimeError):
        fused_optim.multi_tensor_adam(0, None, [[t()], [t()], [t()]], 1e-3, 0.9, 0.99, 1e-8, 1, 1, 1, 0.0)          # three lists
    with pytest.raises(RuntimeError):
        fused_optim.multi_tensor_adam(0, None, [[t()], [t(9)], [t()], [t()]], 1e-3, 0.9, 0.99, 1e-8, 1, 1, 1, 0.0)  # sizes differ
    with pytest.raises(RuntimeError):
        fused_optim.multi_tensor_adam(0, None, [[t()], [t()], [t()], [t()]], 1e-3, 0.9, 0.99, 1e-8, 0, 1, 1, 0.0)   # step 0
    with pytest.raises(RuntimeError):
        fused_optim.multi_tensor_adam(0, None, [[t()], [t().half()], [t()], [t()]], 1e-3, 0.9, 0.99, 1e-8, 1, 1, 1, 0.0)
    fused_optim.multi_tensor_adam(0, None, [[], [], [], []], 1e-3, 0.9, 0.99, 1e-8, 1, 1, 1, 0.0)                    # nothing to do


@pytest.mark.parametrize("src,dst", [(torch.float32, torch.float32), (torch.float16, torch.float32), (torch.float32, torch.bfloat16),
                                     (torch.bfloat16, torch.bfloat16)])
def test_scale_with_overflow_flag(dev, src, dst):
    xs = _tensors(SIZES[:12], src, 5)
    xd = [t.to(dev) for t in xs]
    out = [torch.full((t.numel(),), 7, dtype=dst, device=dev) for t in xs]
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    multi_tensor_applier(fused_optim.multi_tensor_scale, flag, [xd, out], 0.125)
    assert int(flag.item()) == 0
    for o, x in zip(out, xs):
        assert torch.equal(o.cpu(), (x.float() * 0.125).to(dst))                  # a power of two: exact in every dtype
    for poison, where in ((float("inf"), (4, 65535)), (float("nan"), (5, 65536)), (float("-inf"), (1, 6))):
        flag.zero_()
        bad = [t.clone() for t in xd]
        bad[where[0]][where[1]] = poison
        multi_tensor_applier(fused_optim.multi_tensor_scale, flag, [bad, out], 2.0)
        assert int(flag.item()) == 1, (poison, where)
    flag.fill_(1)                                                                  # a raised flag is never lowered
    multi_tensor_applier(fused_optim.multi_tensor_scale, flag, [xd, out], 2.0)
    assert int(flag.item()) == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_l2norm_of_a_list_of_tensors(dev, dtype):
    xs = _tensors(SIZES, dtype, 6)
    xd = [t.to(dev) for t in xs]
    total, each = multi_tensor_applier(fused_optim.multi_tensor_l2norm, None, [xd], True)
    want_total, want_each = ofo.l2norm(xs, D)
    assert total.dtype == torch.float32 and total.shape == (1,) and each.shape == (len(xs),)
    assert_close(total[0], want_total, torch.float32, "norm", rtol=2e-6)
    assert_close(each, want_each, torch.float32, "per-tensor norms", rtol=2e-6)
    again, none = multi_tensor_applier(fused_optim.multi_tensor_l2norm, None, [xd], False)
    assert torch.equal(again, total) and none.numel() == 0                         # deterministic: bit-identical on a second pass
    zero, _ = fused_optim.multi_tensor_l2norm(0, torch.zeros(1, dtype=torch.int32, device=dev), [[]], False)
    assert float(zero.item()) == 0.0


@pytest.mark.parametrize("xdt,odt", [(torch.float32, torch.float32), (torch.float16, torch.float32), (torch.bfloat16, torch.bfloat16)])
def test_axpby_with_overflow_check(dev, xdt, odt):
    xs, ys = _tensors(SIZES[:12], xdt, 11), _tensors(SIZES[:12], odt, 12)
    xd, yd = [t.to(dev) for t in xs], [t.to(dev) for t in ys]
    out = [torch.empty(t.numel(), dtype=odt, device=dev) for t in xs]
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    multi_tensor_applier(fused_optim.multi_tensor_axpby, flag, [xd, yd, out], 0.5, -2.0, -1)
    assert int(flag.item()) == 0
    for o, x, y in zip(out, xs, ys):
        assert_close(o, 0.5 * x.to(D) - 2.0 * y.to(D), odt, "a x + b y", atol=1e-6 if odt == torch.float32 else None)
    bad_x = [t.clone() for t in xd]
    bad_x[4][65535] = float("nan")
    for check, want in ((-1, 1), (0, 1), (1, 0)):                       # the flag follows the operand that is checked
        flag.zero_()
        multi_tensor_applier(fused_optim.multi_tensor_axpby, flag, [bad_x, yd, out], 1.0, 1.0, check)
        assert int(flag.item()) == want, check
    with pytest.raises(RuntimeError):
        fused_optim.multi_tensor_axpby(0, flag, [xd, yd, out], 1.0, 1.0, 2)


@pytest.mark.parametrize("src,dst", [(torch.float32, torch.float32), (torch.float16, torch.float32), (torch.bfloat16, torch.bfloat16)])
def test_l2norm_with_scaling_in_one_pass(dev, src, dst):
    xs = _tensors(SIZES[:12], src, 13)
    xd = [t.to(dev) for t in xs]
    out = [torch.empty(t.numel(), dtype=dst, device=dev) for t in xs]
    total, each = multi_tensor_applier(fused_optim.multi_tensor_l2norm_scale, None, [xd, out], 0.25, True)
    want_total, want_each = ofo.l2norm(xs, D)                           # the norm of the inputs before scaling
    assert_close(total[0], want_total, torch.float32, "norm", rtol=2e-6)
    assert_close(each, want_each, torch.float32, "per-tensor norms", rtol=2e-6)
    for o, x in zip(out, xs):
        assert torch.equal(o.cpu(), (x.float() * 0.25).to(dst))
    same, _ = multi_tensor_applier(fused_optim.multi_tensor_l2norm, None, [xd], False)
    assert torch.equal(same, total)                                     # the same partial sums as the plain norm pass


@pytest.mark.parametrize("dtype,adam_w", [(torch.float32, True), (torch.float32, False), (torch.bfloat16, True)])
def test_fused_adam_follows_torch_adamw(dev, dtype, adam_w):
    torch.manual_seed(8)
    shapes = [(64, 32), (32,), (7, 5, 3), (1,), (300, 129)]
    ref = [torch.randn(s, dtype=D).requires_grad_() for s in shapes]
    ours = [r.detach().to(dtype).to(dev).requires_grad_() for r in ref]
    for r, o in zip(ref, ours):
        r.data.copy_(o.detach().cpu().to(D))                                       # start from the rounded values
    kw = dict(lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.05)
    opt_ref = (torch.optim.AdamW if adam_w else torch.optim.Adam)(ref, **kw)
    opt = FusedAdam(ours, adam_w_mode=adam_w, **kw)
    g = torch.Generator().manual_seed(9)
    for _ in range(4):
        for r, o in zip(ref, ours):
            grad = torch.randn(r.shape, generator=g)
            r.grad, o.grad = grad.to(D), grad.to(dtype).to(dev)
        if dtype != torch.float32:
            for r, o in zip(ref, ours):
                r.grad = o.grad.detach().cpu().to(D)
        opt_ref.step()
        opt.step()
        opt.zero_grad()
        assert all(o.grad is None for o in ours)
    for i, (r, o) in enumerate(zip(ref, ours)):
        assert_close(o, r.detach(), dtype, f"parameter {i} after 4 steps", rtol=2e-5 if dtype == torch.float32 else 4e-2,
                     atol=1e-6 if dtype == torch.float32 else 4e-3)
    with pytest.raises(RuntimeError):
        FusedAdam(ours, amsgrad=True)


@pytest.mark.parametrize("max_norm", [0.5, 1e6, 0.0])
def test_clip_grad_norm_matches_torch(dev, max_norm):
    g = torch.Generator().manual_seed(10)
    shapes = [(40, 30), (30,), (3, 5, 7), (70000,)]
    ref = [torch.zeros(s).requires_grad_() for s in shapes]
    ours = [torch.zeros(s, device=dev).requires_grad_() for s in shapes[:3]] + [torch.zeros(shapes[3], device=dev).bfloat16().requires_grad_()]
    for r, o in zip(ref, ours):
        grad = torch.randn(r.shape, generator=g).to(o.dtype)
        r.grad, o.grad = grad.float(), grad.to(dev)
    frozen = torch.zeros(3, device=dev, requires_grad=True)                      # no gradient: skipped
    exact = torch.linalg.vector_norm(torch.cat([r.grad.flatten().to(D) for r in ref]))      # the norm in fp64
    want = torch.nn.utils.clip_grad_norm_(ref, max_norm) if max_norm > 0 else exact
    got = fused_clip_grad_norm(ours + [frozen], max_norm)
    assert_close(got, exact, torch.float32, "total norm", rtol=2e-6)
    assert_close(got, want, torch.float32, "total norm against torch's fp32 routine", rtol=1e-5)
    for i, (r, o) in enumerate(zip(ref, ours)):
        assert_close(o.grad, r.grad, o.dtype, f"clipped gradient {i}", rtol=1e-5 if o.dtype == torch.float32 else None)
    with pytest.raises(NotImplementedError):
        fused_clip_grad_norm(ours, 1.0, norm_type=1.0)
    assert float(fused_clip_grad_norm([frozen], 1.0)) == 0.0
    ours[0].grad[0, 0] = float("inf")
    with pytest.raises(RuntimeError):
        fused_clip_grad_norm(ours, 1.0, error_if_nonfinite=True)


@pytest.mark.parametrize("name,adam_w", [("adamw", True), ("adam", False)])
def test_fused_optim_golden_fixture(dev, name, adam_w):
    # tests/golden/fused_optim.npz: torch.optim.Adam / AdamW over four steps, clip_grad_norm_ on the last gradients
    F32 = torch.float32
    f = load_golden("fused_optim")
    ps = [f[f"p{i}"].to(F32).to(dev).requires_grad_() for i in range(3)]
    opt = FusedAdam(ps, lr=float(f["lr"]), betas=(float(f["beta1"]), float(f["beta2"])), eps=float(f["eps"]),
                    weight_decay=float(f["weight_decay"]), adam_w_mode=adam_w)
    for step in range(4):
        for i, p in enumerate(ps):
            p.grad = f[f"g{step}_{i}"].to(F32).to(dev)
        if step == 3 and adam_w:                                  # the last gradients, clipped on copies
            holders = [torch.zeros_like(p).requires_grad_() for p in ps]
            for h, p in zip(holders, ps):
                h.grad = p.grad.clone()
            norm = fused_clip_grad_norm(holders, float(f["max_norm"]))
            assert_close(norm, f["norm"], F32, "norm", rtol=2e-6)
            for i, h in enumerate(holders):
                assert_close(h.grad, f[f"clipped{i}"], F32, f"clipped gradient {i}")
        opt.step()
    for i, p in enumerate(ps):
        assert_close(p, f[f"{name}_p{i}"], F32, f"{name} p{i}", rtol=2e-5)
        assert_close(opt.state[p]["exp_avg"], f[f"{name}_m{i}"], F32, f"{name} m{i}", rtol=2e-5)
        assert_close(opt.state[p]["exp_avg_sq"], f[f"{name}_v{i}"], F32, f"{name} v{i}", rtol=2e-5)


@pytest.mark.parametrize("seed", range(3000, 3008))
def test_randomly_drawn_tensor_lists(dev, seed):
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.float32, torch.bfloat16, torch.float16])
    sizes = [rnd.choice([0, 1, 3, 8, 100, 4097, 8191, 8192, 8193, 70001]) for _ in range(rnd.choice([1, 2, 84, 85, 129, 161, 170]))]
    case = f"seed {seed}: {dtype}, {len(sizes)} tensors, {sum(sizes)} elements"
    g, p = _tensors(sizes, dtype, seed), _tensors(sizes, dtype, seed + 1)
    m, v = _tensors(sizes, dtype, seed + 2, 0.1), _tensors(sizes, dtype, seed + 3, 0.01, positive=True)
    gd, pd, md, vd = ([t.to(dev) for t in lst] for lst in (g, p, m, v))
    mode, step = rnd.choice([0, 1]), rnd.choice([1, 2, 10])
    fused_optim.multi_tensor_adam(0, None, [gd, pd, md, vd], 1e-2, 0.9, 0.99, 1e-8, step, mode, 1, 0.01)
    for i in rnd.sample(range(len(sizes)), min(6, len(sizes))):
        want = ofo.adam_step(g[i], p[i], m[i], v[i], 1e-2, 0.9, 0.99, 1e-8, step, mode, True, 0.01, D)
        for got, exp, what in zip((pd[i], md[i], vd[i]), want, "pmv"):
            assert_close(got, exp, dtype, f"{case}: {what} of tensor {i} ({sizes[i]})", atol=1e-6 if dtype == torch.float32 else None)
    total, each = fused_optim.multi_tensor_l2norm(0, None, [gd], True)
    want_total, want_each = ofo.l2norm(g, D)
    assert_close(total[0], want_total, torch.float32, case + ": norm", rtol=2e-6)
    assert_close(each, want_each, torch.float32, case + ": per-tensor norms", rtol=2e-6)
