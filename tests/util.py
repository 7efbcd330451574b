"""Comparison helpers shared by the parity tests.

Tolerances (stated by the benchmark definition): fp32 1e-5 relative; fp16 / bf16 2e-2 relative
and 1e-3 absolute; integer / index / zero-on-padding results bit-exact.
"""
import os

import numpy as np
import torch

TOL = {
    torch.float32: dict(rtol=1e-5, atol=1e-6),
    torch.float16: dict(rtol=2e-2, atol=1e-3),
    torch.bfloat16: dict(rtol=2e-2, atol=1e-3),
}


def assert_close(actual, expected, dtype, what="", rtol=None, atol=None, scale_atol=False, flips=None):
    """actual: tensor from the HIP path (any device / dtype); expected: oracle (CPU, fp32/fp64).

    scale_atol: multiply the absolute tolerance by max|expected| — for reductions over thousands
    of terms (weight / bias gradients) whose magnitude is far above 1.
    flips: an absolute tolerance that at most one element in a thousand may use instead of `atol`. Two chains of the same
    16-bit roundings, one accumulating in fp32 and one in fp64, now and then land on opposite sides of a rounding boundary
    of an intermediate; a result that cancels to a small value then inherits that intermediate's unit in the last place.
    """
    if flips is not None:
        a = actual.detach().to("cpu", torch.float64)
        e = expected.detach().to("cpu", torch.float64)
        tol = dict(TOL[dtype])
        at = (tol["atol"] if atol is None else atol) * (max(1.0, float(e.abs().max())) if scale_atol else 1.0)
        outside = (a - e).abs() > at + (tol["rtol"] if rtol is None else rtol) * e.abs()
        assert outside.double().mean().item() <= 1e-3, f"{what}: {int(outside.sum())}/{outside.numel()} elements beyond atol={at}"
        atol = flips
    tol = dict(TOL[dtype])
    if rtol is not None:
        tol["rtol"] = rtol
    if atol is not None:
        tol["atol"] = atol
    a = actual.detach().to("cpu", torch.float64)
    e = expected.detach().to("cpu", torch.float64)
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    at = tol["atol"]
    if scale_atol:
        at = at * max(1.0, float(e.abs().max()))
    err = (a - e).abs()
    bound = at + tol["rtol"] * e.abs()
    bad = err > bound
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        worst = float((err - bound).max())
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.numel()} elements out of tolerance "
            f"(rtol={tol['rtol']}, atol={at}); first at {idx}: got {a[tuple(idx)].item()} "
            f"want {e[tuple(idx)].item()}; worst excess {worst}")


def rel_err(actual, expected):
    a = actual.detach().to("cpu", torch.float64)
    e = expected.detach().to("cpu", torch.float64)
    return float((a - e).norm() / e.norm().clamp_min(1e-30))


def load_golden(name):
    """A committed fixture tests/golden/<name>.npz as a dict of tensors (written by tests/golden/make_fixtures.py)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name + ".npz")
    with np.load(path, allow_pickle=False) as z:
        return {k: torch.from_numpy(np.array(z[k])) for k in z.files}
