"""Stand-in for the reference module `fast_layer_norm_cuda`
(onmt/modules/extensions/layer_norm/ln_api.cpp:80-257): ln_fwd, ln_bwd."""
import torch

from .. import _lib as L


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def ln_fwd(x, gamma, beta, epsilon):
    """x [rows, hidden] -> [z (weight dtype), mu fp32 [rows], rsigma fp32 [rows]]."""
    L.require_cuda(x, gamma, beta)
    _check(beta.dtype == gamma.dtype, "ln_fwd: beta and gamma dtypes differ")
    _check(x.is_contiguous(), "ln_fwd: x must be contiguous")
    _check(x.dim() == 2, "ln_fwd: x must be 2-D [rows, hidden]")
    rows, cols = x.shape
    _check(gamma.shape == beta.shape, "ln_fwd: gamma and beta shapes differ")
    _check(gamma.numel() == cols, "ln_fwd: hidden size mismatch")
    _check(epsilon >= 0.0, "ln_fwd: epsilon must be >= 0")
    gamma = gamma.contiguous()
    beta = beta.contiguous()
    z = torch.empty((rows, cols), dtype=gamma.dtype, device=x.device)
    mu = torch.empty((rows,), dtype=torch.float32, device=x.device)
    rsigma = torch.empty((rows,), dtype=torch.float32, device=x.device)
    L.call("nmtg_ln_fwd", L.ptr(x), L.ptr(gamma), L.ptr(beta), L.ptr(z), L.ptr(mu), L.ptr(rsigma),
           L.i64(rows), L.i64(cols), L.f32(epsilon), L.i32(L.dtype_code(x)), L.i32(L.dtype_code(gamma)),
           L.stream_of(x))
    return [z, mu, rsigma]


def ln_bwd(dz, x_or_z, mu, rsigma, gamma, beta=None, memory_efficient=False):
    """-> [dx, dgamma, dbeta, dgamma_part, dbeta_part] (partials fp32 [n_part, hidden])."""
    L.require_cuda(dz, x_or_z, mu, rsigma, gamma, beta)
    _check(dz.dtype == gamma.dtype, "ln_bwd: dz must have the weight dtype")
    _check(rsigma.dtype == torch.float32, "ln_bwd: rsigma must be fp32")
    _check(mu is None or mu.dtype == torch.float32, "ln_bwd: mu must be fp32")
    _check(beta is None or beta.dtype == gamma.dtype, "ln_bwd: beta must have the weight dtype")
    _check(x_or_z.is_contiguous() and dz.is_contiguous(), "ln_bwd: dz and x_or_z must be contiguous")
    _check(x_or_z.dim() == 2 and dz.shape == x_or_z.shape, "ln_bwd: dz and x_or_z must be 2-D and equal-shaped")
    rows, cols = x_or_z.shape
    _check(gamma.numel() == cols, "ln_bwd: hidden size mismatch")
    _check(beta is None or beta.numel() == cols, "ln_bwd: beta size mismatch")
    if memory_efficient:
        _check(beta is not None, "ln_bwd: memory_efficient needs beta")
    else:
        _check(mu is not None, "ln_bwd: mu is required unless memory_efficient")
    _check(rsigma.numel() == rows and (mu is None or mu.numel() == rows), "ln_bwd: mu/rsigma size mismatch")
    gamma = gamma.contiguous()
    beta = beta.contiguous() if beta is not None else None
    dx = torch.empty_like(x_or_z)
    dgamma = torch.empty_like(gamma)
    dbeta = torch.empty_like(gamma)
    n_part = int(L.load().nmtg_ln_bwd_parts(L.i64(rows), L.i64(cols)))
    dgamma_part = torch.empty((n_part, cols), dtype=torch.float32, device=x_or_z.device)
    dbeta_part = torch.empty((n_part, cols), dtype=torch.float32, device=x_or_z.device)
    L.call("nmtg_ln_bwd", L.ptr(dz), L.ptr(x_or_z), L.ptr(mu), L.ptr(rsigma), L.ptr(gamma), L.ptr(beta),
           L.ptr(dx), L.ptr(dgamma), L.ptr(dbeta), L.ptr(dgamma_part), L.ptr(dbeta_part), L.i64(n_part),
           L.i64(rows), L.i64(cols), L.i32(1 if memory_efficient else 0), L.i32(L.dtype_code(x_or_z)),
           L.i32(L.dtype_code(gamma)), L.stream_of(x_or_z))
    return [dx, dgamma, dbeta, dgamma_part, dbeta_part]
