"""LayerNorm oracle. Reference: fallback F.layer_norm(x, (H,), gamma, beta, eps)
(onmt/modules/layer_norm.py:111-119,157-168); saved statistics mu / rsigma as the native module
returns them (onmt/modules/extensions/layer_norm/ln_api.cpp:80-153); closed-form backward as the
reference's own test states it (onmt/modules/test_layer_norm.py:53-72)."""
import torch


def ln_fwd(x, gamma, beta, eps, ctype=torch.float32):
    """x [rows, H] -> (z, mu [rows], rsigma [rows]); biased variance, as F.layer_norm."""
    x = x.to(ctype)
    g = gamma.to(ctype)
    b = beta.to(ctype)
    mu = x.mean(dim=1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=1, keepdim=True)
    rsigma = 1.0 / torch.sqrt(var + eps)
    z = (x - mu) * rsigma * g + b
    return z, mu.squeeze(1), rsigma.squeeze(1)


def ln_bwd(dz, x, mu, rsigma, gamma, ctype=torch.float32):
    """-> (dx, dgamma, dbeta) given the saved row statistics."""
    dz = dz.to(ctype)
    x = x.to(ctype)
    g = gamma.to(ctype)
    mu = mu.to(ctype).unsqueeze(1)
    rs = rsigma.to(ctype).unsqueeze(1)
    y = rs * (x - mu)
    dbeta = dz.sum(0)
    dgamma = (dz * y).sum(0)
    dy = dz * g
    mdy = dy.mean(1, keepdim=True)
    mdyy = (dy * y).mean(1, keepdim=True)
    dx = rs * (dy - mdyy * y - mdy)
    return dx, dgamma, dbeta


def ln_bwd_memory_efficient(dz, z, rsigma, gamma, beta, ctype=torch.float32):
    """Backward from the saved OUTPUT: y = (z - beta) / gamma
    (onmt/modules/extensions/layer_norm/ln_bwd_kernels.cuh:91-110)."""
    dz = dz.to(ctype)
    g = gamma.to(ctype)
    y = (z.to(ctype) - beta.to(ctype)) / g
    rs = rsigma.to(ctype).unsqueeze(1)
    dbeta = dz.sum(0)
    dgamma = (dz * y).sum(0)
    dy = dz * g
    mdy = dy.mean(1, keepdim=True)
    mdyy = (dy * y).mean(1, keepdim=True)
    dx = rs * (dy - mdyy * y - mdy)
    return dx, dgamma, dbeta
