"""Oracle for the multi-tensor optimizer passes (TEST INFRASTRUCTURE ONLY, like the rest of this package).

Restates the per-element arithmetic of the reference's AdamFunctor, ScaleFunctor and L2NormFunctor
(onmt/modules/extensions/fused_optim/multi_tensor_adam.cu:22-129 and :131-171 for the bias corrections,
multi_tensor_scale_kernel.cu:29-113, multi_tensor_l2norm_kernel.cu:27-110, :198-232) on whole tensors.
Pinned (tests/test_oracle_pins.py) against torch.optim.Adam and torch.optim.AdamW stepping the same parameters, against
torch.linalg.vector_norm, and against plain multiplication with torch.isfinite for the overflow flag."""
import torch


def adam_step(g, p, m, v, lr, beta1, beta2, eps, step, mode, bias_correction, weight_decay, ctype=torch.float32):
    """One update of one tensor -> (p, m, v) in ctype. mode 0: L2 regularisation, 1: decoupled weight decay."""
    g, p, m, v = (t.to(ctype) for t in (g, p, m, v))
    c1 = 1.0 - beta1 ** step if bias_correction else 1.0
    c2 = 1.0 - beta2 ** step if bias_correction else 1.0
    if mode == 0:
        g = g + weight_decay * p
    m = beta1 * m + (1.0 - beta1) * g
    v = beta2 * v + (1.0 - beta2) * g * g
    update = (m / c1) / (torch.sqrt(v / c2) + eps)
    if mode != 0:
        update = update + weight_decay * p
    return p - lr * update, m, v


def scale(x, factor, ctype=torch.float32):
    """-> (x * factor in ctype, whether any element of x is inf or NaN)."""
    x = x.to(ctype)
    return x * factor, not bool(torch.isfinite(x).all())


def l2norm(tensors, ctype=torch.float32):
    """-> (norm over all tensors, per-tensor norms [n]) in ctype."""
    each = torch.stack([(t.to(ctype) ** 2).sum() for t in tensors]) if tensors else torch.zeros(0, dtype=ctype)
    return each.sum().sqrt(), each.sqrt()
