"""Dropout + residual add oracle. Reference: FusedDropoutAdd
(onmt/modules/optimized/dropout_add.py:32-90): out = residual + x * mask / (1 - p);
eval or p == 0: out = x + residual; backward dx = g * mask / (1 - p), dresidual = g."""
import torch


def dropout_add_fwd(x, residual, mask, p, ctype=torch.float32):
    x = x.to(ctype)
    r = residual.to(ctype)
    if mask is None or p <= 0.0:
        return x + r
    return r + x * mask.to(ctype) / (1.0 - p)


def dropout_add_bwd(g, mask, p, ctype=torch.float32):
    g = g.to(ctype)
    if mask is None or p <= 0.0:
        return g, g
    return g * mask.to(ctype) / (1.0 - p), g
