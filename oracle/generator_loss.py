"""Output projection followed by the label-smoothed cross-entropy, as one function (oracle; test infrastructure).

Reference: Generator.forward (onmt/modules/base_seq2seq.py:26-47: logits = linear(hidden)) feeding
CrossEntropyLossBase._compute_loss (onmt/modules/loss.py:60-109: per-row losses of the logits, minus a constraint,
times optional per-row weights, summed). The reference materialises the logits in the model's dtype between the two;
`store_dtype` is that dtype (the logits and their gradient are rounded to it, everything else is `ctype`).

  logits  = round(hidden W^T + b)
  loss_i  = label-smoothed cross-entropy of row i (oracle/xentropy.py), 0 where the label is the padding index
  dlogits = round(g_i * (softmax - (1 - eps) onehot - eps / V))
  dhidden = dlogits W,   dW = dlogits^T hidden,   db = sum_i dlogits_i
"""
import torch

from . import xentropy


def _logits(hidden, weight, bias, store_dtype, ctype):
    z = hidden.to(ctype) @ weight.to(ctype).t()
    if bias is not None:
        z = z + bias.to(ctype)
    return z.to(store_dtype)


def generator_loss_fwd(hidden, weight, bias, labels, smoothing, padding_idx, store_dtype=torch.float32,
                       ctype=torch.float32):
    """hidden [N, E], weight [V, E], bias [V] or None, labels int64 [N] -> (losses [N], lse [N], argmax [N])."""
    z = _logits(hidden, weight, bias, store_dtype, ctype)
    loss, lse = xentropy.xentropy_fwd(z, labels, smoothing, padding_idx, ctype)
    return loss, lse, z.to(ctype).argmax(dim=1)


def generator_loss_bwd(grad_loss, hidden, weight, bias, labels, smoothing, padding_idx, store_dtype=torch.float32,
                       ctype=torch.float32):
    """-> (dhidden [N, E], dweight [V, E], dbias [V] or None), all in ctype."""
    z = _logits(hidden, weight, bias, store_dtype, ctype)
    _, lse = xentropy.xentropy_fwd(z, labels, smoothing, padding_idx, ctype)
    dz = xentropy.xentropy_bwd(grad_loss, z, lse, labels, smoothing, padding_idx, ctype).to(store_dtype).to(ctype)
    dh = dz @ weight.to(ctype)
    dw = dz.t() @ hidden.to(ctype)
    db = dz.sum(dim=0) if bias is not None else None
    return dh, dw, db
