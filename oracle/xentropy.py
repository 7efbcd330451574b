"""Label-smoothed softmax cross-entropy oracle.

Reference: SoftmaxCrossEntropyLoss (onmt/modules/optimized/softmax_xentropy.py:5-29) over
xentropy_cuda.forward / backward (onmt/modules/extensions/xentropy/xentropy_kernel.cu:382-474),
and the fallback it must agree with,
F.cross_entropy(logits.float(), y, ignore_index=pad, reduction='none', label_smoothing=eps)
(onmt/modules/loss.py:112-114).

  lse_i  = max_j x_ij + log sum_j exp(x_ij - max)
  loss_i = eps * (lse_i - mean_j x_ij) + (1 - eps) * (lse_i - x_{i,y_i});   0 where y_i == pad
  dx_ij  = g_i * (exp(x_ij - lse_i) - (1 - eps) [j == y_i] - eps / V);      0 where y_i == pad
"""
import torch


def xentropy_fwd(logits, labels, smoothing, padding_idx, ctype=torch.float32):
    """logits [N, V], labels int64 [N] -> (losses [N], lse [N])."""
    x = logits.to(ctype)
    mx = x.max(dim=1).values
    lse = mx + torch.log(torch.exp(x - mx.unsqueeze(1)).sum(dim=1))
    pad = labels == padding_idx
    safe = labels.clamp(0, x.shape[1] - 1)
    x_y = x.gather(1, safe.unsqueeze(1)).squeeze(1)
    loss = smoothing * (lse - x.mean(dim=1)) + (1.0 - smoothing) * (lse - x_y)
    loss = loss.masked_fill(pad, 0.0)
    return loss, lse


def xentropy_bwd(grad_loss, logits, lse, labels, smoothing, padding_idx, ctype=torch.float32):
    x = logits.to(ctype)
    n, v = x.shape
    g = grad_loss.to(ctype).masked_fill(labels == padding_idx, 0.0).unsqueeze(1)
    probs = torch.exp(x - lse.to(ctype).unsqueeze(1))
    onehot = torch.zeros_like(x)
    safe = labels.clamp(0, v - 1)
    onehot.scatter_(1, safe.unsqueeze(1), 1.0)
    return g * (probs - (1.0 - smoothing) * onehot - smoothing / v)
