"""Label-smoothed cross-entropy on the HIP kernels.

Mirrors SoftmaxCrossEntropyLoss of the reference (onmt/modules/optimized/softmax_xentropy.py:5-29;
same class in whisper/memory_efficient_whisper.py:17-48):
forward(logits, labels, smoothing=0.0, padding_idx=-100, half_to_float=False) -> losses [N] with
zeros where labels == padding_idx; backward returns the logits gradient. The padding handling
runs inside the kernels instead of the wrapper's two masked_fill_ passes."""
import torch

from ..native import xentropy_cuda as native


class SoftmaxCrossEntropyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, smoothing=0.0, padding_idx=-100, half_to_float=False):
        ctx.settings = (float(smoothing), int(padding_idx))
        per_row, lse = native.forward(logits, labels, ctx.settings[0], half_to_float, padding_idx=ctx.settings[1])
        ctx.save_for_backward(logits, lse, labels)
        return per_row

    @staticmethod
    def backward(ctx, upstream):
        eps, pad = ctx.settings
        logits, lse, labels = ctx.saved_tensors
        # rows whose label is the padding index come back as exact zeros from the kernel
        return native.backward(upstream.contiguous(), logits, lse, labels, eps, padding_idx=pad), None, None, None, None
