"""Label-smoothed cross-entropy on the HIP kernels.

Mirrors SoftmaxCrossEntropyLoss of the reference (onmt/modules/optimized/softmax_xentropy.py:5-29;
same class in whisper/memory_efficient_whisper.py:17-48):
forward(logits, labels, smoothing=0.0, padding_idx=-100, half_to_float=False) -> losses [N] with
zeros where labels == padding_idx; backward returns the logits gradient. The padding handling
runs inside the kernels instead of the wrapper's two masked_fill_ passes."""
import torch

from ..native import xentropy_cuda


class SoftmaxCrossEntropyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, smoothing=0.0, padding_idx=-100, half_to_float=False):
        losses, max_log_sum_exp = xentropy_cuda.forward(logits, labels, smoothing, half_to_float,
                                                        padding_idx=padding_idx)
        ctx.save_for_backward(logits, max_log_sum_exp, labels)
        ctx.smoothing = smoothing
        ctx.padding_idx = padding_idx
        return losses

    @staticmethod
    def backward(ctx, grad_loss):
        logits, max_log_sum_exp, labels = ctx.saved_tensors
        grad_logits = xentropy_cuda.backward(grad_loss.contiguous(), logits, max_log_sum_exp, labels,
                                             ctx.smoothing, padding_idx=ctx.padding_idx)
        return grad_logits, None, None, None, None
