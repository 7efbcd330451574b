"""Dropout + residual add on the HIP kernels.

Mirrors FusedDropoutAdd / fused_dropout_add of the reference
(onmt/modules/optimized/dropout_add.py:32-90): forward(input, residual, dropout_prob,
is_training); the result is written in place into `input`. The reference only takes its native
path for fp16; here fp32, fp16 and bf16 all do. An optional fifth argument replays an explicit
keep-mask."""
import torch

from ..native import fused_dropout_add_cuda
from ._autocast import cast_if_autocast_enabled, no_autocast


class FusedDropoutAdd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, residual, dropout_prob, is_training, mask=None):
        input = input.contiguous()
        residual = residual.contiguous()
        ctx.training = bool(is_training) and dropout_prob > 0.0
        ctx.p = dropout_prob
        dropout_mask, output = fused_dropout_add_cuda.forward(is_training, input, residual, dropout_prob, mask)
        if ctx.training:
            ctx.save_for_backward(dropout_mask)
        ctx.mark_dirty(input)
        return output

    @staticmethod
    def backward(ctx, output_grads):
        if not ctx.training:
            return output_grads, output_grads, None, None, None
        (dropout_mask,) = ctx.saved_tensors
        grad_input = fused_dropout_add_cuda.backward(output_grads, dropout_mask, ctx.p)
        return grad_input, output_grads, None, None, None


def fused_dropout_add(*args):
    args = cast_if_autocast_enabled(*args)
    with no_autocast():
        return FusedDropoutAdd.apply(*args)
