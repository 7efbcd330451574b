"""Autograd function of the gated activation + dropout kernel (nmtgminor_amd/native/glu_dropout.py)."""
import torch

from ..native import glu_dropout


class GatedActivationDropout(torch.autograd.Function):
    """(x [..., 2 * inner], activation name, p, is_training, mask or None) -> y [..., inner]."""

    @staticmethod
    def forward(ctx, x, act, p, is_training, mask=None):
        p = p if is_training else 0.0
        y, mask = glu_dropout.forward(x, act, p, mask)
        ctx.act, ctx.p = act, p
        ctx.save_for_backward(x, mask if mask is not None else torch.empty(0, dtype=torch.uint8, device=x.device))
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, mask = ctx.saved_tensors
        return glu_dropout.backward(grad_y, x, ctx.act, ctx.p, mask if mask.numel() else None), None, None, None, None


def gated_activation_dropout(x, act, p, is_training, mask=None):
    return GatedActivationDropout.apply(x, act, p, is_training, mask)
