"""Fused-MLP autograd functions on the HIP kernels.

Mirrors onmt/modules/mlp/mlp.py:55-211 of the reference: MlpReluFunction, MlpSiluFunction,
MlpGELUFunction, MlpAGELUFunction with forward(ctx, p, recompute, *args) where
args = (x, W_1..W_n, b_1..b_n), and the callables mlp_relu_function, mlp_silu_function,
mlp_gelu_function, mlp_agelu_function (autocast-aware). An optional keyword `mask=` on the
callables replays an explicit dropout keep-mask (the reference draws its own)."""
import torch

from ..native import fused_mlp_agelu, fused_mlp_gelu, fused_mlp_relu, fused_mlp_silu, mlp_gelu_blaslt
from ._autocast import cast_if_autocast_enabled, no_autocast


class MlpReluFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, p, recompute, mask, *args):
        output = fused_mlp_relu.forward(p, recompute, args, mask)
        ctx.save_for_backward(*args)
        ctx.recompute = recompute
        if not recompute:
            ctx.outputs = output
            ctx.dropout_mask = None
        else:
            ctx.dropout_mask = output[-1]
            ctx.outputs = None
        ctx.p = p
        return output[0]

    @staticmethod
    def backward(ctx, *grad_o):
        p = ctx.p
        if not ctx.recompute:
            grads = fused_mlp_relu.backward(p, grad_o[0], ctx.outputs, ctx.saved_tensors)
            del ctx.outputs
        else:
            grads = fused_mlp_relu.backward_recompute(p, grad_o[0], ctx.dropout_mask, ctx.saved_tensors)
            del ctx.dropout_mask
        return (None, None, None, *grads)


def _make(native, name):
    class _Fn(torch.autograd.Function):
        @staticmethod
        def forward(ctx, p, recompute, mask, *args):
            output = native.forward(p, args, mask)
            ctx.save_for_backward(*args)
            ctx.outputs = output
            ctx.p = p
            return output[0]

        @staticmethod
        def backward(ctx, *grad_o):
            grads = native.backward(ctx.p, grad_o[0], ctx.outputs, ctx.saved_tensors)
            del ctx.outputs
            return (None, None, None, *grads)

    _Fn.__name__ = _Fn.__qualname__ = name
    return _Fn


MlpSiluFunction = _make(fused_mlp_silu, "MlpSiluFunction")
MlpAGELUFunction = _make(fused_mlp_agelu, "MlpAGELUFunction")


class MlpGELUFunction(torch.autograd.Function):
    """forward(ctx, p, recompute, mask, *args); with recompute only (out, mask) are kept and the
    activations are rebuilt in the backward (mlp_gelu_blaslt contract,
    onmt/modules/mlp/mlp.py:127-173)."""

    @staticmethod
    def forward(ctx, p, recompute, mask, *args):
        output = mlp_gelu_blaslt.forward(p, args, mask)
        ctx.outputs = (output[0], output[-1]) if recompute else output
        ctx.save_for_backward(*args)
        ctx.p = p
        ctx.recompute = recompute
        ctx.requires_grad_weight = args[1].requires_grad
        return output[0]

    @staticmethod
    def backward(ctx, *grad_o):
        p, recompute = ctx.p, ctx.recompute
        if ctx.requires_grad_weight:
            grads = mlp_gelu_blaslt.backward(p, recompute, grad_o[0], ctx.outputs, ctx.saved_tensors)
        else:
            outputs = ctx.outputs
            if recompute:
                outputs = mlp_gelu_blaslt.forward(p, ctx.saved_tensors, outputs[-1] if p > 0.0 else None)
            grads = mlp_gelu_blaslt.backward_input_only(p, grad_o[0], outputs, ctx.saved_tensors)
            grads = grads + [None] * (len(ctx.saved_tensors) - 1)
        del ctx.outputs
        return (None, None, None, *grads)


def _callable(fn):
    def call(p, recompute, *args, mask=None):
        args = cast_if_autocast_enabled(*args)
        with no_autocast():
            return fn.apply(p, recompute, mask, *args)
    return call


mlp_relu_function = _callable(MlpReluFunction)
mlp_silu_function = _callable(MlpSiluFunction)
mlp_gelu_function = _callable(MlpGELUFunction)
mlp_agelu_function = _callable(MlpAGELUFunction)
