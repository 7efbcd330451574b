"""Linear layer on the MFMA GEMM with the reference's classes (onmt/modules/optimized/linear.py:25-73): LinearFunction
(forward / backward through the `linear_blaslt` stand-in, input gradient only when the weight is frozen), linear_function
(autocast handling) and Linear (an nn.Linear whose forward takes that path). fp16 / bf16 on the GPU; a missing bias takes
the same kernels without the bias epilogue (the reference hands that case to F.linear). What the GEMM does not cover (fp32
operands, CPU tensors) raises."""
import torch
from torch import Tensor

from ..native import linear_blaslt, linear_gemm
from ._autocast import cast_if_autocast_enabled, no_autocast


class LinearFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, bias):
        output = linear_blaslt.forward(input, weight, bias)
        ctx.save_for_backward(input, weight)
        ctx.has_bias = bias is not None
        return output

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if weight.requires_grad:
            if ctx.has_bias:
                return linear_blaslt.backward(input, weight, grad_output, True)
            g2, x2 = grad_output.reshape(-1, grad_output.size(-1)), input.reshape(-1, input.size(-1))
            return linear_gemm.gemm(g2, weight).view(input.shape), linear_gemm.gemm(g2, x2, trans_a=True), None
        return linear_blaslt.backward_input_only(input, weight, grad_output), None, None


def linear_function(input, weight, bias):
    input, weight, bias = cast_if_autocast_enabled(input, weight, bias)
    with no_autocast():
        return LinearFunction.apply(input, weight, bias)


class Linear(torch.nn.Linear):
    def forward(self, input: Tensor) -> Tensor:
        return linear_function(input, self.weight, self.bias)
