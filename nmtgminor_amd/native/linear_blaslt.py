"""Stand-in for the reference's extension module `linear_blaslt` (onmt/modules/extensions/mlp_blaslt/linear.cpp:21-56
forward, :59-104 backward, :142-144 bindings; Python face onmt/modules/optimized/linear.py:25-73): a linear layer
y = x W^T + b over the last dimension and its three gradients, on nmtg_gemm and nmtg_colsum."""
from . import linear_gemm


def forward(input, weight, bias):
    """input [..., in], weight [out, in], bias [out] -> [..., out]."""
    x2 = input.reshape(-1, input.size(-1))
    out = linear_gemm.gemm(x2, weight, trans_b=True, bias=bias)
    return out.view(*input.shape[:-1], weight.size(0))


def backward(input, weight, grad_output, compute_grad_input):
    """-> (d_input or None, d_weight [out, in], d_bias [out])."""
    x2 = input.reshape(-1, input.size(-1))
    g2 = grad_output.reshape(-1, grad_output.size(-1))
    d_weight = linear_gemm.gemm(g2, x2, trans_a=True)
    d_bias = linear_gemm.colsum(g2)
    d_input = linear_gemm.gemm(g2, weight).view(input.shape) if compute_grad_input else None
    return d_input, d_weight, d_bias


def backward_input_only(input, weight, grad_output):
    """-> d_input (the weight is frozen: no weight or bias gradient; linear.cpp:108-140)."""
    g2 = grad_output.reshape(-1, grad_output.size(-1))
    return linear_gemm.gemm(g2, weight).view(input.shape)
