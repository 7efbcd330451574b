"""Stand-in for the reference module `fused_mlp_agelu`
(onmt/modules/extensions/mlp/mlp_agelu.cpp: forward(p, inputs), backward(p, grad_o, fprop_outputs,
inputs), backward_input_only(...)). `forward` takes an optional explicit keep-mask to replay."""
from . import _mlp_common as M

_ACT = "agelu"


def forward(p, inputs, mask=None):
    """-> [out, reserved_space, reserved_activations, reserved_mask]"""
    out, post, pre, mask = M.forward(_ACT, p, inputs, mask)
    return [out, post, pre, mask]


def backward(p, grad_o, fprop_outputs, inputs):
    """-> [dx, dW_1..dW_n, db_1..db_n]"""
    _, post, pre, mask = fprop_outputs[:4]
    return M.backward(_ACT, p, grad_o, post, pre, mask, inputs)


def backward_input_only(p, grad_o, fprop_outputs, inputs):
    """-> [dx]"""
    _, post, pre, mask = fprop_outputs[:4]
    return M.backward(_ACT, p, grad_o, post, pre, mask, inputs, input_only=True)
