"""Stand-in for the reference module `fused_mlp_relu`
(onmt/modules/extensions/mlp/mlp_relu.cpp:68-133 forward(p, store_dropout_mask, inputs) ->
[out, reserved_space, mask]; :135-199 backward(p, grad_o, fprop_outputs, inputs);
:201-272 backward_recompute(p, grad_o, mask, inputs)). Only the dropped output is kept: a zero
there means "relu-zeroed or dropped", which is all the backward needs."""
from . import _mlp_common as M


def forward(p, store_dropout_mask, inputs, mask=None):
    out, post, _, mask = M.forward("relu", p, inputs, mask, save_pre=False)
    return [out, post, mask]


def backward(p, grad_o, fprop_outputs, inputs):
    post = fprop_outputs[1]
    mask = fprop_outputs[2] if len(fprop_outputs) > 2 else None
    return M.backward("relu", p, grad_o, post, None, mask, inputs)


def backward_recompute(p, grad_o, mask, inputs):
    _, post, _, _ = M.forward("relu", p, inputs, mask if p > 0.0 else None, save_pre=False)
    return M.backward("relu", p, grad_o, post, None, mask, inputs)
