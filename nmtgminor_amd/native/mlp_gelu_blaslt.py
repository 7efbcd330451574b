"""Stand-in for the reference module `mlp_gelu_blaslt`
(onmt/modules/extensions/mlp_blaslt/mlp_gelu.cpp:75-242): forward(p, inputs),
backward(p, recompute, grad_o, outputs, inputs), backward_input_only(p, grad_o, outputs, inputs).
With recompute the caller keeps only (out, mask) and the activations are rebuilt from the inputs
and the stored mask before the backward."""
from . import _mlp_common as M


def forward(p, inputs, mask=None):
    out, post, pre, mask = M.forward("gelu", p, inputs, mask)
    return [out, post, pre, mask]


def backward(p, recompute, grad_o, outputs, inputs):
    if recompute:
        mask = outputs[-1]
        _, post, pre, _ = M.forward("gelu", p, inputs, mask if p > 0.0 else None)
    else:
        _, post, pre, mask = outputs[:4]
    return M.backward("gelu", p, grad_o, post, pre, mask, inputs)


def backward_input_only(p, grad_o, outputs, inputs):
    _, post, pre, mask = outputs[:4]
    return M.backward("gelu", p, grad_o, post, pre, mask, inputs, input_only=True)
