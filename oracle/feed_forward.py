"""CPU restatement of the reference's PositionWiseFeedForward in its PyTorch-op form, with the gated and the
variational-dropout variants. Test infrastructure only: nothing under nmtgminor_amd/ imports this.

Reference: onmt/modules/optimized/feed_forward.py:176-205 (F.linear; `hidden, gate = chunk(2); act(hidden) * gate`, or
F.glu for the 'sigmoid' activation; dropout; F.linear; optional dropout + residual) and variational_dropout
(onmt/modules/dropout.py:32-48: one mask of shape [1, batch, width], scaled by 1 / (1 - p), for every time step).
Which elements are dropped is the generator's business: keep-masks are inputs here (broadcastable to the tensor they
apply to, so a [1, B, W] mask is the variational form). Differentiable PyTorch in `ctype`; gradients come from autograd."""
import torch

from .mlp import act_fwd


class _Stored(torch.autograd.Function):
    """A tensor that the kernels store in a 16-bit type: its value is rounded on the way forward and so is its gradient on
    the way back (the backward kernels store the gradient of every such tensor in the same type)."""

    @staticmethod
    def forward(ctx, t, round_to):
        ctx.round_to = round_to
        return t.to(round_to).to(t.dtype)

    @staticmethod
    def backward(ctx, g):
        return g.to(ctx.round_to).to(g.dtype), None


def _r(t, round_to):
    return t if round_to is None else _Stored.apply(t, round_to)


def gated_activation(lin, act):
    """lin [..., 2 * inner] -> act(first half) * second half; 'sigmoid': first half * sigmoid(second half) (F.glu)."""
    a, b = lin.chunk(2, dim=-1)
    if act == "sigmoid":
        return a * torch.sigmoid(b)
    return act_fwd(a, "silu" if act == "swish" else act) * b


def feed_forward(x, w_in, b_in, w_out, b_out, act, glu=False, p=0.0, keep_mask=None, dropout_residual=False, res_p=0.0,
                 res_keep_mask=None, ctype=torch.float64, round_to=None):
    """x [T, B, model] -> [T, B, model]. round_to: the 16-bit type the kernels store their intermediate tensors in."""
    x, w_in, b_in, w_out, b_out = (t.to(ctype) for t in (x, w_in, b_in, w_out, b_out))
    lin = _r(x @ w_in.t() + b_in, round_to)
    hidden = gated_activation(lin, act) if glu else act_fwd(lin, "silu" if act == "swish" else act)
    if p > 0.0:
        hidden = hidden * keep_mask.to(ctype) / (1.0 - p)
    hidden = _r(hidden, round_to)
    out = hidden @ w_out.t() + b_out
    if dropout_residual:
        out = _r(out, round_to)
        if res_p > 0.0:
            out = out * res_keep_mask.to(ctype) / (1.0 - res_p)
        out = out + x
    return out
