"""Fused-MLP oracle: y = W_n(... act(W_1 x + b_1) * m_1/(1-p) ...) + b_n.

Reference: the fallback F.linear -> activation -> dropout -> F.linear
(onmt/modules/optimized/feed_forward.py:176-198) with the mask replayed as in the reference's
test (onmt/modules/mlp/test_mlp_gelu.py:229-249), and the native contract it stands behind
(onmt/modules/extensions/mlp/mlp_gelu.cpp:69-194: returns y, post-activations, pre-activations,
mask; backward returns dx, dW.., db..). Activations: relu, exact-erf gelu
(mlp_gelu_cuda.cu:66-81), silu (mlp_silu_cuda.cu:60-81), tanh-approximated gelu "agelu"
(mlp_agelu_cuda.cu:56-90). Weights are nn.Linear layout [out, in]."""
import math

import torch


def act_fwd(h, act):
    if act == "none":
        return h
    if act == "relu":
        return torch.clamp(h, min=0.0)
    if act == "gelu":
        return 0.5 * h * (1.0 + torch.erf(h / math.sqrt(2.0)))
    if act == "silu":
        return h / (1.0 + torch.exp(-h))
    if act == "agelu":
        return 0.5 * h * (1.0 + torch.tanh(0.7978845608028654 * (h + 0.044715 * h ** 3)))
    raise ValueError(act)


def act_bwd(h, act):
    """d act(h) / dh."""
    if act == "none":
        return torch.ones_like(h)
    if act == "relu":
        return (h > 0).to(h.dtype)
    if act == "gelu":
        cdf = 0.5 * (1.0 + torch.erf(h / math.sqrt(2.0)))
        pdf = torch.exp(-0.5 * h * h) / math.sqrt(2.0 * math.pi)
        return cdf + h * pdf
    if act == "silu":
        s = 1.0 / (1.0 + torch.exp(-h))
        return s * (1.0 + h * (1.0 - s))
    if act == "agelu":
        k = 0.7978845608028654
        u = k * (h + 0.044715 * h ** 3)
        t = torch.tanh(u)
        du = k * (1.0 + 3.0 * 0.044715 * h * h)
        return 0.5 * (1.0 + t) + 0.5 * h * (1.0 - t * t) * du
    raise ValueError(act)


def _round(t, round_to):
    """The fallback materialises its intermediate tensors in the working dtype (fp16 / bf16);
    round_to reproduces those rounding points, the arithmetic in between stays in ctype."""
    return t if round_to is None else t.to(round_to).to(t.dtype)


def mlp_fwd(x, weights, biases, act, p=0.0, masks=None, ctype=torch.float32, round_to=None):
    """x [N, in]; weights[i] [out_i, in_i]; biases[i] [out_i] or None; masks[i] uint8 [N, out_i]
    for every hidden layer (None / p == 0: no dropout). round_to: dtype in which the fallback
    stores the pre- and post-activations (None: keep full precision).
    -> (y, pre_acts [h_1..h_{n-1}], post_acts [a_1..a_{n-1}])."""
    a = x.to(ctype)
    n = len(weights)
    pre, post = [], []
    for i in range(n):
        h = a @ weights[i].to(ctype).t()
        if biases is not None and biases[i] is not None:
            h = h + biases[i].to(ctype)
        if i == n - 1:
            return h, pre, post
        h = _round(h, round_to)
        pre.append(h)
        a = act_fwd(h, act)
        if masks is not None and p > 0.0:
            a = a * masks[i].to(ctype) / (1.0 - p)
        a = _round(a, round_to)
        post.append(a)


def mlp_bwd(dy, x, weights, pre, post, act, p=0.0, masks=None, ctype=torch.float32, round_to=None):
    """-> (dx, [dW_1..dW_n], [db_1..db_n]) from the saved pre / post activations. round_to: dtype
    in which the fallback stores the hidden-layer gradients."""
    n = len(weights)
    g = dy.to(ctype)
    dws, dbs = [None] * n, [None] * n
    for i in reversed(range(n)):
        inp = x.to(ctype) if i == 0 else post[i - 1].to(ctype)
        dbs[i] = g.sum(0)
        dws[i] = g.t() @ inp
        g = g @ weights[i].to(ctype)
        if i > 0:
            g = _round(g, round_to)
            g = g * act_bwd(pre[i - 1].to(ctype), act)
            if masks is not None and p > 0.0:
                g = g * masks[i - 1].to(ctype) / (1.0 - p)
            g = _round(g, round_to)
    return g, dws, dbs
