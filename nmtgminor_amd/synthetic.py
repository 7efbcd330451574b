"""Seeded synthetic inputs for the benchmark workloads and their scaled-down test versions (plain PyTorch on the CPU; no
kernel and no reference arithmetic is involved).

Everything is generated on the CPU in fp32 from `torch.Generator().manual_seed(seed)`, then
rounded to the workload's dtype, so a CPU check and the HIP path see identical bits.
"""
import math

import torch


def _gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def xavier_uniform(shape, gen):
    fan_out, fan_in = shape
    bound = math.sqrt(6.0 / (fan_in + fan_out))
    return (torch.rand(shape, generator=gen) * 2.0 - 1.0) * bound


def bernoulli_mask(shape, keep, gen):
    return (torch.rand(shape, generator=gen) < keep).to(torch.uint8)


def layer_norm_inputs(rows=4096, hidden=512, dtype=torch.float32, wdtype=None, seed=1001):
    """Workload 1: x ~ N(0,1), gamma = 1 + 0.1 N(0,1), beta = 0.1 N(0,1), dy ~ N(0,1), eps 1e-5."""
    g = _gen(seed)
    wdtype = wdtype or dtype
    return dict(
        x=torch.randn(rows, hidden, generator=g).to(dtype),
        gamma=(1.0 + 0.1 * torch.randn(hidden, generator=g)).to(wdtype),
        beta=(0.1 * torch.randn(hidden, generator=g)).to(wdtype),
        dy=torch.randn(rows, hidden, generator=g).to(wdtype),
        eps=1e-5,
    )


def mlp_inputs(tokens=8192, d_model=512, d_inner=2048, dtype=torch.float16, p=0.1, seed=1002, zero_bias=True):
    """Workload 2: x ~ N(0,1); W1 [inner, model], W2 [model, inner] xavier-uniform; biases 0;
    dropout keep-mask Bernoulli(1-p) on the hidden activations; dy ~ N(0,1)."""
    g = _gen(seed)
    d = dict(
        x=torch.randn(tokens, d_model, generator=g).to(dtype),
        w1=xavier_uniform((d_inner, d_model), g).to(dtype),
        w2=xavier_uniform((d_model, d_inner), g).to(dtype),
        mask=bernoulli_mask((tokens, d_inner), 1.0 - p, g),
        dy=torch.randn(tokens, d_model, generator=g).to(dtype),
        p=p,
    )
    if zero_bias:
        d["b1"] = torch.zeros(d_inner, dtype=dtype)
        d["b2"] = torch.zeros(d_model, dtype=dtype)
    else:
        d["b1"] = (0.1 * torch.randn(d_inner, generator=g)).to(dtype)
        d["b2"] = (0.1 * torch.randn(d_model, generator=g)).to(dtype)
    return d


def lengths_mask(batch, t, lo, hi, gen):
    """Key-padding mask [batch, t], True = padded key; lengths uniform in [lo, hi]."""
    lens = torch.randint(lo, hi + 1, (batch,), generator=gen)
    return torch.arange(t).unsqueeze(0) >= lens.unsqueeze(1), lens


def self_attn_inputs(t=512, batch=32, d_model=1024, heads=16, dtype=torch.bfloat16, p=0.1, seed=1003,
                     min_len=None, zero_bias=True, causal=False):
    """Workload 3: x ~ N(0,1) [T,B,E]; W_in [3E,E], W_out [E,E] xavier-uniform; key-padding mask
    with lengths uniform in [T/2, T]; dropout keep-mask on [B*H, T, T]; dout ~ N(0,1).
    causal=True gives the decoder self-attention of workload 4 (time mask, no padding mask)."""
    g = _gen(seed)
    e = d_model
    d = dict(
        x=torch.randn(t, batch, e, generator=g).to(dtype),
        w_in=xavier_uniform((3 * e, e), g).to(dtype),
        w_out=xavier_uniform((e, e), g).to(dtype),
        heads=heads, p=p,
    )
    if zero_bias:
        d["b_in"] = torch.zeros(3 * e, dtype=dtype)
        d["b_out"] = torch.zeros(e, dtype=dtype)
    else:
        d["b_in"] = (0.1 * torch.randn(3 * e, generator=g)).to(dtype)
        d["b_out"] = (0.1 * torch.randn(e, generator=g)).to(dtype)
    if causal:
        d["time_mask"] = torch.triu(torch.ones(t, t), diagonal=1).bool()
        d["pad_mask"] = None
    else:
        lo = t // 2 if min_len is None else min_len
        d["pad_mask"], d["lengths"] = lengths_mask(batch, t, lo, t, g)
        d["time_mask"] = None
    d["dropout_mask"] = bernoulli_mask((batch * heads, t, t), 1.0 - p, g) if p > 0 else None
    d["dout"] = torch.randn(t, batch, e, generator=g).to(dtype)
    return d


def rel_self_attn_inputs(t=64, batch=2, d_model=256, heads=4, dtype=torch.bfloat16, p=0.1, seed=1006, len_r=None,
                         pos_batch=1, causal=False):
    """Self-attention with relative positions: the self-attention inputs plus sinusoid-sized position states
    pos ~ N(0,1) [R, 1 or B, E] (R >= T), W_pos [E, E] xavier-uniform, b_pos and r_w_bias, r_r_bias [H, D] ~ 0.1 N(0,1)."""
    d = self_attn_inputs(t, batch, d_model, heads, dtype, p, seed, zero_bias=False, causal=causal)
    g = _gen(seed + 7919)
    e = d_model
    r = t if len_r is None else len_r
    d["pos"] = torch.randn(r, pos_batch, e, generator=g).to(dtype)
    d["w_pos"] = xavier_uniform((e, e), g).to(dtype)
    d["b_pos"] = (0.1 * torch.randn(e, generator=g)).to(dtype)
    d["r_w_bias"] = (0.1 * torch.randn(heads, e // heads, generator=g)).to(dtype)
    d["r_r_bias"] = (0.1 * torch.randn(heads, e // heads, generator=g)).to(dtype)
    return d


def encdec_attn_inputs(tq=128, tk=1500, batch=16, d_model=1024, heads=16, dtype=torch.bfloat16, p=0.0,
                       seed=1004, zero_bias=True):
    """Workload 4: encoder states [Tk,B,E], decoder states [Tq,B,E] ~ N(0,1); W_q [E,E],
    W_kv [2E,E], W_out [E,E] xavier-uniform; key-padding lengths uniform in [Tk/2, Tk]."""
    g = _gen(seed)
    e = d_model
    d = dict(
        x_kv=torch.randn(tk, batch, e, generator=g).to(dtype),
        x_q=torch.randn(tq, batch, e, generator=g).to(dtype),
        w_q=xavier_uniform((e, e), g).to(dtype),
        w_kv=xavier_uniform((2 * e, e), g).to(dtype),
        w_out=xavier_uniform((e, e), g).to(dtype),
        heads=heads, p=p,
    )
    if zero_bias:
        d["b_q"] = torch.zeros(e, dtype=dtype)
        d["b_kv"] = torch.zeros(2 * e, dtype=dtype)
        d["b_out"] = torch.zeros(e, dtype=dtype)
    else:
        d["b_q"] = (0.1 * torch.randn(e, generator=g)).to(dtype)
        d["b_kv"] = (0.1 * torch.randn(2 * e, generator=g)).to(dtype)
        d["b_out"] = (0.1 * torch.randn(e, generator=g)).to(dtype)
    d["pad_mask"], d["lengths"] = lengths_mask(batch, tk, tk // 2, tk, g)
    d["dropout_mask"] = bernoulli_mask((batch * heads, tq, tk), 1.0 - p, g) if p > 0 else None
    d["dout"] = torch.randn(tq, batch, e, generator=g).to(dtype)
    return d


def zipf_targets(n, vocab, s, gen):
    """Zipf(s) over [0, vocab) by inverse CDF of weights 1 / k^s, k = 1..vocab (id = k - 1)."""
    w = torch.arange(1, vocab + 1, dtype=torch.float64).pow(-s)
    cdf = torch.cumsum(w, 0)
    cdf = cdf / cdf[-1]
    u = torch.rand(n, generator=gen, dtype=torch.float64)
    return torch.searchsorted(cdf, u).clamp_(max=vocab - 1)


def xentropy_inputs(tokens=16384, vocab=250054, dtype=torch.bfloat16, smoothing=0.1, padding_idx=1,
                    pad_fraction=0.1, seed=1005, with_logits=True):
    """Workload 5: logits ~ N(0, sigma=2); targets Zipf(1.1) over the vocabulary; a seeded 10 %
    of the positions is set to the padding index; grad_loss = 1 (sum reduction)."""
    g = _gen(seed)
    labels = zipf_targets(tokens, vocab, 1.1, g)
    perm = torch.randperm(tokens, generator=g)
    labels[perm[: int(round(tokens * pad_fraction))]] = padding_idx
    d = dict(labels=labels, smoothing=smoothing, padding_idx=padding_idx,
             grad_loss=torch.ones(tokens, dtype=torch.float32))
    if with_logits:
        d["logits"] = (2.0 * torch.randn(tokens, vocab, generator=g)).to(dtype)
    return d
