"""Masked softmax (+ inverted dropout) oracle over the last dimension.

Reference: the softmax stage of the attention fallback — masked_fill_(mask, -inf), F.softmax,
dropout, NaN -> 0 (onmt/modules/optimized/self_attention_func.py:206-233;
encdec_attention_func_bias.py:243-267) — and the native softmax's treatment of rows whose keys
are all masked, which yields zeros (onmt/modules/extensions/multihead_attn_blaslt/
softmax_apex.h:209-211). Backward: g = mask * dP / (1 - p); dS = P * (g - sum_k P * g)
(self_attention_func.py:440-447)."""
import torch


def masked_scores(scores, pad_mask=None, time_mask=None, heads=1):
    """scores [B*H, Tq, Tk]; pad_mask [B, Tk] (True = masked key) or time_mask [Tq, Tk]."""
    s = scores.clone()
    if time_mask is not None:
        s.masked_fill_(time_mask.bool().unsqueeze(0), float("-inf"))
    if pad_mask is not None:
        bh, tq, tk = s.shape
        b = bh // heads
        s = s.view(b, heads, tq, tk).masked_fill(pad_mask.bool().view(b, 1, 1, tk), float("-inf")).view(bh, tq, tk)
    return s


def softmax_dropout_fwd(scores, dropout_mask=None, p=0.0, ctype=torch.float32):
    """scores already hold -inf on masked keys. -> (softmax, dropped); fully masked rows -> 0."""
    s = scores.to(ctype)
    m = s.max(dim=-1, keepdim=True).values
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    sm = torch.where(den > 0, e / den, torch.zeros_like(e))
    if dropout_mask is not None and p > 0.0:
        dr = sm * dropout_mask.to(ctype) / (1.0 - p)
    else:
        dr = sm
    return sm, dr


def softmax_dropout_bwd(grad_dropped, softmax, dropout_mask=None, p=0.0, ctype=torch.float32):
    g = grad_dropped.to(ctype)
    sm = softmax.to(ctype)
    if dropout_mask is not None and p > 0.0:
        g = g * dropout_mask.to(ctype) / (1.0 - p)
    return sm * (g - (sm * g).sum(dim=-1, keepdim=True))
