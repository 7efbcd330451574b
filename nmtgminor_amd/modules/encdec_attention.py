"""EncdecMultiheadAttn module with the reference's parameter names and forward signature
(onmt/modules/optimized/encdec_attention.py:10-155): in_proj_weight_q [E, E], in_proj_weight_kv
[2E, E] (rows ordered head, {k,v}, head_dim), out_proj_weight [E, E]; no biases."""
import math

import torch
from torch import nn
from torch.nn import Parameter

from .encdec_attention_func import encdec_attn_func


class EncdecMultiheadAttn(nn.Module):
    def __init__(self, num_heads, embed_dim, attn_drop=0.):
        super().__init__()
        self.embed_dim = embed_dim
        self.num_heads = num_heads
        self.dropout = attn_drop
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == self.embed_dim, "embed_dim must be divisible by num_heads"
        self.bias = False
        self.scaling = self.head_dim ** -0.5
        self.in_proj_weight_q = Parameter(torch.empty(embed_dim, embed_dim))
        self.in_proj_weight_kv = Parameter(torch.empty(2 * embed_dim, embed_dim))
        self.out_proj_weight = Parameter(torch.empty(embed_dim, embed_dim))
        self.register_parameter("in_proj_bias_q", None)
        self.register_parameter("in_proj_bias_kv", None)
        self.out_proj_bias = None
        self.attn_func = encdec_attn_func
        self.reset_parameters()

    def reset_parameters(self, init="normal"):
        if init == "normal":
            std_ = math.sqrt(2.0 / (self.embed_dim + self.embed_dim))
            for w in (self.in_proj_weight_q, self.in_proj_weight_kv, self.out_proj_weight):
                nn.init.normal_(w, 0.0, std_)
        else:
            std_ = math.sqrt(6.0 / (self.embed_dim + self.embed_dim))
            for w in (self.in_proj_weight_q, self.in_proj_weight_kv, self.out_proj_weight):
                nn.init.uniform_(w, -std_, std_)

    def forward(self, query, key, value, attn_mask=None, incremental=False, incremental_cache=None,
                rotary_pos_enc=False, pos_emb_q=None, pos_emb_k=None, **kwargs):
        """query [Tq, B, E]; key (= value) [Tk, B, E]; attn_mask: key padding [B, Tk], 1 = pad."""
        assert value is key, "ERROR: Keys and values must be the same."
        mask = attn_mask
        if mask is not None and mask.dim() == 3:
            mask = mask.squeeze(1)
        # the bias-free function, as in the reference (encdec_attention.py:145-151): double precision off, coverage on;
        # the coverage is the probabilities before dropout
        outputs, coverage = self.attn_func(False, self.training, self.num_heads, query, key, self.in_proj_weight_q,
                                           self.in_proj_weight_kv, self.out_proj_weight, mask, self.dropout, incremental,
                                           incremental_cache, rotary_pos_enc, pos_emb_q, pos_emb_k, False, True)
        return outputs, coverage
