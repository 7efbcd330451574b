"""SelfMultiheadAttn module with the reference's parameter names and forward signature
(onmt/modules/optimized/self_attention.py:21-146): in_proj_weight [3E, E] (rows ordered head,
{q,k,v}, head_dim), out_proj_weight [E, E], in_proj_bias [3E], out_proj_bias [E]."""
import math

import torch
from torch import nn
from torch.nn import Parameter

from .self_attention_func import self_attn_func


class SelfMultiheadAttn(nn.Module):
    def __init__(self, embed_dim, num_heads, dropout=0., rotary_pos_enc=False):
        super().__init__()
        self.embed_dim = embed_dim
        self.num_heads = num_heads
        self.dropout = dropout
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == self.embed_dim, "embed_dim must be divisible by num_heads"
        self.bias = True
        self.scaling = self.head_dim ** -0.5
        self.rotary_pos_enc = rotary_pos_enc
        self.in_proj_weight = Parameter(torch.empty(3 * embed_dim, embed_dim))
        self.out_proj_weight = Parameter(torch.empty(embed_dim, embed_dim))
        self.in_proj_bias = Parameter(torch.empty(3 * embed_dim))
        self.out_proj_bias = Parameter(torch.empty(embed_dim))
        self.reset_parameters()
        self.attn_func = self_attn_func

    def reset_parameters(self):
        std_ = math.sqrt(2.0 / (self.embed_dim + self.embed_dim))
        nn.init.normal_(self.in_proj_weight, 0.0, std_)
        nn.init.normal_(self.out_proj_weight, 0.0, std_)
        nn.init.constant_(self.in_proj_bias, 0.)
        nn.init.constant_(self.out_proj_bias, 0.)

    def forward(self, inputs, pos=None, key_padding_mask=None, attn_mask=None, incremental=False,
                incremental_cache=None, return_coverage=True, **kwargs):
        """inputs [T, B, E]; key_padding_mask [B, T] (1 = pad) or attn_mask [T, T] (1 = masked). return_coverage (not in
        the reference's module, which always asks for it): a caller that drops the coverage passes False, and a training
        call with a key padding mask then writes no [B*H, T, T] tensor (the second result is an empty tensor)."""
        mask = None
        if key_padding_mask is not None:
            assert attn_mask is None, "ERROR attn_mask and key_padding_mask should not be both defined!"
            mask = key_padding_mask
            if mask.dim() == 3:
                mask = mask.squeeze(1)
        elif attn_mask is not None:
            mask = attn_mask
            if mask.dim() == 3:
                mask = mask.squeeze(0)
            mask = mask.to(torch.bool)
        outputs, coverage = self.attn_func(attn_mask is not None, self.training, self.num_heads, inputs,
                                           self.in_proj_weight, self.out_proj_weight, self.in_proj_bias,
                                           self.out_proj_bias, mask, self.dropout, self.rotary_pos_enc, pos, incremental,
                                           incremental_cache, True, bool(return_coverage), False)
        return outputs, coverage
