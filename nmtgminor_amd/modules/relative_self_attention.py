"""RelativeSelfMultiheadAttn module with the reference's parameter names and forward signature
(onmt/modules/optimized/relative_self_attention.py:14-230): in_proj_weight [3E, E] (rows ordered head, {q,k,v},
head_dim), out_proj_weight [E, E], their biases, r_w_bias and r_r_bias [H, D], and either pos_proj_weight [E, E] with its
bias (sinusoidal positions, projected) or, with `learnable_pos=True`, pos_emb, an embedding of 2 max_pos + 1 relative
distances to head_dim that heads and batch share."""
import math

import torch
from torch import nn
from torch.nn import Parameter

from .relative_self_attention_func import relative_self_attn_func


class RelativeSelfMultiheadAttn(nn.Module):
    def __init__(self, embed_dim, num_heads, dropout=0., learnable_pos=False, max_pos=0):
        super().__init__()
        self.embed_dim = embed_dim
        self.num_heads = num_heads
        self.dropout = dropout
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == self.embed_dim, "embed_dim must be divisible by num_heads"
        self.bias = True
        self.learnable_pos = learnable_pos
        self.in_proj_weight = Parameter(torch.empty(3 * embed_dim, embed_dim))
        self.out_proj_weight = Parameter(torch.empty(embed_dim, embed_dim))
        if self.learnable_pos:
            # one embedding per relative distance in [-max_pos, max_pos], shared across heads
            assert max_pos >= 1
            self.pos_emb = nn.Embedding(2 * max_pos + 1, self.head_dim)
            self.pos_proj_weight, self.pos_proj_bias = None, None
        else:
            self.pos_proj_weight = Parameter(torch.empty(embed_dim, embed_dim))
            self.pos_proj_bias = Parameter(torch.empty(embed_dim))
        self.in_proj_bias = Parameter(torch.empty(3 * embed_dim))
        self.out_proj_bias = Parameter(torch.empty(embed_dim))
        self.r_w_bias = Parameter(torch.empty(self.num_heads, self.head_dim))
        self.r_r_bias = Parameter(torch.empty(self.num_heads, self.head_dim))
        self.reset_parameters()
        self.attn_func = relative_self_attn_func

    def reset_parameters(self, init='normal'):
        if init == 'normal':  # xavier normal
            std_ = math.sqrt(2.0 / (self.embed_dim + self.embed_dim))
            for w in (self.in_proj_weight, self.out_proj_weight, self.pos_proj_weight):
                if w is not None:
                    nn.init.normal_(w, 0.0, std_)
        else:
            std_ = math.sqrt(6.0 / (self.embed_dim + self.embed_dim))
            for w in (self.in_proj_weight, self.out_proj_weight, self.pos_proj_weight):
                if w is not None:
                    nn.init.uniform_(w, -std_, std_)
        for b in (self.in_proj_bias, self.out_proj_bias, self.pos_proj_bias):
            if b is not None:
                nn.init.constant_(b, 0.)
        nn.init.normal_(self.r_w_bias, 0.0, 0.02)
        nn.init.normal_(self.r_r_bias, 0.0, 0.02)

    def forward(self, input, pos, key_padding_mask=None, attn_mask=None, mems=None, incremental=False,
                incremental_cache=None, recompute=False):
        """input [T, B, E]; pos [R, 1, E] or [R, B, E], R >= T (with learnable positions: the [T, T] table of distance
        indices into pos_emb); key_padding_mask [1, T, B] or [B, T] (1 = pad) or attn_mask [T, T] (1 = masked).
        -> (outputs [T, B, E], coverage [B*H, T, T])."""
        if key_padding_mask is not None:
            assert attn_mask is None, "ERROR attn_mask and key_padding_mask should not be both defined!"
            mask = key_padding_mask
            if mask.dim() == 3:
                mask = mask.squeeze(0).transpose(0, 1)      # [1, T, B] -> [B, T]
        elif attn_mask is not None:
            mask = attn_mask
            if mask.dim() == 3:
                mask = mask.squeeze(-1)
        else:
            mask = None
        if self.learnable_pos:
            pos = self.pos_emb(pos)                 # [len_q, len_k] -> [len_q, len_k, head_dim]
        outputs, coverage = self.attn_func(input, pos, attn_mask is not None, self.training, self.num_heads,
                                           self.in_proj_weight, self.out_proj_weight, self.pos_proj_weight,
                                           self.in_proj_bias, self.out_proj_bias, self.pos_proj_bias, self.r_w_bias,
                                           self.r_r_bias, mask, self.dropout, incremental, incremental_cache, False,
                                           self.learnable_pos, True, recompute)
        return outputs, coverage
