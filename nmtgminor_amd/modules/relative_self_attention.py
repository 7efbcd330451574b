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
        if embed_dim % num_heads:
            raise AssertionError("embed_dim must be divisible by num_heads")
        self.embed_dim, self.num_heads, self.head_dim = embed_dim, num_heads, embed_dim // num_heads
        self.dropout, self.learnable_pos, self.bias = dropout, bool(learnable_pos), True
        shapes = {"in_proj_weight": (3 * embed_dim, embed_dim), "out_proj_weight": (embed_dim, embed_dim)}
        if self.learnable_pos:
            # one embedding per relative distance in [-max_pos, max_pos], shared by the heads
            if max_pos < 1:
                raise AssertionError("learnable positions need max_pos >= 1")
            self.pos_emb = nn.Embedding(2 * max_pos + 1, self.head_dim)
            self.pos_proj_weight = self.pos_proj_bias = None
        else:
            shapes.update(pos_proj_weight=(embed_dim, embed_dim), pos_proj_bias=(embed_dim,))
        shapes.update(in_proj_bias=(3 * embed_dim,), out_proj_bias=(embed_dim,), r_w_bias=(num_heads, self.head_dim),
                      r_r_bias=(num_heads, self.head_dim))
        for name, shape in shapes.items():                       # registration order = the reference's state_dict order
            self.register_parameter(name, Parameter(torch.empty(shape)))
        self.reset_parameters()
        self.attn_func = relative_self_attn_func

    def reset_parameters(self, init='normal'):
        """'normal': Xavier-normal projection weights, anything else Xavier-uniform; zero projection biases;
        r_w_bias, r_r_bias ~ N(0, 0.02) (relative_self_attention.py:84-105)."""
        weights = [w for w in (self.in_proj_weight, self.out_proj_weight, self.pos_proj_weight) if w is not None]
        fan = 2.0 * self.embed_dim
        for w in weights:
            if init == 'normal':
                nn.init.normal_(w, 0.0, math.sqrt(2.0 / fan))
            else:
                bound = math.sqrt(6.0 / fan)
                nn.init.uniform_(w, -bound, bound)
        for b in (self.in_proj_bias, self.out_proj_bias, self.pos_proj_bias):
            if b is not None:
                nn.init.zeros_(b)
        for b in (self.r_w_bias, self.r_r_bias):
            nn.init.normal_(b, 0.0, 0.02)

    def forward(self, input, pos, key_padding_mask=None, attn_mask=None, mems=None, incremental=False,
                incremental_cache=None, recompute=False):
        """input [T, B, E]; pos [R, 1, E] or [R, B, E], R >= T (with learnable positions: the [T, T] table of distance
        indices into pos_emb); key_padding_mask [1, T, B] or [B, T] (1 = pad) or attn_mask [T, T] (1 = masked).
        -> (outputs [T, B, E], coverage [B*H, T, T])."""
        if key_padding_mask is not None and attn_mask is not None:
            raise AssertionError("ERROR attn_mask and key_padding_mask should not be both defined!")
        mask = key_padding_mask if key_padding_mask is not None else attn_mask
        if mask is not None and mask.dim() == 3:
            # [1, T, B] -> [B, T] for key padding; a trailing singleton on a [T, T, 1] time mask
            mask = mask.squeeze(0).transpose(0, 1) if key_padding_mask is not None else mask.squeeze(-1)
        if self.learnable_pos:
            pos = self.pos_emb(pos)                 # [len_q, len_k] -> [len_q, len_k, head_dim]
        return self.attn_func(input, pos, attn_mask is not None, self.training, self.num_heads, self.in_proj_weight,
                              self.out_proj_weight, self.pos_proj_weight, self.in_proj_bias, self.out_proj_bias,
                              self.pos_proj_bias, self.r_w_bias, self.r_r_bias, mask, self.dropout, incremental,
                              incremental_cache, False, self.learnable_pos, True, recompute)
