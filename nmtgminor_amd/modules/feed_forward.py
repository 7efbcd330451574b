"""PositionWiseFeedForward with the reference's parameter names and constructor
(onmt/modules/optimized/feed_forward.py:25-207): in_proj_weight [inner, model], out_proj_weight
[model, inner], in_proj_bias, out_proj_bias; forward(input [T, B, model]). The two linear layers,
the activation and the dropout run as one fused MLP call; `dropout_residual` adds the fused
dropout + residual kernel. Gated (glu) and variational-dropout variants have no HIP kernel and
raise."""
import math

import torch
from torch import nn
from torch.nn import Parameter

from . import mlp as fused
from .dropout_add import fused_dropout_add

recompute = False  # process-wide switch, the counterpart of onmt.constants.recompute


class PositionWiseFeedForward(nn.Module):
    def __init__(self, model_size, inner_size, dropout=0., variational=False, activation="relu", glu=False,
                 weight_drop=0.0, dropout_residual=False, res_dropout=0.0):
        super().__init__()
        if glu or variational or weight_drop > 0.0:
            raise NotImplementedError("PositionWiseFeedForward: glu / variational dropout / weight drop have no HIP kernel")
        fns = {"relu": fused.mlp_relu_function, "gelu": fused.mlp_gelu_function, "silu": fused.mlp_silu_function,
               "swish": fused.mlp_silu_function, "agelu": fused.mlp_agelu_function}
        if activation not in fns:
            raise NotImplementedError(f"PositionWiseFeedForward: activation {activation!r} has no HIP kernel")
        self.model_size, self.inner_size = model_size, inner_size
        self.dropout, self.activation = dropout, activation
        self.bias, self.glu, self.variational = True, False, False
        self.dropout_residual, self.res_dropout = dropout_residual, res_dropout
        self.fused, self.fused_function = True, fns[activation]
        self.in_proj_weight = Parameter(torch.empty(inner_size, model_size))
        self.out_proj_weight = Parameter(torch.empty(model_size, inner_size))
        self.in_proj_bias = Parameter(torch.empty(inner_size))
        self.out_proj_bias = Parameter(torch.empty(model_size))
        self.reset_parameters()

    def reset_parameters(self, init="normal"):
        if init == "normal":
            std_ = math.sqrt(2.0 / (self.model_size + self.inner_size))
            nn.init.normal_(self.in_proj_weight, 0.0, std_)
            nn.init.normal_(self.out_proj_weight, 0.0, std_)
        else:
            std_ = math.sqrt(6.0 / (self.model_size + self.inner_size))
            nn.init.uniform_(self.in_proj_weight, -std_, std_)
            nn.init.uniform_(self.out_proj_weight, -std_, std_)
        nn.init.constant_(self.in_proj_bias, 0.0)
        nn.init.constant_(self.out_proj_bias, 0.0)

    def forward(self, input, *args, **kwargs):
        seq_len, bsz, hidden_size = input.shape
        dropout = self.dropout if self.training else 0.0
        hidden = self.fused_function(dropout, recompute, input.reshape(seq_len * bsz, hidden_size), self.in_proj_weight,
                                     self.out_proj_weight, self.in_proj_bias, self.out_proj_bias)
        hidden = hidden.view(seq_len, bsz, hidden_size)
        if self.dropout_residual:
            hidden = fused_dropout_add(hidden, input, self.res_dropout, self.training)
        return hidden
