"""PositionWiseFeedForward with the reference's parameter names and constructor
(onmt/modules/optimized/feed_forward.py:25-207): in_proj_weight [inner, model], out_proj_weight
[model, inner], in_proj_bias, out_proj_bias; forward(input [T, B, model]). The two linear layers,
the activation and the dropout run as one fused MLP call; `dropout_residual` adds the fused
dropout + residual kernel.

The variants that the reference leaves to PyTorch ops (:176-205) run on the same kernels here:
 * glu: in_proj_weight is [2 * inner, model]; projection, gated activation + dropout kernel
   (act(a) * b, or a * sigmoid(b) for activation 'sigmoid'), projection;
 * variational: one dropout mask row per batch column, shared by all time steps
   (onmt/modules/dropout.py:32-48), drawn with the reference's own bernoulli_ call and replayed by the fused kernels;
 * weight_drop is stored and, as in the reference's forward, not used."""
import math

import torch
from torch import nn
from torch.nn import Parameter

from . import mlp as fused
from .dropout_add import fused_dropout_add
from .glu import gated_activation_dropout
from .linear import linear_function

recompute = False  # process-wide switch, the counterpart of onmt.constants.recompute


class PositionWiseFeedForward(nn.Module):
    def __init__(self, model_size, inner_size, dropout=0., variational=False, activation="relu", glu=False,
                 weight_drop=0.0, dropout_residual=False, res_dropout=0.0):
        super().__init__()
        fns = {"relu": fused.mlp_relu_function, "gelu": fused.mlp_gelu_function, "silu": fused.mlp_silu_function,
               "swish": fused.mlp_silu_function, "agelu": fused.mlp_agelu_function}
        if activation == "sigmoid" and not glu:
            raise NotImplementedError("PositionWiseFeedForward: the sigmoid activation exists as a gate only (glu=True)")
        if activation not in fns and activation != "sigmoid":
            raise NotImplementedError(f"PositionWiseFeedForward: activation {activation!r} has no HIP kernel")
        self.model_size, self.inner_size = model_size, inner_size
        self.dropout, self.activation = dropout, activation
        self.bias, self.glu, self.variational, self.weight_drop = True, glu, variational, weight_drop
        self.dropout_residual, self.res_dropout = dropout_residual, res_dropout
        self.fused, self.fused_function = not glu, fns.get(activation)
        self.in_proj_weight = Parameter(torch.empty(inner_size * (2 if glu else 1), model_size))
        self.out_proj_weight = Parameter(torch.empty(model_size, inner_size))
        self.in_proj_bias = Parameter(torch.empty(inner_size * (2 if glu else 1)))
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

    def _shared_mask(self, input, width, p):
        """The reference's variational mask: x.new(1, batch, width).bernoulli_(1 - p) (onmt/modules/dropout.py:40-41), as
        keep flags."""
        return input.new_empty(1, input.shape[1], width).bernoulli_(1 - p).to(torch.uint8).view(input.shape[1], width)

    def forward(self, input, *args, **kwargs):
        seq_len, bsz, hidden_size = input.shape
        dropout = self.dropout if self.training else 0.0
        mask = None
        if self.variational and dropout > 0.0:
            mask = self._shared_mask(input, self.inner_size, dropout)                 # [batch, inner]
        if self.glu:
            lin = linear_function(input, self.in_proj_weight, self.in_proj_bias)      # [T, B, 2 * inner]
            hidden = gated_activation_dropout(lin, self.activation, dropout, self.training, mask)
            hidden = linear_function(hidden, self.out_proj_weight, self.out_proj_bias)
            if self.dropout_residual:
                hidden = hidden.clone()          # the residual kernel writes in place, which a function's own output view forbids
        else:
            if mask is not None:                                                       # the fused kernels replay a dense mask
                mask = mask.repeat(seq_len, 1)
            hidden = self.fused_function(dropout, recompute, input.reshape(seq_len * bsz, hidden_size), self.in_proj_weight,
                                         self.out_proj_weight, self.in_proj_bias, self.out_proj_bias, mask=mask)
            hidden = hidden.view(seq_len, bsz, hidden_size)
        if self.dropout_residual:
            if self.variational:
                # the reference's variational branch drops with the layer's own rate, not res_dropout (:203-205)
                res_mask = None
                if dropout > 0.0:
                    res_mask = self._shared_mask(input, hidden_size, dropout).repeat(seq_len, 1).view(-1)
                hidden = fused_dropout_add(hidden, input, dropout, self.training, res_mask)
            else:
                hidden = fused_dropout_add(hidden, input, self.res_dropout, self.training)
        return hidden
