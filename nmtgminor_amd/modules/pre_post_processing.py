"""PrePostProcessing: the step sequence the reference wraps around every sub-layer
(onmt/modules/pre_post_processing.py:10-82). `sequence` is a string of steps applied in order:
    n  LayerNorm over the model dimension      d  dropout      a  add the residual `input_tensor`
    z  ReZero: scale by a learned scalar `g` (initially 0), then add the residual
Constructor arguments, attribute names and state_dict keys (`layer_norm.function.weight`, `.bias`, `g`) are the
reference's. On the HIP path "n" is the LayerNorm kernel and an adjacent "d", "a" pair with plain (element-wise)
dropout is the fused dropout + residual-add kernel, in place on the sub-layer's output; the variational dropout
(one mask per sequence position-independent [1, B, H] slice) keeps the reference's tensor expression.
With multilingual=True "n" is the MultilingualLayerNorm (one affine pair per language; `forward(..., factor=)` picks it; state_dict
keys `layer_norm.weight`, `.bias` as in the reference, which does not wrap that module in Bottle).
"""
import torch
from torch import nn

from .dropout_add import fused_dropout_add
from .layer_norm import LayerNorm, MultilingualLayerNorm


class Bottle(nn.Module):
    """Holder that calls `function` on its input (onmt/modules/bottle.py:13-30); kept for the state_dict key."""

    def __init__(self, function):
        super().__init__()
        self.function = function

    def forward(self, input, mask=None):
        return self.function(input)


class VariationalDropout(nn.Module):
    """One keep-mask per (batch, feature), shared over time (onmt/modules/dropout.py:8-30)."""

    def __init__(self, p=0.5, batch_first=False, inplace=False):
        super().__init__()
        self.p, self.batch_first, self.inplace = p, batch_first, inplace

    def forward(self, x):
        if not self.training or not self.p:
            return x
        shape = (x.size(0), 1, x.size(2)) if self.batch_first else (1, x.size(1), x.size(2))
        m = x.new_empty(shape).bernoulli_(1 - self.p).div_(1 - self.p)
        if self.inplace:
            return x.mul_(m)
        return x * m


class PrePostProcessing(nn.Module):
    def __init__(self, d_model, dropout_p, sequence="nda", variational=False, elementwise_affine=True,
                 multilingual=False, n_languages=1):
        super().__init__()
        self.d_model = d_model
        self.dropout_p = dropout_p
        self.multilingual = multilingual
        self.variational = variational
        self.steps = list(sequence)
        if "n" in self.steps:
            if multilingual:      # one affine pair per language, picked by forward's `factor` (pre_post_processing.py:40-42)
                self.layer_norm = MultilingualLayerNorm((d_model,), eps=1e-5, elementwise_affine=True, n_languages=n_languages)
            else:
                self.layer_norm = Bottle(LayerNorm((d_model,), elementwise_affine=elementwise_affine))
        if "d" in self.steps:
            self.dropout = VariationalDropout(dropout_p, batch_first=False) if variational \
                else nn.Dropout(dropout_p, inplace=False)
        if "z" in self.steps:
            self.g = nn.Parameter(torch.tensor(0.0))

    def _fusable(self, i, output, input_tensor):
        """May steps i, i + 1 ("d", "a") run as the in-place dropout + add kernel on `output`?"""
        if not (self.steps[i] == "d" and i + 1 < len(self.steps) and self.steps[i + 1] == "a" and not self.variational
                and input_tensor is not None and input_tensor.shape == output.shape and input_tensor.dtype == output.dtype
                and output.dtype in (torch.float32, torch.float16, torch.bfloat16)):
            return False
        if i > 0 and self.steps[i - 1] == "n":
            return False        # the LayerNorm output may be what its backward reads (memory-efficient form)
        # autograd forbids writing into a view that a custom Function created itself (its backward would be bypassed)
        if output.requires_grad and output._is_view() and isinstance(output.grad_fn, torch.autograd.function.BackwardCFunction):
            return False
        return True

    def forward(self, tensor, input_tensor=None, mask=None, factor=None):
        output = tensor
        i = 0
        while i < len(self.steps):
            step = self.steps[i]
            if step == "n":
                output = self.layer_norm(output, factor) if self.multilingual else self.layer_norm(output)
            elif step == "d":
                if self._fusable(i, output, input_tensor):
                    # dropout and the residual add in one pass over the tensor
                    output = fused_dropout_add(output, input_tensor, self.dropout_p, self.training)
                    i += 1
                else:
                    output = self.dropout(output)
            elif step == "a":
                if input_tensor is not None:
                    output = output + input_tensor
            elif step == "z":
                output = output * self.g
                if input_tensor is not None:
                    output = output + input_tensor
            i += 1
        return output
