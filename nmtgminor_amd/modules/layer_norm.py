"""LayerNorm on the HIP kernels, with the reference's wrapper names.

Mirrors onmt/modules/layer_norm.py:37-168 (FastLayerNormFN, fast_layer_norm_affine,
layer_norm_func, LayerNorm) and the in-sync variant with `memory_efficient`
(whisper/memory_efficient_whisper.py:73-140), and MultilingualLayerNorm (:175-227: one affine pair per language, the
pair of the call picked by `factor`). The reference only routes hidden sizes
768/1024/2048/3072/4096 to its native kernels; here every hidden size takes the native path.
"""
import numbers

import torch
from torch.nn import init
from torch.nn.parameter import Parameter

from ..native import fast_layer_norm_cuda
from ._autocast import cast_if_autocast_enabled, no_autocast


class FastLayerNormFN(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gamma, beta, epsilon, memory_efficient=False):
        ctx.x_shape = x.shape
        ctx.memory_efficient = memory_efficient
        x = x.contiguous()
        gamma = gamma.contiguous()
        beta = beta.contiguous()
        xmat = x.view(-1, gamma.numel())
        ymat, mu, rsigma = fast_layer_norm_cuda.ln_fwd(xmat, gamma, beta, epsilon)
        if memory_efficient:
            ctx.save_for_backward(ymat, gamma, None, rsigma, beta)
        else:
            ctx.save_for_backward(xmat, gamma, mu, rsigma, None)
        return ymat.view(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x_or_y, gamma, mu, rsigma, beta = ctx.saved_tensors
        dymat = dy.contiguous().view(x_or_y.shape)
        if dymat.dtype != gamma.dtype:
            dymat = dymat.to(gamma.dtype)
        dx, dgamma, dbeta, _, _ = fast_layer_norm_cuda.ln_bwd(dymat, x_or_y, mu, rsigma, gamma, beta,
                                                              ctx.memory_efficient)
        return dx.view(ctx.x_shape), dgamma, dbeta, None, None


def fast_layer_norm_affine(input, weight, bias, normalized_shape, eps=1e-5, memory_efficient=False):
    args = cast_if_autocast_enabled(input, weight, bias, eps, memory_efficient)
    with no_autocast():
        return FastLayerNormFN.apply(*args)


def _affine_or_identity(input, weight, bias, hidden):
    if weight is None:
        weight = torch.ones(hidden, dtype=input.dtype, device=input.device)
    if bias is None:
        bias = torch.zeros(hidden, dtype=weight.dtype, device=input.device)
    return weight, bias


def layer_norm_func(input, weight, bias, normalized_shape, eps=1e-05):
    hidden = input.size(-1)
    weight, bias = _affine_or_identity(input, weight, bias, hidden)
    return fast_layer_norm_affine(input, weight, bias, normalized_shape, eps)


class LayerNorm(torch.nn.Module):
    """Same parameters (`weight`, `bias`) and constructor as the reference module
    (onmt/modules/layer_norm.py:123-172); `forward(input, fast=True)`."""

    def __init__(self, normalized_shape, eps=1e-5, elementwise_affine=True, bias=True, device=None,
                 dtype=None, memory_efficient=False):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        if len(normalized_shape) != 1:
            raise ValueError("LayerNorm normalises over the last dimension only")
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        self.memory_efficient = memory_efficient
        kw = {"device": device, "dtype": dtype}
        if elementwise_affine:
            self.weight = Parameter(torch.empty(*normalized_shape, **kw))
            if bias:
                self.bias = Parameter(torch.empty(*normalized_shape, **kw))
            else:
                self.register_parameter("bias", None)
        else:
            self.register_parameter("weight", None)
            self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        if self.elementwise_affine:
            init.ones_(self.weight)
            if self.bias is not None:
                init.zeros_(self.bias)

    def forward(self, input, fast=True):
        hidden = self.normalized_shape[0]
        weight, bias = _affine_or_identity(input, self.weight, self.bias, hidden)
        # the memory-efficient backward divides by gamma and needs beta: only with a real affine
        me = self.memory_efficient and self.weight is not None and self.bias is not None
        return fast_layer_norm_affine(input, weight, bias, self.normalized_shape, self.eps, me)

    def extra_repr(self):
        return "{normalized_shape}, eps={eps}, elementwise_affine={elementwise_affine}".format(**self.__dict__)


class MultilingualLayerNorm(torch.nn.Module):
    """One (weight, bias) pair per language, [n_languages, hidden] each; `forward(input, factor)` normalises with the pair
    that `factor` (an index tensor with one element) selects (onmt/modules/layer_norm.py:175-227). The selection is an
    index_select, so the gradient lands in the selected rows and the others get zeros, as in the reference."""

    def __init__(self, normalized_shape, eps=1e-5, elementwise_affine=True, n_languages=1):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        if len(normalized_shape) != 1:
            raise ValueError("MultilingualLayerNorm normalises over the last dimension only")
        self.n_languages = n_languages
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        if elementwise_affine:
            self.weight = Parameter(torch.empty(n_languages, *normalized_shape))
            self.bias = Parameter(torch.empty(n_languages, *normalized_shape))
        else:
            self.register_parameter("weight", None)
            self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        if self.elementwise_affine:
            init.ones_(self.weight)
            init.zeros_(self.bias)

    def forward(self, input, factor):
        weight = bias = None
        if self.elementwise_affine:
            if factor is None or factor.numel() != 1:
                raise RuntimeError("MultilingualLayerNorm: `factor` must be an index tensor with one element (the language)")
            weight = torch.index_select(self.weight, 0, factor.view(1)).squeeze(0)
            bias = torch.index_select(self.bias, 0, factor.view(1)).squeeze(0)
        weight, bias = _affine_or_identity(input, weight, bias, self.normalized_shape[0])
        return fast_layer_norm_affine(input, weight, bias, self.normalized_shape, self.eps)

    def extra_repr(self):
        return "{normalized_shape}, eps={eps}, elementwise_affine={elementwise_affine}, n_languages={n_languages}".format(**self.__dict__)
