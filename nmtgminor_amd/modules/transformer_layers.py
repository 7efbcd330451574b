"""EncoderLayer / DecoderLayer: the pre-norm residual blocks of the reference's Transformer
(onmt/models/transformer_layers.py:83-351), composed of this package's fused operators.

    x = x + dropout(attention(LayerNorm(x)))          [decoder: once more with the encoder context]
    x = x + dropout(ffn_scale * FFN(LayerNorm(x)))

with the optional macaron half-step FFN in front (ffn_scale 0.5), stochastic depth (a layer is skipped with
probability `death_rate` during training and its sub-layer outputs are scaled by 1 / (1 - death_rate) when it
runs), and the clamp of inf / nan that fp16 training occasionally produces. Attribute names are the reference's,
so state_dicts interchange. `opt` is the reference's option namespace; the fields read are model_size, inner_size,
n_heads, dropout, attn_dropout, variational_dropout, macaron, rezero, ffn_activation, ffn_glu, fast_self_attention,
fast_xattention, fast_feed_forward and (decoder) ignore_source. Only the fast_* = True forms exist here: they are the
ones that run on the native extensions; the reference's plain-PyTorch attention and feed-forward modules are not part
of this package and asking for them raises.
"""
import torch
from torch import nn

from .encdec_attention import EncdecMultiheadAttn
from .feed_forward import PositionWiseFeedForward
from .pre_post_processing import PrePostProcessing
from .self_attention import SelfMultiheadAttn


class Identity(nn.Module):
    def forward(self, x, *args, **kwargs):
        return x


def preprocessing(rezero, *args, **kwargs):
    """ReZero layers carry no pre-normalisation (transformer_layers.py:75-80)."""
    return Identity() if rezero else PrePostProcessing(*args, **kwargs)


def _opt(opt, name, default):
    return getattr(opt, name, default)


def _require_fast(opt, *names):
    for n in names:
        if not _opt(opt, n, True):
            raise NotImplementedError(f"{n}=False selects the reference's plain-PyTorch module, which this package does not carry")


def _clamp_non_finite_(x):
    if torch.isinf(x).any() or torch.isnan(x).any():
        clamp_value = torch.finfo(x.dtype).max - 1000
        x.clamp_(min=-clamp_value, max=clamp_value)
    return x


class _Layer(nn.Module):
    def _common(self, opt, death_rate):
        self.variational = _opt(opt, "variational_dropout", False)
        self.death_rate = death_rate
        self.fast_self_attention = _opt(opt, "fast_self_attention", True)
        self.macaron = _opt(opt, "macaron", False)
        self.ffn_scale = 0.5 if self.macaron else 1
        rezero = _opt(opt, "rezero", False)
        if self.macaron:
            self.preprocess_mcr_ffn = preprocessing(rezero, opt.model_size, opt.dropout, sequence="n")
            self.postprocess_mcr_ffn = PrePostProcessing(opt.model_size, opt.dropout, sequence="da", variational=self.variational)
            self.mcr_feedforward = self._ffn(opt)
        self.preprocess_attn = PrePostProcessing(opt.model_size, opt.dropout, sequence="n")
        self.postprocess_attn = PrePostProcessing(opt.model_size, opt.dropout, sequence="da", variational=self.variational)

    def _ffn(self, opt):
        return PositionWiseFeedForward(opt.model_size, opt.inner_size, opt.dropout, variational=self.variational,
                                       activation=_opt(opt, "ffn_activation", "relu"), glu=_opt(opt, "ffn_glu", False))

    def _ffn_blocks(self, opt):
        self.preprocess_ffn = PrePostProcessing(opt.model_size, opt.dropout, sequence="n")
        self.postprocess_ffn = PrePostProcessing(opt.model_size, opt.dropout, sequence="da", variational=self.variational)
        self.feedforward = self._ffn(opt)

    def _alive(self):
        if self.training:
            return torch.rand(1)[0].item() >= self.death_rate
        return True

    def _scaled_ffn_scale(self):
        if self.training and self.death_rate > 0:
            return self.ffn_scale / (1 - self.death_rate)
        return self.ffn_scale

    def _survivor_scale(self, out):
        if self.training and self.death_rate > 0:
            return out / (1 - self.death_rate)
        return out

    def _times(self, out, scale):
        return out if scale == 1 else out * scale

    def _macaron_step(self, input):
        if self.macaron:
            out = self.mcr_feedforward(self.preprocess_mcr_ffn(input))
            input = self.postprocess_mcr_ffn(self._times(out, self._scaled_ffn_scale()), input)
        return input

    def _ffn_step(self, input):
        out = self.feedforward(self.preprocess_ffn(input))
        return self.postprocess_ffn(self._times(out, self._scaled_ffn_scale()), input)


class EncoderLayer(_Layer):
    """forward(input [T, B, model_size], attn_mask: key-padding mask [B, T], nonzero = padded) -> [T, B, model_size]."""

    def __init__(self, opt, death_rate=0.0, **kwargs):
        super().__init__()
        _require_fast(opt, "fast_self_attention", "fast_feed_forward")
        self._common(opt, death_rate)
        self._ffn_blocks(opt)
        self.multihead = SelfMultiheadAttn(opt.model_size, opt.n_heads, opt.attn_dropout)

    def forward(self, input, attn_mask):
        if self._alive():
            input = self._macaron_step(input)
            query = self.preprocess_attn(input)
            out, _ = self.multihead(query, None, attn_mask, None, return_coverage=False)    # the coverage is dropped here
            input = self.postprocess_attn(self._survivor_scale(out), input)
            input = self._ffn_step(input)
        return _clamp_non_finite_(input)


class DecoderLayer(_Layer):
    """forward(input [Tq, B, E], context [Tk, B, E], mask_tgt: time mask [Tq, Tq], mask_src: key-padding mask
    [B, Tk]) -> (output, coverage, incremental_cache)."""

    def __init__(self, opt, death_rate=0.0):
        super().__init__()
        _require_fast(opt, "fast_self_attention", "fast_feed_forward")
        self.ignore_source = _opt(opt, "ignore_source", False)
        if not self.ignore_source:
            _require_fast(opt, "fast_xattention")
        self._common(opt, death_rate)
        self.multihead_tgt = SelfMultiheadAttn(opt.model_size, opt.n_heads, opt.attn_dropout)
        if not self.ignore_source:
            self.preprocess_src_attn = PrePostProcessing(opt.model_size, opt.dropout, sequence="n")
            self.postprocess_src_attn = PrePostProcessing(opt.model_size, opt.dropout, sequence="da",
                                                          variational=self.variational)
            self.multihead_src = EncdecMultiheadAttn(opt.n_heads, opt.model_size, opt.attn_dropout)
        self._ffn_blocks(opt)

    def forward(self, input, context, mask_tgt, mask_src, incremental=False, incremental_cache=None, reuse_source=True):
        if incremental and incremental_cache is None:
            incremental_cache = dict()
        coverage = None
        if self._alive():
            input = self._macaron_step(input)
            query = self.preprocess_attn(input)
            out, _ = self.multihead_tgt(query, None, None, mask_tgt, incremental=incremental,
                                        incremental_cache=incremental_cache, return_coverage=False)   # dropped here
            input = self.postprocess_attn(self._survivor_scale(out), input)
            if not self.ignore_source:
                query = self.preprocess_src_attn(input)
                out, coverage = self.multihead_src(query, context, context, mask_src, incremental=incremental,
                                                   incremental_cache=incremental_cache)
                input = self.postprocess_src_attn(self._survivor_scale(out), input)
            input = self._ffn_step(input)
        return _clamp_non_finite_(input), coverage, incremental_cache
