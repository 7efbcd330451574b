"""Encoder / decoder layer oracle: the composition the reference's layers perform
(onmt/models/transformer_layers.py:145-185 encoder, :283-343 decoder; the step sequences "n" and "da" of
onmt/modules/pre_post_processing.py:53-82), written over this package's per-op functions in differentiable tensor
arithmetic, so that gradients of a whole layer come from autograd in fp64.

    x = x + dropout(s * SelfAttention(LayerNorm(x)))
    x = x + dropout(s * CrossAttention(LayerNorm(x), context))        (decoder, unless ignore_source)
    x = x + dropout(f * FFN(LayerNorm(x)))             preceded, with macaron, by the same line with its own FFN

s = 1 / (1 - death_rate) and f = ffn_scale / (1 - death_rate) in training (ffn_scale = 0.5 with macaron), else 1 and
ffn_scale. Dropout is the identity here (evaluation mode, or p = 0): the modules under test draw their own masks,
which cannot be replayed through the layer interface. `params` is a state_dict with the reference's key names.

round_to (a 16-bit type, or None): the tensors that pass between operators, and those the operators store inside, are
rounded to it, in the forward and (the cast being differentiable: its backward casts the gradient) in the backward — the
residual stream, each LayerNorm output, the attention and feed-forward intermediates that the per-op functions round, and
each branch's output. attn_core ("stored" / "tiled") picks which attention kernels' rounding points are modelled (see
oracle/attention.py). With round_to=None nothing is rounded.

Pinned by tests/test_oracle_pins.py::test_layer_oracle_matches_torch_modules: an nn.TransformerEncoderLayer /
nn.TransformerDecoderLayer (norm_first, gelu) given the same weights (de-interleaved) produces the same output.
"""
import torch

from . import attention, layer_norm, mlp
from .attention import _r


def _ln(x, params, prefix, ctype, round_to=None, eps=1e-5):
    t, b, e = x.shape
    x = _r(x, round_to)          # x is a stored tensor already: a no-op forward; backward, LayerNorm's input gradient is stored rounded
    z, _, _ = layer_norm.ln_fwd(x.reshape(t * b, e), params[prefix + ".layer_norm.function.weight"],
                                params[prefix + ".layer_norm.function.bias"], eps, ctype)
    return _r(z.view(t, b, e), round_to)


def _ffn(x, params, prefix, act, ctype, round_to=None):
    t, b, e = x.shape
    y, _, _ = mlp.mlp_fwd(x.reshape(t * b, e), [params[prefix + ".in_proj_weight"], params[prefix + ".out_proj_weight"]],
                          [params[prefix + ".in_proj_bias"], params[prefix + ".out_proj_bias"]], act, ctype=ctype, round_to=round_to)
    return _r(y.view(t, b, e), round_to)


def _self_attn(x, params, prefix, heads, pad_mask, time_mask, ctype, round_to=None, core="stored"):
    r = attention.self_attn_fwd(x, params[prefix + ".in_proj_weight"], params[prefix + ".out_proj_weight"],
                                params[prefix + ".in_proj_bias"], params[prefix + ".out_proj_bias"], heads, pad_mask, time_mask,
                                ctype=ctype, round_to=round_to, core=core)
    r["outputs"] = _r(r["outputs"], round_to)
    return r


def encoder_layer(x, params, heads, pad_mask, act="relu", macaron=False, death_rate=0.0, training=False,
                  ctype=torch.float64, round_to=None, attn_core="stored"):
    """x [T, B, E]; pad_mask [B, T] (True = padded key) or None. -> [T, B, E] in ctype."""
    x = x.to(ctype)
    s = 1.0 / (1.0 - death_rate) if training and death_rate > 0 else 1.0
    f = (0.5 if macaron else 1.0) * s
    rt = round_to
    if macaron:
        x = _r(x + f * _ffn(_ln(x, params, "preprocess_mcr_ffn", ctype, rt), params, "mcr_feedforward", act, ctype, rt), rt)
    x = _r(x + s * _self_attn(_ln(x, params, "preprocess_attn", ctype, rt), params, "multihead", heads, pad_mask, None, ctype, rt,
                              attn_core)["outputs"], rt)
    x = _r(x + f * _ffn(_ln(x, params, "preprocess_ffn", ctype, rt), params, "feedforward", act, ctype, rt), rt)
    return x


def decoder_layer(x, context, params, heads, time_mask, src_pad_mask, act="relu", macaron=False, ignore_source=False,
                  death_rate=0.0, training=False, ctype=torch.float64, round_to=None, attn_core="stored"):
    """x [Tq, B, E], context [Tk, B, E]; time_mask [Tq, Tq], src_pad_mask [B, Tk] (True = masked).
    -> (output [Tq, B, E], coverage [B*H, Tq, Tk] = the cross-attention probabilities, or None)."""
    x = x.to(ctype)
    s = 1.0 / (1.0 - death_rate) if training and death_rate > 0 else 1.0
    f = (0.5 if macaron else 1.0) * s
    coverage = None
    rt = round_to
    if macaron:
        x = _r(x + f * _ffn(_ln(x, params, "preprocess_mcr_ffn", ctype, rt), params, "mcr_feedforward", act, ctype, rt), rt)
    x = _r(x + s * _self_attn(_ln(x, params, "preprocess_attn", ctype, rt), params, "multihead_tgt", heads, None, time_mask, ctype, rt,
                              attn_core)["outputs"], rt)
    if not ignore_source:
        p = "multihead_src"
        # the reference's EncdecMultiheadAttn carries no biases (optimized/encdec_attention.py:22-33): absent keys = None
        r = attention.encdec_attn_fwd(_ln(x, params, "preprocess_src_attn", ctype, rt), context.to(ctype), params[p + ".in_proj_weight_q"],
                                      params[p + ".in_proj_weight_kv"], params[p + ".out_proj_weight"], params.get(p + ".in_proj_bias_q"),
                                      params.get(p + ".in_proj_bias_kv"), params.get(p + ".out_proj_bias"), heads, src_pad_mask,
                                      ctype=ctype, round_to=rt)
        x = _r(x + s * _r(r["outputs"], rt), rt)
        coverage = r["softmax_results"]
    x = _r(x + f * _ffn(_ln(x, params, "preprocess_ffn", ctype, rt), params, "feedforward", act, ctype, rt), rt)
    return x, coverage
