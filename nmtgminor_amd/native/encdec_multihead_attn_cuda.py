"""Stand-in for the reference's bias-free extension `encdec_multihead_attn_cuda` (not built by its setup.py by default,
onmt/modules/extensions/setup.py:113-126; bound by onmt/modules/optimized/encdec_attention_func.py:15-18, call sites
:81-86, :322-345, :355-362): the same function names, argument order and returned lists, on the HIP kernels. What sets
it apart from the biased extension: no bias arguments, and the tensor it returns and takes back for the softmax stage is
`softmax_results` (the probabilities before dropout), not the masked scores."""
import torch

from .. import _lib as L
from . import _attn_common as A
from . import encdec_multihead_attn_bias_blaslt as biased


def forward(is_training, heads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, pad_mask,
            dropout_prob, *, dropout_mask=None):
    """-> [input_lin_q_results, input_lin_kv_results, softmax_results, dropout_results, dropout_mask,
    matmul2_results, outputs]. pad_mask: None, [B, Tk], or the reference's broadcast form [B, 1, 1, Tk]."""
    tensors = (inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights)
    L.require_cuda(*tensors, pad_mask, dropout_mask)
    A.check_half(*tensors)
    tq, tk, b, e = biased._shapes(inputs_q, inputs_kv, heads, 1)
    A.check(input_weights_q.shape == (e, e) and input_weights_kv.shape == (2 * e, e) and output_weights.shape == (e, e),
            "weight shapes do not match the inputs")
    if pad_mask is not None and pad_mask.dim() > 2:
        pad_mask = pad_mask.reshape(b, tk)
    c = lambda z: z.contiguous()
    softmax = torch.empty(b * heads, tq, tk, dtype=inputs_q.dtype, device=inputs_q.device)
    q_lin, kv_lin, _, dropped, dmask, ctx, out = biased._fwd(
        is_training, heads, c(inputs_q), c(inputs_kv), c(input_weights_q), c(input_weights_kv), c(output_weights), None, None,
        None, None, None, pad_mask, dropout_prob, dropout_mask, tq, tk, b, e, inputs_q.device, inputs_q.dtype,
        softmax_out=softmax)
    return [q_lin, kv_lin, softmax, dropped, dmask, ctx, out]


def backward(heads, output_grads, matmul2_results, dropout_results, softmax_results, input_lin_q_results,
             input_lin_kv_results, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights, dropout_mask,
             dropout_prob):
    """-> [input_q_grads, input_kv_grads, input_weight_q_grads, input_weight_kv_grads, output_weight_grads]"""
    n = biased._bwd(heads, output_grads, matmul2_results, dropout_results, softmax_results, input_lin_q_results,
                    input_lin_kv_results, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights,
                    dropout_mask, dropout_prob, from_probs=True)
    return [n[k] for k in ("dxq", "dxkv", "dwq", "dwkv", "dwo")]


def backward_recompute(heads, output_grads, inputs_q, inputs_kv, input_weights_q, input_weights_kv, output_weights,
                       dropout_mask, pad_mask, dropout_prob):
    """Re-runs the forward from the inputs and the stored dropout mask, then the backward."""
    training = dropout_mask is not None and dropout_mask.numel() > 0 and dropout_prob > 0.0
    q_lin, kv_lin, softmax, dropped, dmask, ctx, _ = forward(training, heads, inputs_q, inputs_kv, input_weights_q,
                                                             input_weights_kv, output_weights, pad_mask, dropout_prob,
                                                             dropout_mask=dropout_mask if training else None)
    return backward(heads, output_grads, ctx, dropped, softmax, q_lin, kv_lin, inputs_q, inputs_kv, input_weights_q,
                    input_weights_kv, output_weights, dmask, dropout_prob)
