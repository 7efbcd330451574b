"""Stand-alone masked softmax + dropout stage.

Mirrors AttentionSoftmaxDropout of the reference (onmt/modules/optimized/attention_softmax.py:16-67):
forward(inputs, double_precision, dropout_prob, is_training, heads) ->
(dropout_mask, softmax_results, dropout_results); backward(grad_outputs, softmax_results,
dropout_prob_t, heads_t, dropout_mask) -> softmax_grads. The reference's native branch is
fp16-only with len_k <= 2048; here fp32 / fp16 / bf16 up to 2048 keys (4096 when aligned)."""
from ..native import mask_softmax_dropout_cuda


class AttentionSoftmaxDropout(object):
    @staticmethod
    def forward(inputs, double_precision, dropout_prob, is_training, heads, dropout_mask=None):
        if double_precision:
            raise RuntimeError("AttentionSoftmaxDropout: fp64 is not supported by the HIP kernels")
        return mask_softmax_dropout_cuda.forward(is_training, heads, inputs.contiguous(), dropout_prob,
                                                 dropout_mask=dropout_mask)

    @staticmethod
    def backward(grad_outputs, softmax_results, dropout_prob_t, heads_t, dropout_mask):
        p = float(dropout_prob_t[0]) if hasattr(dropout_prob_t, "__getitem__") else float(dropout_prob_t)
        heads = int(heads_t[0]) if hasattr(heads_t, "__getitem__") else int(heads_t)
        return mask_softmax_dropout_cuda.backward(heads, grad_outputs, softmax_results, dropout_mask, p)
