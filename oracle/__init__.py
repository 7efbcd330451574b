"""CPU oracle for the fused transformer-layer ops — TEST INFRASTRUCTURE ONLY.

This package restates, in plain PyTorch tensor arithmetic on the CPU, what the reference's own
PyTorch fallback computes for each op on the hot path. It exists to check the HIP kernels. Only
`tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import it; the
product package `nmtgminor_amd` never does and has no CPU path of its own.

Every function takes CPU tensors, converts them to `ctype` (fp32 by default, fp64 for stricter
checks) and returns tensors in `ctype`: the inputs may already be rounded to fp16/bf16, the
arithmetic here is not. Dropout is always an explicit uint8 keep-mask (1 = keep), applied as
x * mask / (1 - p), which is how the reference replays masks in its own tests
(onmt/modules/mlp/test_mlp_gelu.py:229-249).

How each function is pinned (tests/test_oracle_*.py, all CPU): against the PyTorch library
routine the reference falls back to (F.layer_norm, F.cross_entropy, F.linear/F.gelu,
F.scaled_dot_product_attention, nn.MultiheadAttention after de-interleaving the weights, softmax
autograd), against closed forms and invariants, by brute-force Python loops on tiny shapes and
by fp64 finite differences (torch.autograd.gradcheck, the reference's own method for its
hand-written backward, onmt/modules/optimized/self_attention_func.py:955-967). The reference
tree holds no stored golden vectors for these ops; tests/golden/ holds small fixtures written by
tests/golden/make_fixtures.py from PyTorch's library routines and autograd (not from this
package), against which tests/test_golden_cpu.py checks every function here, including the
fallback's 16-bit rounding points (round_to=).
"""
from . import (attention, dropout_add, fused_optim, inputs, layer_norm, mlp, relative_attention, softmax_dropout,  # noqa: F401
               transformer_layers, xentropy)
