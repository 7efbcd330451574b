"""Host-side mirror of the reference's autograd.Function / nn.Module layer for the fused ops.

Same class names, positional signatures and return arity as onmt/modules/{layer_norm.py,
mlp/mlp.py, optimized/*.py}; every forward/backward runs in libnmtg_hip.so. Unlike the reference
there is no silent PyTorch fallback: unsupported inputs raise.
"""
