"""MI355X-native fused transformer-layer ops with the call signatures of NMTGMinor's extensions.

`nmtgminor_amd.native.*` mirror the reference's pybind modules by name and signature
(fast_layer_norm_cuda, xentropy_cuda, fused_mlp_gelu, ...); `nmtgminor_amd.modules.*` mirror its
autograd.Function / nn.Module layer. All compute runs in libnmtg_hip.so (hand-written HIP for
gfx950) through a C ABI; nothing here falls back to PyTorch ops.
"""
from . import _lib  # noqa: F401

__version__ = "0.1.0"
