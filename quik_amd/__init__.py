"""MI355X-native implementation of the forward path of QUIK's MixedQLinear.

The package mirrors the reference's Python surface for this path:
  quik_amd.asymmetric / quik_amd.symmetric / quik_amd.matmul  <->  quik._C submodules
  quik_amd.qlinear.MixedQLinear / SharedQuantizedInput         <->  experiments/qlinear.py
All compute runs in libquik_hip.so (hand-written HIP for gfx950) through a C ABI declared in
include/quik_hip.h; there is no CPU or PyTorch fallback.
"""
from . import asymmetric, matmul, symmetric  # noqa: F401
from .version import __version__  # noqa: F401

__all__ = ["asymmetric", "matmul", "symmetric", "__version__"]
