"""MI355X-native implementation of the Gaudi MME compute path (GEMM, batched GEMM, convolution fwd/dedx/dedw, casts).

The product is ``csrc/libmme_hip.so`` (hand-written HIP for gfx950 behind the C ABI of ``include/mme_hip.h``); this
package holds its ctypes mirror (``abi``), a Python form of the reference calculator's host API (``calculator``) and
the build step (``build``).
"""
from . import abi  # noqa: F401
from .calculator import ConvolutionParams, Epilogue, HipCalculator, MMEStackException, MmeSimTensor  # noqa: F401
