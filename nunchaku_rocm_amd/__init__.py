"""MI355X-native SVDQuant kernel path behind nunchaku-rocm's operator API.

``nunchaku_rocm_amd.ops`` mirrors ``nunchaku.ops`` (same function names, argument order and error behaviour) for
the activation quantizer, the W4A4 GEMM with its fused epilogues and the AWQ W4A16 GEMV; ``nunchaku_rocm_amd.linear``
mirrors ``nunchaku.models.linear``.  Everything runs through ``libsvdq_mi355x.so`` (hand-written HIP for gfx950, C ABI
in ``include/svdq_mi355x.h``); there is no fallback path, and importing :mod:`nunchaku_rocm_amd._lib` raises when the
library has not been built.
"""

__version__ = "0.1.0"
