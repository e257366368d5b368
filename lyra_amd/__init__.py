"""MI355X-native decode kernels behind Lyra's kernel call signatures.

``lyra_amd.kernels.decode_attention.decode_attention`` and
``lyra_amd.kernels.decode_gemm.decode_gemm`` keep the positional/keyword
contract of ``lyra/kernels/decode_attention.py:364`` and
``lyra/kernels/decode_gemm.py:404`` of the reference; they run hand-written
gfx950 HIP kernels through the C ABI declared in ``include/lyra_hip.h``.
"""
from lyra_amd import _lib  # noqa: F401  (fails loudly when the HIP library is absent)

__all__ = ["_lib"]
