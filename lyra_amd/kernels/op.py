"""The plugin seam: mode -> operator (lyra/kernels/op.py:12-27).

Only the DECODE operators exist in this package; training/prefill modes belong to the reference.
"""
from __future__ import annotations

from enum import Enum, auto
from functools import partial

from lyra_amd.kernels.common import Implementation
from lyra_amd.kernels.decode_attention import decode_attention
from lyra_amd.kernels.decode_gemm import decode_gemm


class Mode(Enum):
    NOCACHE = auto()
    PREFILL = auto()
    DECODE = auto()


def _decode_only(mode: Mode) -> None:
    if mode != Mode.DECODE:
        raise NotImplementedError(f"lyra_amd implements Mode.DECODE only; {mode} stays with the reference kernels")


def attn_op(mode: Mode, implementation: Implementation):
    _decode_only(mode)
    return partial(decode_attention, implementation=implementation)


def gmm_op(mode: Mode, implementation: Implementation):
    _decode_only(mode)
    return partial(decode_gemm, implementation=implementation)
