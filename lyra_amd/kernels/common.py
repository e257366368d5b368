"""Dispatch contract and shared maths of the kernel layer (lyra/kernels/common.py).

``Implementation`` keeps the reference's three literals so call sites need no change:
  "pallas" - the hand-written kernel (here: HIP for gfx950); ``ValueError`` if the shape has no kernel
  "xla"    - the plain-framework restatement (here: torch ops on the same device)
  "auto"   - the kernel when the shape is supported, else the plain-framework path, logged once.
"hip" is accepted as a synonym of "pallas".
"""
from __future__ import annotations

import math
import os
import sys
from collections.abc import Callable
from typing import Literal

import torch

Implementation = Literal["auto", "pallas", "xla", "hip"]

LOG2_E = math.log2(math.e)


def require(condition: object, message: str) -> None:
    if not condition:
        raise ValueError(message)


def swiglu(x: torch.Tensor, beta: float = 1.702, limit: float = 7.0, shift: float = 1.0, interleaved: bool = False) -> torch.Tensor:
    """lyra/kernels/common.py:98-114."""
    dtype = x.dtype
    if interleaved:
        glu, lin = x[..., ::2], x[..., 1::2]
    else:
        glu, lin = x.chunk(2, dim=-1)
    glu = glu.clamp(max=limit)
    lin = lin.clamp(min=-limit, max=limit)
    gate = glu * torch.sigmoid(beta * glu)
    return ((lin + shift) * gate).to(dtype)


_KERNEL_LOG_SEEN: set[str] = set()
_KERNEL_LOG_ENABLED = os.environ.get("LYRA_LOG_KERNELS", "1") != "0"


def log_kernel_resolution(op: str, *, shape: str, impl: str, tiling: str | None = None) -> None:
    """One stderr line per (op, shape, implementation, tiling); LYRA_LOG_KERNELS=0 silences it (common.py:117-129)."""
    if not _KERNEL_LOG_ENABLED:
        return
    key = f"{op}|{shape}|{impl}|{tiling}"
    if key in _KERNEL_LOG_SEEN:
        return
    _KERNEL_LOG_SEEN.add(key)
    detail = impl if tiling is None else f"{impl:<6} {tiling}"
    print(f"[kernel] {op:<15} {shape:<26} -> {detail}", file=sys.stderr)


def dispatch_kernel(
    op: str,
    *,
    implementation: Implementation,
    shape: str,
    config: object | None,
    tiling: str | None,
    kernel: Callable[[], torch.Tensor],
    reference: Callable[[], torch.Tensor],
    fallback_reason: str | None = None,
) -> torch.Tensor:
    """lyra/kernels/common.py:132-155 with "hip" for "pallas" in messages."""
    if implementation not in ("auto", "pallas", "xla", "hip"):
        raise ValueError(f"{op}: unknown implementation {implementation!r}")
    if config is not None and implementation != "xla":
        assert tiling is not None
        log_kernel_resolution(op, shape=shape, impl="hip", tiling=tiling)
        return kernel()
    if implementation in ("pallas", "hip"):
        raise ValueError(
            f"{op}: no HIP kernel configuration supports inputs ({shape}). "
            "Pass implementation='auto' or 'xla', or pad the inputs to a supported shape."
        )
    reason = fallback_reason or "no HIP kernel for shape"
    fallback = f" ({reason})" if implementation == "auto" else ""
    log_kernel_resolution(op, shape=shape, impl=f"xla{fallback}")
    return reference()
