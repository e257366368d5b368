"""Block-scaled FP8 arrays on torch tensors - the data format of lyra/nn/quant.py.

``QArray(qval, scale, block)`` keeps the reference's field names and block convention
(lyra/nn/quant.py:14-31): ``block`` covers the trailing dims, ``scale`` has the leading dims
followed by ``dim // block`` per blocked dim.  The functions here are the (torch, any device)
producers of that format; the decode kernels consume it directly without dequantising.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)


def is_scaled(dt) -> bool:
    """lyra/nn/quant.py:11."""
    return dt in FP8_DTYPES


@dataclass(frozen=True)
class QArray:
    qval: torch.Tensor
    scale: torch.Tensor
    block: tuple[int, ...]

    dtype = property(lambda self: self.qval.dtype)
    shape = property(lambda self: tuple(self.qval.shape))
    ndim = property(lambda self: self.qval.ndim)
    stype = property(lambda self: self.scale.dtype)
    device = property(lambda self: self.qval.device)

    @property
    def ldim(self) -> int:
        return self.qval.ndim - len(self.block)

    def eff_block(self, axis: int) -> int:
        return 1 if axis < self.ldim else self.block[axis - self.ldim]


def tile(x: torch.Tensor, block: tuple[int, ...]) -> torch.Tensor:
    """lyra/nn/quant.py:34-40."""
    n = len(block)
    lead, tail = tuple(x.shape[: x.ndim - n]), tuple(x.shape[x.ndim - n :])
    bad = [(d, b) for d, b in zip(tail, block) if d % b]
    if bad:
        raise ValueError(f"block {block} does not divide trailing dims {tail}")
    return x.reshape(*lead, *(v for d, b in zip(tail, block) for v in (d // b, b)))


def block_axes(ldim: int, sdim: int) -> tuple[int, ...]:
    """lyra/nn/quant.py:43-45."""
    return tuple(ldim + 2 * i + 1 for i in range(sdim))


def _expand(scale: torch.Tensor, axes: tuple[int, ...]) -> torch.Tensor:
    for a in axes:
        scale = scale.unsqueeze(a)
    return scale


def quantize(x, dtype=torch.float8_e4m3fn, block: tuple[int, ...] = (128, 128), scale_dtype=torch.float32) -> QArray:
    """lyra/nn/quant.py:48-75: scale = amax/fmax (1 where amax == 0); qval = clip(x / scale) -> fp8."""
    if isinstance(x, QArray):
        if x.block != tuple(block) or x.dtype != dtype:
            raise ValueError(f"already quantized as {x.dtype}/{x.block}; requested {dtype}/{block}")
        return x
    if not is_scaled(dtype):
        raise ValueError(f"quantize target must be fp8, got {dtype}")
    if is_scaled(scale_dtype):
        raise ValueError("scale dtype must be unscaled (fp32/bf16)")
    block = tuple(block)
    sdim = len(block)
    ldim = x.ndim - sdim
    axes = block_axes(ldim, sdim)
    tiled = tile(x, block)
    fmax = float(torch.finfo(dtype).max)
    amax = tiled.abs().amax(dim=axes).to(torch.float32)
    scale = torch.where(amax > 0, amax / fmax, torch.ones_like(amax)).to(scale_dtype)
    qinv = _expand(1.0 / scale.to(torch.float32), axes)
    # x * qinv promotes like JAX: a bf16 x times an f32 scale is computed in f32
    qval = (tiled.to(torch.float32) * qinv).clamp(-fmax, fmax).to(dtype).reshape(x.shape)
    return QArray(qval, scale, block)


def dequantize(qx: QArray, dtype=torch.bfloat16) -> torch.Tensor:
    """lyra/nn/quant.py:78-86."""
    axes = block_axes(qx.ldim, len(qx.block))
    tiled = tile(qx.qval.to(torch.float32), qx.block)
    scale = _expand(qx.scale.to(torch.float32), axes)
    return (tiled * scale).reshape(qx.shape).to(dtype)


def qupdate(qx: QArray, x: torch.Tensor, start: tuple) -> QArray:
    """lyra/nn/quant.py:89-98 (functional: returns new arrays, inputs untouched)."""
    for axis, s in enumerate(start):
        b = qx.eff_block(axis)
        if isinstance(s, int) and s % b:
            raise ValueError(f"start {s} on axis {axis} is not aligned to block {b}")
    qnew = quantize(x, qx.dtype, qx.block, qx.stype)
    qval, scale = qx.qval.clone(), qx.scale.clone()
    sl = tuple(slice(int(s), int(s) + d) for s, d in zip(start, qnew.qval.shape))
    qval.view(torch.uint8)[sl] = qnew.qval.view(torch.uint8)
    sstart = tuple(int(s) // qx.eff_block(axis) for axis, s in enumerate(start))
    ssl = tuple(slice(s, s + d) for s, d in zip(sstart, qnew.scale.shape))
    scale[ssl] = qnew.scale
    return QArray(qval, scale, qx.block)


def maybe_dequant(x, dtype) -> torch.Tensor:
    """lyra/nn/quant.py:101-103."""
    return dequantize(x, dtype) if isinstance(x, QArray) else x
