"""Block-scaled FP8 arrays on torch tensors - the data format of lyra/nn/quant.py.

``QArray(qval, scale, block)`` keeps the reference's field names and block convention
(lyra/nn/quant.py:14-31): ``block`` covers the trailing dims, ``scale`` has the leading dims
followed by ``dim // block`` per blocked dim.  The functions here are the (torch, any device)
producers of that format; the decode kernels consume it directly without dequantising.

``dot`` / ``einsum`` (lyra/nn/quant.py:106-113) are the seam of the dense projections: an activation of a few
rows times a [C, N] weight (bf16 or QArray) runs on the one-group HIP decode matmul, everything else on torch ops.
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


# ---- the dense-projection seam -------------------------------------------------------------------------
def _flat_weight(rhs):
    """A weight [C, *rest] (contracted over its first axis) as the [1, C, N] stack the decode matmul takes, or None when
    a QArray's scale blocks do not survive flattening ``rest`` into one axis (then the caller dequantises)."""
    if not isinstance(rhs, QArray):
        return rhs.reshape(1, rhs.shape[0], -1)
    if len(rhs.block) != rhs.ndim or any(b != 1 for b in rhs.block[1:-1]):
        return None
    C = rhs.shape[0]
    bk, bn = rhs.block[0], rhs.block[-1]
    return QArray(rhs.qval.reshape(1, C, -1), rhs.scale.reshape(1, C // bk, -1), (bk, bn))


def _dot_general_torch(lhs, rhs, dimension_numbers, out_dtype):
    """lax.dot_general on torch tensors: output axes are batch, then lhs free, then rhs free."""
    (lc, rc), (lb, rb) = dimension_numbers
    names = iter("abcdefghijklmnopqrstuvwxyz")
    ln, rn = [None] * lhs.ndim, [None] * rhs.ndim
    for i, j in list(zip(lb, rb)) + list(zip(lc, rc)):
        ln[i] = rn[j] = next(names)
    ln = [c if c is not None else next(names) for c in ln]
    rn = [c if c is not None else next(names) for c in rn]
    out = [ln[i] for i in lb] + [c for i, c in enumerate(ln) if i not in lb and i not in lc] + \
          [c for j, c in enumerate(rn) if j not in rb and j not in rc]
    acc = torch.float32 if out_dtype == torch.float32 else lhs.dtype
    return torch.einsum(f"{''.join(ln)},{''.join(rn)}->{''.join(out)}", lhs.to(acc), rhs.to(acc)).to(out_dtype)


def dot(lhs: torch.Tensor, rhs, *, dimension_numbers=None, preferred_element_type=None, implementation: str = "auto"):
    """lyra/nn/quant.py:106-108: ``lax.dot(lhs, maybe_dequant(rhs, lhs.dtype), **kw)``.

    The decode step's projections (lyra/model.py:307-309, 366, 614, 628: ``[B, 1, C] . [C, N]`` with
    ``dimension_numbers=NN_INNER``, N possibly several trailing axes as in the ``[C, 2, Hd]`` up projection) contract the
    last axis of a bf16 activation with the first axis of a bf16 or FP8 weight: those run as the one-group decode matmul
    on the HIP kernel, reading the FP8 codes directly.  ``implementation``: "auto" = the kernel when the shapes allow it,
    "pallas"/"hip" = the kernel or ValueError, "xla" = torch ops on the dequantised weight (also what any other
    contraction, dtype or device gets).  Output dtype: ``preferred_element_type`` or ``lhs.dtype``."""
    out_dtype = preferred_element_type or lhs.dtype
    if dimension_numbers is None:
        dimension_numbers = (((lhs.ndim - 1,), (0,)), ((), ()))
    (lc, rc), (lb, rb) = (tuple(map(tuple, d)) for d in dimension_numbers)
    inner = lc == (lhs.ndim - 1,) and rc == (0,) and not lb and not rb
    flat = _flat_weight(rhs) if inner and rhs.ndim >= 2 else None
    fp8 = isinstance(rhs, QArray)
    kernel_ok = (flat is not None and lhs.is_cuda and lhs.dtype == torch.bfloat16 and out_dtype in (torch.bfloat16, torch.float32)
                 and (rhs.dtype in FP8_DTYPES if fp8 else rhs.dtype == torch.bfloat16))
    if not kernel_ok:
        if implementation in ("pallas", "hip"):
            raise ValueError(f"quant.dot: no HIP kernel for lhs {tuple(lhs.shape)} {lhs.dtype} . rhs {tuple(rhs.shape)} {rhs.dtype} "
                             f"with dimension_numbers {dimension_numbers}")
        return _dot_general_torch(lhs, maybe_dequant(rhs, lhs.dtype), ((lc, rc), (lb, rb)), out_dtype)
    from lyra_amd.kernels.decode_gemm import decode_gemm  # (the kernels package imports this module)

    rows = lhs.reshape(-1, lhs.shape[-1])
    if out_dtype == torch.float32:
        rows = rows.to(torch.float32)  # the operator's output dtype is its lhs dtype; the values stay bf16-representable
    sizes = torch.full((1,), rows.shape[0], dtype=torch.int32, device=lhs.device)
    out = decode_gemm(rows, flat, sizes, quant_dtype=rhs.dtype if fp8 else None, implementation=implementation)
    return out.reshape(*lhs.shape[:-1], *rhs.shape[1:])


def einsum(subscript: str, lhs: torch.Tensor, rhs, *, preferred_element_type=None, implementation: str = "auto"):
    """lyra/nn/quant.py:111-113.  A subscript that contracts only the last axis of lhs with the first axis of rhs
    ("btc,cn->btn") is ``dot``; any other is torch.einsum on the dequantised weight."""
    spec = subscript.replace(" ", "")
    if "->" in spec and "." not in spec:
        ins, out = spec.split("->")
        a, b = ins.split(",") if ins.count(",") == 1 else ("", "")
        if a and b and a[-1] == b[0] and out == a[:-1] + b[1:] and len(set(a + b[1:])) == len(a + b[1:]) \
                and len(a) == lhs.ndim and len(b) == rhs.ndim:
            return dot(lhs, rhs, preferred_element_type=preferred_element_type, implementation=implementation)
    if implementation in ("pallas", "hip"):
        raise ValueError(f"quant.einsum: no HIP kernel for '{subscript}'")
    out_dtype = preferred_element_type or lhs.dtype
    acc = torch.float32 if out_dtype == torch.float32 else lhs.dtype
    return torch.einsum(spec, lhs.to(acc), maybe_dequant(rhs, lhs.dtype).to(acc)).to(out_dtype)
