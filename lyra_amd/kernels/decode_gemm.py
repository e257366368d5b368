"""Decode grouped matmul behind the call signature of lyra/kernels/decode_gemm.py:404-415.

``decode_gemm(lhs, rhs, group_sizes, *, bias, fused_swiglu, swiglu_beta, swiglu_limit, quant_dtype,
implementation)`` runs the gfx950 HIP kernel through ``lyra_decode_gemm`` (include/lyra_hip.h).
``group_sizes`` stays on the device; the kernel skips experts that have no rows.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from lyra_amd import _lib
from lyra_amd.kernels.common import Implementation, dispatch_kernel, swiglu
from lyra_amd.nn.quant import QArray, dequantize, is_scaled, quantize


@dataclass(frozen=True)
class DecodeGEMMConfig:
    """Mirrors decode_gemm.py:40-51; scale_k/scale_n are only the default on-the-fly quantisation block."""

    scale_k: int = 256
    scale_n: int = 256
    fwd_dtype: torch.dtype | None = None


_MAX_GROUPS = 8191  # the kernel's limit (LYRA_E_UNSUPPORTED beyond it)


def _scale_layout_supported(k: int, n: int, block: tuple[int, int]) -> bool:
    bk, bn = block
    if bk <= 0 or bn <= 0 or k % bk or n % bn or bn & (bn - 1):
        return False
    if bn % 8 == 0 and (bk % 32 == 0 or bk == k):
        return True
    return bk == k


def select_decode_gemm_config(m: int, groups: int, k: int, n: int, quant_dtype=None, block=None, fused_swiglu=False) -> DecodeGEMMConfig | None:
    """Support predicate of the HIP kernel (cf. decode_gemm.py:70-94)."""
    if min(m, groups, k, n) <= 0 or groups > _MAX_GROUPS:
        return None
    quant_dtype = quant_dtype if quant_dtype is not None and is_scaled(quant_dtype) else None
    if k % 32 or n % 8 or (fused_swiglu and n % 16):  # (whole 128-column spans get the streaming kernels, other widths the general one)
        return None
    if quant_dtype is not None:
        if quant_dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
            return None
        if block is not None and not _scale_layout_supported(k, n, tuple(block)):
            return None
    return DecodeGEMMConfig(fwd_dtype=quant_dtype)


def _expert_ids(group_sizes: torch.Tensor, total: int) -> torch.Tensor:
    """lyra/kernels/gemm.py:450-456; rows at or beyond sum(group_sizes) get id G-1."""
    G = group_sizes.shape[0]
    ids = torch.repeat_interleave(torch.arange(G, dtype=torch.int32, device=group_sizes.device), group_sizes.to(torch.int64))
    if ids.shape[0] < total:
        ids = torch.cat([ids, torch.full((total - ids.shape[0],), G - 1, dtype=torch.int32, device=ids.device)])
    return ids[:total]


def normalize_bias(bias, groups: int, features: int, dtype) -> torch.Tensor:
    """lyra/kernels/gemm.py:393-400."""
    if bias is None:
        raise ValueError("normalize_bias needs a bias")
    if bias.ndim == 2:
        bias = bias[:, None, :]
    if tuple(bias.shape) != (groups, 1, features):
        raise ValueError(f"Unsupported bias shape: {tuple(bias.shape)}")
    return bias.to(dtype)


def _decode_gemm(lhs, rhs, group_sizes, config: DecodeGEMMConfig, *, bias, fused_swiglu, swiglu_beta, swiglu_limit, out_dtype):
    """Launch the HIP kernel (the counterpart of decode_gemm.py:301-365, with the epilogue fused)."""
    M, K = lhs.shape
    G, _, N = rhs.shape
    if not lhs.is_cuda:
        raise ValueError("the HIP decode GEMM kernel needs device tensors")
    dev = lhs.device
    if config.fwd_dtype is not None:
        if not isinstance(rhs, QArray):
            raise ValueError("FP8 decode GEMM requires a block-scaled QArray RHS")
        if rhs.dtype != config.fwd_dtype:
            raise ValueError(f"FP8 decode RHS dtype must be {config.fwd_dtype}, got {rhs.dtype}")
        bk, bn = rhs.block
        expected = (G, K // bk, N // bn)
        if tuple(rhs.scale.shape) != expected:
            raise ValueError(f"FP8 decode RHS scale must be {expected}, got {tuple(rhs.scale.shape)}")
        rhs_val = rhs.qval.contiguous()
        rhs_scale = rhs.scale.to(torch.float32).contiguous()
        rhs_dtype = _lib.fp8_code(rhs.qval.dtype)
    else:
        if isinstance(rhs, QArray):
            raise ValueError("dense decode GEMM config received a QArray RHS")
        rhs_val = rhs.to(torch.bfloat16).contiguous()
        rhs_scale, bk, bn = None, 0, 0
        rhs_dtype = _lib.DTYPE_BF16
    lhs_c = lhs.to(torch.bfloat16).contiguous()
    gs = group_sizes.to(device=dev, dtype=torch.int32).contiguous()
    bias_c = None
    if bias is not None:
        bias_c = normalize_bias(bias, G, N, torch.float32).to(dev).reshape(G, N).contiguous()
    NO = N // 2 if fused_swiglu else N
    k_out = torch.float32 if out_dtype == torch.float32 else torch.bfloat16
    out = torch.empty((M, NO), dtype=k_out, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    need = _lib.lib.lyra_decode_gemm_workspace(M, G, K, N, int(fused_swiglu))
    ws = _lib.workspace("gemm", dev, stream, need)
    with torch.cuda.device(dev):
        rc = _lib.lib.lyra_decode_gemm(
            lhs_c.data_ptr(), rhs_val.data_ptr(), rhs_scale.data_ptr() if rhs_scale is not None else None, bk, bn,
            gs.data_ptr(), bias_c.data_ptr() if bias_c is not None else None, out.data_ptr(), ws.data_ptr(), ws.numel(),
            M, G, K, N, rhs_dtype, _lib.DTYPE_F32 if k_out == torch.float32 else _lib.DTYPE_BF16,
            int(fused_swiglu), float(swiglu_beta), float(swiglu_limit), stream,
        )
    _lib.check(rc, "lyra_decode_gemm")
    return out if out.dtype == out_dtype else out.to(out_dtype)


def grouped_gemm_reference(lhs, rhs, group_sizes, *, bias=None, fused_swiglu=False, swiglu_beta=1.702, swiglu_limit=7.0):
    """lyra/kernels/gemm.py:1575-1617 with quant_dtype=None: ragged dot in f32, f32 bias, f32 SwiGLU, cast."""
    M, K = lhs.shape
    G, _, N = rhs.shape
    rhs_f = dequantize(rhs, lhs.dtype) if isinstance(rhs, QArray) else rhs
    sizes = group_sizes.to(torch.int64).tolist()
    t = torch.zeros((M, N), dtype=torch.float32, device=lhs.device)
    off = 0
    for g, n in enumerate(sizes):
        n = min(n, M - off)
        if n > 0:
            t[off : off + n] = lhs[off : off + n].to(torch.float32) @ rhs_f[g].to(torch.float32)
        off += max(n, 0)
    if bias is not None:
        ids = _expert_ids(group_sizes, M).to(torch.int64)
        t = t + normalize_bias(bias, G, N, torch.float32).to(lhs.device)[ids, 0, :]
    if fused_swiglu:
        t = swiglu(t, swiglu_beta, swiglu_limit)
    return t.to(lhs.dtype)


def decode_gemm_reference(lhs, rhs, group_sizes, *, bias=None, fused_swiglu=False, swiglu_beta=1.702, swiglu_limit=7.0, quant_dtype=None):
    """lyra/kernels/decode_gemm.py:368-401: (quantise,) dequantise every expert to lhs.dtype, then the grouped product."""
    if quant_dtype is not None and is_scaled(quant_dtype):
        if isinstance(rhs, QArray):
            rhs_q = rhs
        else:
            block = (math.gcd(rhs.shape[-2], 256), math.gcd(rhs.shape[-1], 256))
            rhs_q = quantize(rhs, quant_dtype, block)
        rhs = dequantize(rhs_q, lhs.dtype)
    return grouped_gemm_reference(
        lhs, rhs, group_sizes, bias=bias, fused_swiglu=fused_swiglu, swiglu_beta=swiglu_beta, swiglu_limit=swiglu_limit
    )


def decode_gemm(
    lhs: torch.Tensor,
    rhs,
    group_sizes: torch.Tensor,
    *,
    bias: torch.Tensor | None = None,
    fused_swiglu: bool = False,
    swiglu_beta: float = 1.702,
    swiglu_limit: float = 7.0,
    quant_dtype: torch.dtype | None = None,
    implementation: Implementation = "auto",
) -> torch.Tensor:
    """lhs [M,K] (rows sorted by group); rhs [G,K,N] tensor or QArray; group_sizes [G] int32; returns [M,N] or [M,N/2]."""
    M, _ = lhs.shape
    G, K, N = rhs.shape
    dtype = quant_dtype if quant_dtype is not None and is_scaled(quant_dtype) else None

    # decode_gemm.py:422-437: which weights the kernel and the plain path see
    if dtype is not None:
        if isinstance(rhs, QArray):
            rhs_q = rhs
        else:
            scale_config = DecodeGEMMConfig(fwd_dtype=dtype)
            block = (math.gcd(K, scale_config.scale_k), math.gcd(N, scale_config.scale_n))
            rhs_q = quantize(rhs, dtype, block)
        rhs_kernel = rhs_q
        block = rhs_q.block
    elif isinstance(rhs, QArray):
        rhs_kernel = dequantize(rhs, lhs.dtype)
        block = None
    else:
        rhs_kernel = rhs
        block = None
    out_dtype = lhs.dtype

    config = (
        select_decode_gemm_config(m=M, groups=G, k=K, n=N, quant_dtype=dtype, block=block, fused_swiglu=fused_swiglu)
        if lhs.is_cuda
        else None
    )

    def reference():
        rhs_reference = dequantize(rhs_kernel, lhs.dtype) if isinstance(rhs_kernel, QArray) else rhs_kernel.to(lhs.dtype)
        return decode_gemm_reference(
            lhs, rhs_reference, group_sizes, bias=bias, fused_swiglu=fused_swiglu, swiglu_beta=swiglu_beta, swiglu_limit=swiglu_limit
        )

    def kernel():
        assert config is not None
        return _decode_gemm(
            lhs, rhs_kernel, group_sizes, config, bias=bias, fused_swiglu=fused_swiglu,
            swiglu_beta=swiglu_beta, swiglu_limit=swiglu_limit, out_dtype=out_dtype,
        )

    tiling = None if config is None else f"n8/k32 dtype={'fp8' if config.fwd_dtype else 'bf16'}"
    op_shape = f"m{M} g{G} k{K} n{N}"
    return dispatch_kernel(
        "decode_gemm", implementation=implementation, shape=op_shape, config=config, tiling=tiling, kernel=kernel, reference=reference
    )
