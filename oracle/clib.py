"""ctypes binding of liblyra_oracle.so (the C restatement).  Test infrastructure: tests, smoke and the bench CPU leg only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

ORACLE_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def load() -> ctypes.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    path = os.path.join(ORACLE_DIR, "liblyra_oracle.so")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", ORACLE_DIR], check=True, capture_output=True)
    lib = ctypes.CDLL(path)
    c = ctypes
    lib.lyra_oracle_fp8_e4m3fn_to_f32.restype = c.c_float
    lib.lyra_oracle_fp8_e4m3fn_to_f32.argtypes = [c.c_uint8]
    lib.lyra_oracle_f32_to_fp8_e4m3fn.restype = c.c_uint8
    lib.lyra_oracle_f32_to_fp8_e4m3fn.argtypes = [c.c_float]
    lib.lyra_oracle_fp8_e5m2_to_f32.restype = c.c_float
    lib.lyra_oracle_fp8_e5m2_to_f32.argtypes = [c.c_uint8]
    lib.lyra_oracle_f32_to_fp8_e5m2.restype = c.c_uint8
    lib.lyra_oracle_f32_to_fp8_e5m2.argtypes = [c.c_float]
    lib.lyra_oracle_quantize_rows_fmt.restype = None
    lib.lyra_oracle_quantize_rows_fmt.argtypes = [c.c_void_p, c.c_int64, c.c_int, c.c_void_p, c.c_void_p, c.c_int]
    lib.lyra_oracle_quantize_blocks_fmt.restype = c.c_int
    lib.lyra_oracle_quantize_blocks_fmt.argtypes = [c.c_void_p] + [c.c_int] * 5 + [c.c_void_p] * 2 + [c.c_int]
    lib.lyra_oracle_f32_to_bf16.restype = c.c_uint16
    lib.lyra_oracle_f32_to_bf16.argtypes = [c.c_float]
    lib.lyra_oracle_quantize_rows.restype = None
    lib.lyra_oracle_quantize_rows.argtypes = [c.c_void_p, c.c_int64, c.c_int, c.c_void_p, c.c_void_p]
    lib.lyra_oracle_quantize_blocks.restype = c.c_int
    lib.lyra_oracle_quantize_blocks.argtypes = [c.c_void_p] + [c.c_int] * 5 + [c.c_void_p] * 2
    for name in ("lyra_oracle_decode_window",):
        getattr(lib, name).restype = c.c_int
        getattr(lib, name).argtypes = [c.c_int]
    lib.lyra_oracle_is_sw.restype = c.c_int
    lib.lyra_oracle_is_sw.argtypes = [c.c_int, c.c_int]
    lib.lyra_oracle_sliding_start.restype = c.c_int
    lib.lyra_oracle_sliding_start.argtypes = [c.c_int, c.c_int, c.c_int]
    lib.lyra_oracle_decode_attention.restype = c.c_int
    lib.lyra_oracle_decode_attention.argtypes = [c.c_void_p] * 9 + [c.c_int] * 5 + [c.c_float] + [c.c_int] * 3
    lib.lyra_oracle_decode_gemm.restype = c.c_int
    lib.lyra_oracle_decode_gemm.argtypes = (
        [c.c_void_p] * 3 + [c.c_int] * 2 + [c.c_void_p] * 4 + [c.c_int] * 6 + [c.c_float] * 2 + [c.c_int]
    )
    lib.lyra_oracle_num_threads.restype = c.c_int
    _LIB = lib
    return lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def quantize_rows(x: np.ndarray, fp8_format: int = 1):
    """Block (1,H) quantiser (KV cache); bit-identical to lyra_oracle.quantize(x, (1, H)).  fp8_format 1: e4m3fn, 2: e5m2."""
    lib = load()
    H = x.shape[-1]
    flat = np.ascontiguousarray(x.reshape(-1, H), dtype=np.float32)
    q = np.empty(flat.shape, dtype=np.uint8)
    s = np.empty(flat.shape[0], dtype=np.float32)
    lib.lyra_oracle_quantize_rows_fmt(_p(flat), flat.shape[0], H, _p(q), _p(s), int(fp8_format))
    return q.reshape(x.shape), s.reshape(*x.shape[:-1], 1)


def quantize_blocks(w: np.ndarray, block, fp8_format: int = 1):
    """Block (bk,bn) quantiser of [G,K,N] weights; bit-identical to lyra_oracle.quantize(w, block).  fp8_format 1: e4m3fn, 2: e5m2."""
    lib = load()
    G, K, N = w.shape
    bk, bn = block
    w = np.ascontiguousarray(w, dtype=np.float32)
    q = np.empty(w.shape, dtype=np.uint8)
    s = np.empty((G, K // bk, N // bn), dtype=np.float32)
    if lib.lyra_oracle_quantize_blocks_fmt(_p(w), G, K, N, bk, bn, _p(q), _p(s), int(fp8_format)):
        raise ValueError(f"block {block} does not divide {(K, N)}")
    return q, s


def decode_attention(q_bits, k, v, k_scale, v_scale, sinks, position, gate, sm_scale, sliding_window, *, ref_rounding=False,
                     fp8_format: int = 1):
    """q_bits uint16 [B,N,1,H]; k,v uint8 (fp8 codes of ``fp8_format``: 1 e4m3fn, 2 e5m2) or uint16 (bf16) [B,K,S,H]; returns f32
    [B,N,1,H]."""
    lib = load()
    B, N, _, H = q_bits.shape
    _, K, S, _ = k.shape
    fp8 = k.dtype == np.uint8
    q_bits = np.ascontiguousarray(q_bits)
    k, v = np.ascontiguousarray(k), np.ascontiguousarray(v)
    ks = np.ascontiguousarray(k_scale, dtype=np.float32) if fp8 else None
    vs = np.ascontiguousarray(v_scale, dtype=np.float32) if fp8 else None
    sinks = np.ascontiguousarray(sinks, dtype=np.float32)
    pos = np.ascontiguousarray(np.broadcast_to(np.asarray(position, dtype=np.int32).reshape(-1), (B,)))
    g = None if gate is None else np.ascontiguousarray(gate, dtype=np.float32)
    out = np.empty((B, N, 1, H), dtype=np.float32)
    rc = lib.lyra_oracle_decode_attention(
        _p(q_bits), _p(k), _p(v), _p(ks), _p(vs), _p(sinks), _p(pos), _p(g), _p(out),
        B, N, K, S, H, float(sm_scale), int(sliding_window), int(fp8_format) if fp8 else 0, int(ref_rounding),
    )
    if rc:
        raise RuntimeError(f"lyra_oracle_decode_attention failed: {rc}")
    return out


def decode_gemm(lhs_bits, rhs, rhs_scale, block, group_sizes, bias, *, fused_swiglu=False, beta=1.702, limit=7.0,
                ref_rounding=False, scratch=None, dequant_bf16=False, fp8_format: int = 1):
    """lhs_bits uint16 [M,K]; rhs uint8 (fp8 codes of ``fp8_format``: 1 e4m3fn, 2 e5m2; with rhs_scale/block) or uint16 (bf16)
    [G,K,N]; returns f32.
    ref_rounding: dequantised weights and outputs rounded to bf16; dequant_bf16 (without it): only the dequantised weights."""
    lib = load()
    M, K = lhs_bits.shape
    G, _, N = rhs.shape
    fp8 = rhs.dtype == np.uint8
    bk, bn = block if fp8 else (0, 0)
    lhs_bits, rhs = np.ascontiguousarray(lhs_bits), np.ascontiguousarray(rhs)
    sc = np.ascontiguousarray(rhs_scale, dtype=np.float32) if fp8 else None
    gs = np.ascontiguousarray(group_sizes, dtype=np.int32)
    b = None if bias is None else np.ascontiguousarray(np.asarray(bias, dtype=np.float32).reshape(G, N))
    out = np.empty((M, N // 2 if fused_swiglu else N), dtype=np.float32)
    if scratch is None:
        scratch = np.empty((G, K, N), dtype=np.float32)
    rc = lib.lyra_oracle_decode_gemm(
        _p(lhs_bits), _p(rhs), _p(sc), bk, bn, _p(gs), _p(b), _p(out), _p(scratch),
        M, G, K, N, int(fp8_format) if fp8 else 0, int(fused_swiglu), float(beta), float(limit), 1 if ref_rounding else (2 if dequant_bf16 else 0),
    )
    if rc:
        raise RuntimeError(f"lyra_oracle_decode_gemm failed: {rc}")
    return out
