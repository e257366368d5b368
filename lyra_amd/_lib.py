"""ctypes binding of liblyra_hip.so.  There is no fallback: a missing library is an error."""
from __future__ import annotations

import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "liblyra_hip.so")

DTYPE_BF16, DTYPE_E4M3FN, DTYPE_F32, DTYPE_E5M2 = 0, 1, 2, 3
RHS_SPAN_MAJOR, RHS_SPAN_MAJOR_GLU = 0x100, 0x200  # LYRA_RHS_SPAN_MAJOR(_GLU): OR-ed into a matmul's rhs_dtype
LHS_TILED16, OUT_TILED16 = 0x400, 0x800  # LYRA_LHS_TILED16 / LYRA_OUT_TILED16, likewise
ABI_VERSION = 15
E_UNSUPPORTED = -2  # LYRA_E_UNSUPPORTED: a shape or dtype the kernels do not cover


def fp8_code(dtype) -> int:
    """The C ABI's dtype code of a torch FP8 dtype (the two the reference's ``FP8_DTYPES`` names, lyra/nn/quant.py:10)."""
    import torch

    if dtype == torch.float8_e4m3fn:
        return DTYPE_E4M3FN
    if dtype == torch.float8_e5m2:
        return DTYPE_E5M2
    raise ValueError(f"no kernel reads {dtype}")

_c = ctypes
SIGNATURES = {
    "lyra_abi_version": (_c.c_int, []),
    "lyra_strerror": (_c.c_char_p, [_c.c_int]),
    "lyra_decode_attention": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_int] + [_c.c_void_p] * 3 + [_c.c_size_t] + [_c.c_int] * 5 + [_c.c_float] + [_c.c_int] * 3 + [_c.c_void_p],
    ),
    "lyra_decode_attention_workspace": (_c.c_size_t, [_c.c_int] * 6),
    "lyra_attention_rank": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p]),
    "lyra_decode_attention_ranked": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_int] + [_c.c_void_p] * 4 + [_c.c_size_t] + [_c.c_int] * 5 + [_c.c_float] + [_c.c_int] * 3 + [_c.c_void_p],
    ),
    "lyra_decode_attention_xsa": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_int] + [_c.c_void_p] * 5 + [_c.c_size_t] + [_c.c_int] * 5 + [_c.c_float] + [_c.c_int] * 3 + [_c.c_void_p],
    ),
    "lyra_decode_attention_qkv": (
        _c.c_int,
        [_c.c_void_p] * 2 + [_c.c_int] + [_c.c_void_p] * 4 + [_c.c_int, _c.c_float] + [_c.c_void_p] * 6 + [_c.c_int] + [_c.c_void_p] * 3
        + [_c.c_size_t] + [_c.c_int] * 5 + [_c.c_float] + [_c.c_int] * 3 + [_c.c_void_p],
    ),
    "lyra_decode_attention_qkv_bias": (
        _c.c_int,
        [_c.c_void_p] * 2 + [_c.c_int] + [_c.c_void_p] * 5 + [_c.c_int, _c.c_float] + [_c.c_void_p] * 6 + [_c.c_int] + [_c.c_void_p] * 3
        + [_c.c_size_t] + [_c.c_int] * 5 + [_c.c_float] + [_c.c_int] * 3 + [_c.c_void_p],
    ),
    "lyra_decode_attention_static": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_int] + [_c.c_void_p] * 2 + [_c.c_int] * 5 + [_c.c_float] + [_c.c_int] * 3 + [_c.c_void_p],
    ),
    "lyra_workspace_init": (_c.c_int, [_c.c_void_p, _c.c_size_t, _c.c_void_p]),
    "lyra_decode_gemm": (
        _c.c_int,
        [_c.c_void_p] * 3 + [_c.c_int] * 2 + [_c.c_void_p] * 4 + [_c.c_size_t] + [_c.c_int] * 7 + [_c.c_float] * 2 + [_c.c_void_p],
    ),
    "lyra_decode_gemm_workspace": (_c.c_size_t, [_c.c_int] * 5),
    "lyra_decode_gemm_workspace_for": (_c.c_size_t, [_c.c_int] * 6),
    "lyra_decode_gemm_ex": (
        _c.c_int,
        [_c.c_void_p] * 4 + [_c.c_int] * 2 + [_c.c_void_p] * 3 + [_c.c_float, _c.c_int] + [_c.c_void_p] * 2 + [_c.c_size_t]
        + [_c.c_int] * 7 + [_c.c_float] * 2 + [_c.c_void_p],
    ),
    "lyra_rmsnorm_proj": (_c.c_int, [_c.c_void_p] * 6 + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p]),
    "lyra_qkv_post": (
        _c.c_int,
        [_c.c_void_p] * 6 + [_c.c_int] + [_c.c_void_p] * 6 + [_c.c_int] * 7 + [_c.c_float, _c.c_void_p],
    ),
    "lyra_moe_route": (_c.c_int, [_c.c_void_p] * 5 + [_c.c_int] * 4 + [_c.c_void_p]),
    "lyra_moe_combine": (_c.c_int, [_c.c_void_p] * 5 + [_c.c_int] * 3 + [_c.c_float, _c.c_void_p]),
    "lyra_decode_gemm_splits": (_c.c_int, [_c.c_int] * 4),
    "lyra_gemm_packed_bytes": (_c.c_size_t, [_c.c_int] * 5),
    "lyra_gemm_pack": (_c.c_int, [_c.c_void_p] * 2 + [_c.c_int] * 5 + [_c.c_void_p]),
    "lyra_decode_gemm_partials": (
        _c.c_int,
        [_c.c_void_p] * 3 + [_c.c_int] * 2 + [_c.c_void_p] * 2 + [_c.c_size_t] + [_c.c_int] * 4 + [_c.c_void_p],
    ),
    "lyra_rmsnorm_proj_sum": (
        _c.c_int,
        [_c.c_void_p] * 2 + [_c.c_int, _c.c_void_p, _c.c_float] + [_c.c_void_p] * 6 + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p],
    ),
    "lyra_rmsnorm_proj_sum_bias": (
        _c.c_int,
        [_c.c_void_p] * 2 + [_c.c_int, _c.c_void_p, _c.c_void_p, _c.c_float] + [_c.c_void_p] * 6 + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p],
    ),
    "lyra_rmsnorm_proj_embed": (
        _c.c_int,
        [_c.c_void_p] * 2 + [_c.c_int] + [_c.c_void_p] * 6 + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p],
    ),
    "lyra_rmsnorm_proj_combine": (
        _c.c_int,
        [_c.c_void_p] * 3 + [_c.c_int, _c.c_void_p, _c.c_float] + [_c.c_void_p] * 6 + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p],
    ),
    "lyra_qkv_post_sum": (
        _c.c_int,
        [_c.c_void_p] * 2 + [_c.c_int] + [_c.c_void_p] * 5 + [_c.c_int] + [_c.c_void_p] * 6 + [_c.c_int] * 7 + [_c.c_float, _c.c_void_p],
    ),
    "lyra_argmax": (_c.c_int, [_c.c_void_p] * 3 + [_c.c_size_t] + [_c.c_int] * 3 + [_c.c_void_p] * 2),
    "lyra_argmax_workspace": (_c.c_size_t, [_c.c_int] * 2),
    "lyra_sample_topk": (_c.c_int, [_c.c_void_p] * 4 + [_c.c_size_t] + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p, _c.c_void_p]),
    "lyra_sample_topk_rng": (_c.c_int, [_c.c_void_p] * 4 + [_c.c_size_t] + [_c.c_int] * 4 + [_c.c_float, _c.c_void_p, _c.c_void_p]),
    "lyra_sample_topk_workspace": (_c.c_size_t, [_c.c_int] * 3),
    "lyra_decode_gemm_tile_max": (
        _c.c_int,
        [_c.c_void_p] * 4 + [_c.c_int] * 2 + [_c.c_void_p] * 5 + [_c.c_size_t] + [_c.c_int] * 6 + [_c.c_void_p],
    ),
    "lyra_argmax_tiles": (_c.c_int, [_c.c_void_p] * 3 + [_c.c_int] * 4 + [_c.c_void_p] * 2),
    "lyra_sample_topk_tiles": (
        _c.c_int,
        [_c.c_void_p] * 6 + [_c.c_size_t] + [_c.c_int] * 5 + [_c.c_float, _c.c_void_p, _c.c_void_p],
    ),
    "lyra_selftest": (_c.c_int, [_c.c_void_p, _c.c_void_p]),
}


class LyraHipError(RuntimeError):
    pass


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise LyraHipError(
            f"{LIB_PATH} is missing: build it with `python -m lyra_amd.build` (hipcc, gfx950). "
            "lyra_amd has no non-HIP code path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means a stale library
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.lyra_abi_version() != ABI_VERSION:
        raise LyraHipError(f"liblyra_hip.so has ABI {lib.lyra_abi_version()}, bindings expect {ABI_VERSION}: rebuild it")
    return lib


lib = _load()


def check(code: int, what: str) -> None:
    if code != 0:
        raise LyraHipError(f"{what}: {lib.lyra_strerror(code).decode()} ({code})")


_WORKSPACES: dict[tuple[str, int, int], "object"] = {}
_SUPERSEDED: list = []  # outgrown buffers stay allocated: a captured HIP graph may still hold their address


def workspace(kind: str, device, stream_ptr: int, nbytes: int):
    """A reusable, zero-initialised device scratch buffer per (operator, device, stream); grows, never shrinks, and a
    buffer that a larger one replaces is never freed (graphs captured earlier replay against it).

    The attention kernel keeps arrival counters in it and returns them to zero, so it is zeroed only when
    allocated and never shared with another operator.
    """
    import torch

    key = (kind, device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _SUPERSEDED.append(buf)
        buf = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = buf
    return buf
