"""The C-ABI shared library: every function include/lyra_hip.h declares is exported, the Python binding table covers
them all, and argument validation answers before anything touches a GPU (no compute is launched here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lyra_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lyra_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("lyra_decode_attention", "lyra_decode_attention_workspace", "lyra_decode_gemm", "lyra_decode_gemm_workspace",
                 "lyra_strerror", "lyra_abi_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from lyra_amd import _lib

    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(raw, name), f"{name} is declared in include/lyra_hip.h but not exported by liblyra_hip.so"
    assert set(_lib.SIGNATURES) == set(declared_functions())


def test_abi_version_and_error_strings():
    from lyra_amd import _lib

    text = open(HEADER).read()
    assert _lib.lib.lyra_abi_version() == int(re.search(r"#define LYRA_ABI_VERSION (\d+)", text).group(1)) == _lib.ABI_VERSION
    seen = set()
    for code in (0, -1, -2, -3, -4, -5):
        msg = _lib.lib.lyra_strerror(code).decode()
        assert msg and msg not in seen
        seen.add(msg)
    with pytest.raises(_lib.LyraHipError):
        _lib.check(-2, "probe")


def test_argument_validation_needs_no_gpu():
    from lyra_amd import _lib

    L = _lib.lib
    bad = L.lyra_decode_attention(None, None, None, None, None, None, None, 0, None, None, None, 0, 1, 16, 4, 512, 128, 0.1, 0, 0, 0, None)
    assert bad == -1
    one = ctypes.c_void_p(256)  # never dereferenced: shapes are rejected first
    assert L.lyra_decode_attention(one, one, one, None, None, one, one, 0, None, one, None, 0, 1, 16, 5, 512, 128, 0.1, 0, 0, 0, None) == -1  # N % K
    assert L.lyra_decode_attention(one, one, one, None, None, one, one, 0, None, one, None, 0, 1, 16, 4, 512, 96, 0.1, 0, 0, 0, None) == -2  # head dim
    assert L.lyra_decode_gemm(None, None, None, 0, 0, None, None, None, None, 0, 4, 1, 64, 128, 0, 0, 0, 1.702, 7.0, None) == -1
    # the attention launch with the front step: neither form of the projection given; a head width it does not cover
    assert L.lyra_decode_attention_qkv(None, None, 0, None, None, one, one, 512, 1e-5, one, one, None, None, one, one, 0, None, one, None, 0,
                                       1, 16, 4, 512, 128, 0.1, 0, 0, 0, None) == -1
    assert L.lyra_decode_attention_qkv(one, None, 0, None, None, one, one, 512, 1e-5, one, one, None, None, one, one, 0, None, one, None, 0,
                                       1, 16, 4, 512, 96, 0.1, 0, 0, 0, None) == -2
    assert L.lyra_decode_gemm(one, one, None, 0, 0, one, None, one, None, 0, 4, 1, 48, 128, 0, 0, 0, 1.702, 7.0, None) == -2  # K % 32
    assert L.lyra_decode_gemm(one, one, None, 0, 0, one, None, one, None, 0, 4, 1, 64, 128, 1, 0, 0, 1.702, 7.0, None) == -1  # fp8 without scales
    assert L.lyra_rmsnorm_proj(None, None, None, None, None, None, 1, 64, 0, 2, 1e-5, None) == -1
    assert L.lyra_rmsnorm_proj_combine(one, one, None, 4, one, 1.0, one, one, one, None, None, None, 1, 64, 0, 2, 1e-5, None) == -1  # no dest
    assert L.lyra_rmsnorm_proj_combine(one, one, one, 17, one, 1.0, one, one, one, None, None, None, 1, 64, 0, 2, 1e-5, None) == -2  # topk > 16
    assert L.lyra_qkv_post(one, None, None, one, one, one, 0, one, one, one, None, None, None, 1, 4, 2, 16, 96, 16, 0, 1e-5, None) == -2
    assert L.lyra_moe_route(one, one, one, one, one, 4, 15, 1, 9, None) == -2  # more than 8 routed picks
    assert L.lyra_moe_combine(None, None, None, None, None, 1, 1, 1, 1.0, None) == -1
    assert L.lyra_argmax(None, None, None, 0, 1, 1, 4, None, None) == -1
    assert L.lyra_argmax(one, one, None, 0, 2, 10, 6, None, None) == -1  # leading dimension shorter than the row


def test_workspace_sizes_are_host_arithmetic():
    from lyra_amd import _lib

    L = _lib.lib
    small = L.lyra_decode_attention_workspace(1, 16, 4, 512, 128, 0)
    big = L.lyra_decode_attention_workspace(64, 16, 4, 4096, 128, 0)
    assert small % 256 == 0 and big % 256 == 0 and small > 0 and big > 0  # (a launch that is not chunked needs no partials)
    assert L.lyra_argmax_workspace(64, 201088) % 256 == 0 and L.lyra_argmax_workspace(0, 5) == 0
    assert L.lyra_decode_attention_workspace(0, 16, 4, 512, 128, 0) == 0
    moe = L.lyra_decode_gemm_workspace(256, 16, 2048, 4096, 1)
    assert moe == 65536 + 256 * 64 * 256 * 4  # arrival counters + one 64-row x 256-column float32 tile slot per workgroup
    splits = L.lyra_decode_gemm_splits(64, 2048, 3072, 2048)
    assert splits >= 2 and L.lyra_decode_gemm_workspace(64, 1, 2048, 3072, 0) == 65536 + splits * 64 * 3072 * 4  # counters + K slices
    assert L.lyra_decode_gemm_splits(64, 2048, 100, 2048) == 0


def test_matmul_workspace_covers_the_launched_plan_for_every_scale_block():
    """lyra_decode_gemm_workspace does not know the scale block, which decides the kernel and its K slices: its answer
    must cover the exact need for every block, including blocks that send a small projection to the general kernel."""
    from lyra_amd import _lib

    L = _lib.lib
    worse = 0
    for M in (1, 16, 64, 128, 256, 300):
        for K in (512, 2048, 4096, 8192, 12288):
            for N in (512, 2048, 4096, 8192, 32768):
                for swiglu in (0, 1):
                    cover = L.lyra_decode_gemm_workspace(M, 1, K, N, swiglu)
                    for bk in (0, 32, 96, 128, 256, 512, 1024, 2048, K):
                        if bk and K % bk:
                            continue
                        need = L.lyra_decode_gemm_workspace_for(M, 1, K, N, bk, swiglu)
                        assert need <= cover, (M, K, N, swiglu, bk, need, cover)
                        worse += need > L.lyra_decode_gemm_workspace_for(M, 1, K, N, 0, swiglu)
    assert worse > 0  # the sweep does contain blocks that need more than the plan without a block
    # three shapes where the launched plan has more K slices than the K-split plan of the same shape
    for (M, K, N, bk, slices) in ((16, 8192, 8192, 1024, 8), (128, 2048, 32768, 1024, 2), (16, 12288, 8192, 96, 32)):
        assert L.lyra_decode_gemm_splits(M, K, N, bk) == 0
        assert L.lyra_decode_gemm_workspace_for(M, 1, K, N, bk, 0) == 65536 + slices * M * N * 4
