"""Shared helpers of the GPU parity tests: seeded inputs as numpy (for the oracle) and torch (for the kernels)."""
from __future__ import annotations

import numpy as np
import torch

from oracle import lyra_oracle as O

# Acceptance tolerance of the decode kernels against the fp32 oracle:
# |got - want| <= 2e-2 + 1e-2 * |want| elementwise (bf16 outputs, FP8 paths after identical dequantisation).
ATOL, RTOL = 2e-2, 1e-2


def dev():
    return torch.device("cuda:0")


def t_bf16(x: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev()).to(torch.bfloat16)


def t_f32(x: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev())


def t_fp8(codes: np.ndarray, fmt: int = 1) -> torch.Tensor:
    """Device tensor of 1-byte codes; fmt 1: e4m3fn, 2: e5m2 (the format numbers of the oracle)."""
    dt = torch.float8_e5m2 if fmt == 2 else torch.float8_e4m3fn
    return torch.from_numpy(np.ascontiguousarray(codes, dtype=np.uint8)).to(dev()).view(dt)


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().to(torch.float32).cpu().numpy()


def quantize_rows(x: np.ndarray, fmt: int = 1):
    """Block (1,H) quantiser through the C oracle (bit-identical to oracle.quantize, much faster on big caches)."""
    from oracle import clib

    return clib.quantize_rows(x, fp8_format=fmt)


def attention_case(seed, B, N, K, S, H, *, fp8, q_scale=1.0, fmt=1):
    """Q/K/V ~ N(0,1) rounded to bf16, sinks ~ N(0,1); FP8 cache quantised per token and kv head (block (1,H)) to format
    ``fmt`` (1: e4m3fn, 2: e5m2)."""
    rng = np.random.default_rng(seed)
    q = O.bf16_round((rng.standard_normal((B, N, 1, H)) * q_scale).astype(np.float32))
    k = O.bf16_round(rng.standard_normal((B, K, S, H), dtype=np.float32))
    v = O.bf16_round(rng.standard_normal((B, K, S, H), dtype=np.float32))
    sinks = rng.standard_normal(N).astype(np.float32)
    case = {"q": q, "sinks": sinks, "fp8": fp8, "fmt": fmt}
    if fp8:
        big = k.size > (1 << 22)
        kq, ks = quantize_rows(k, fmt) if big else O.quantize(k, (1, H), fmt)
        vq, vs = quantize_rows(v, fmt) if big else O.quantize(v, (1, H), fmt)
        case.update(k=(kq, ks), v=(vq, vs))
    else:
        case.update(k=k, v=v)
    return case


def attention_torch_inputs(case):
    from lyra_amd.nn.quant import QArray

    q = t_bf16(case["q"])
    sinks = t_f32(case["sinks"])
    if case["fp8"]:
        (kq, ks), (vq, vs) = case["k"], case["v"]
        H = kq.shape[-1]
        k = QArray(t_fp8(kq, case.get("fmt", 1)), t_f32(ks), (1, H))
        v = QArray(t_fp8(vq, case.get("fmt", 1)), t_f32(vs), (1, H))
    else:
        k, v = t_bf16(case["k"]), t_bf16(case["v"])
    return q, k, v, sinks


def assert_close(got: np.ndarray, want: np.ndarray, atol=ATOL, rtol=RTOL, what=""):
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    bound = atol + rtol * np.abs(want)
    worst = int(np.argmax(err - bound))
    assert (err <= bound).all(), (
        f"{what}: max abs err {err.max():.4g}, worst at flat index {worst}: got {got.flat[worst]:.6g} want {want.flat[worst]:.6g}"
    )
