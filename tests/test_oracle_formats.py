"""Pins the oracle's number formats and quantiser against torch's dtypes and closed forms.

Covers lyra/nn/quant.py:48-98 as restated in oracle/lyra_oracle.py and oracle/lyra_oracle.c.
"""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O


def _torch_fp8_decode(codes: np.ndarray) -> np.ndarray:
    return torch.from_numpy(codes.astype(np.uint8)).view(torch.float8_e4m3fn).to(torch.float32).numpy()


def _torch_fp8_encode(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x.astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_fp8_decode_all_256_codes_match_torch():
    codes = np.arange(256, dtype=np.uint8)
    want = _torch_fp8_decode(codes)
    got = O.fp8_e4m3fn_decode(codes)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
    lib = clib.load()
    got_c = np.array([lib.lyra_oracle_fp8_e4m3fn_to_f32(int(c)) for c in codes], dtype=np.float32)
    np.testing.assert_array_equal(got_c[~np.isnan(want)], want[~np.isnan(want)])
    assert np.nanmax(got) == 448.0 and got[0x7E] == 448.0  # quant.py:68 fmax
    assert np.isnan(got[0x7F]) and np.isnan(got[0xFF])  # "fn": no infinities


def test_fp8_encode_values_midpoints_and_neighbours_match_torch():
    table = O.fp8_e4m3fn_decode(np.arange(128, dtype=np.uint8))[:127]  # positive finite codes, ascending
    mids = (table[:-1].astype(np.float64) + table[1:].astype(np.float64)) / 2  # exact ties
    eps = np.float32(1e-3)
    pts = np.concatenate([table, mids.astype(np.float32), np.nextafter(mids.astype(np.float32), np.float32(0)),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9)), table * (1 + eps), table * (1 - eps)])
    pts = np.concatenate([pts, -pts, [0.0, -0.0, 2.0**-10, 2.0**-11, 3 * 2.0**-11, 447.9, 448.0]]).astype(np.float32)
    pts = pts[np.abs(pts) <= 448.0]
    want = _torch_fp8_encode(pts)
    got = O.fp8_e4m3fn_encode(pts)
    np.testing.assert_array_equal(got, want)
    lib = clib.load()
    got_c = np.array([lib.lyra_oracle_f32_to_fp8_e4m3fn(float(p)) for p in pts], dtype=np.uint8)
    np.testing.assert_array_equal(got_c, want)


def test_fp8_encode_random_matches_torch():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * rng.choice([1e-3, 0.05, 1.0, 50.0, 200.0], 20000)).astype(np.float32)
    x = np.clip(x, -448, 448)
    np.testing.assert_array_equal(O.fp8_e4m3fn_encode(x), _torch_fp8_encode(x))


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(10000) * 10.0 ** rng.integers(-20, 20, 10000),
                        [0.0, -0.0, 1.0, 1.00390625, 1.0078125, 1.01171875, 3.3895314e38]]).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(O.bf16_round(x), want)
    bits = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(O.bf16_bits(x), bits)
    np.testing.assert_array_equal(O.bf16_from_bits(bits), want)
    lib = clib.load()
    got_c = np.array([lib.lyra_oracle_f32_to_bf16(float(v)) for v in x[:2000]], dtype=np.uint16)
    np.testing.assert_array_equal(got_c, bits[:2000])


def test_quantize_closed_forms():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((3, 5, 8, 64)).astype(np.float32)
    x[1, 2, 3, :] = 0.0  # an all-zero block
    q, s = O.quantize(x, (1, 64))
    assert q.shape == x.shape and s.shape == (3, 5, 8, 1) and s.dtype == np.float32
    amax = np.abs(x).max(-1, keepdims=True)
    np.testing.assert_array_equal(s[amax > 0], (amax[amax > 0] / np.float32(448.0)).astype(np.float32))
    assert s[1, 2, 3, 0] == 1.0  # quant.py:70: amax == 0 -> scale 1
    assert (q[1, 2, 3] == 0).all()
    # the largest-magnitude element of every non-zero block lands on +-448 (code 0x7e / 0xfe)
    idx = np.abs(x).argmax(-1)
    top = np.take_along_axis(q, idx[..., None], -1)[..., 0]
    nz = amax[..., 0] > 0
    assert set(np.unique(top[nz] & 0x7F)) <= {0x7E}
    # dequantised value of that element returns amax to within f32 rounding of (448 * amax/448)
    d = O.dequantize(q, s, (1, 64), to_bf16=False)
    dtop = np.abs(np.take_along_axis(d, idx[..., None], -1))
    np.testing.assert_allclose(dtop[nz[..., None]], amax[nz[..., None]], rtol=2e-7)
    # round-trip error: <= half an ulp (2^-4 relative) in the normal range, <= scale * 2^-10 below it
    err = np.abs(d - x)
    bound = np.maximum(np.abs(x) * 2.0**-4, s * 2.0**-10) * (1 + 1e-6)
    assert (err <= bound).all()


def test_quantize_2d_blocks_and_scale_layout():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((2, 512, 768)) * 0.02).astype(np.float32)
    q, s = O.quantize(w, (256, 256))
    assert s.shape == (2, 2, 3)
    for g in range(2):
        for kb in range(2):
            for nb in range(3):
                blk = w[g, kb * 256 : (kb + 1) * 256, nb * 256 : (nb + 1) * 256]
                assert s[g, kb, nb] == np.float32(np.abs(blk).max()) / np.float32(448.0)
    # per-output-channel = block (K, 1) -> scale [G, 1, N]
    q2, s2 = O.quantize(w, (512, 1))
    assert s2.shape == (2, 1, 768)
    np.testing.assert_array_equal(s2[:, 0, :], (np.abs(w).max(1) / np.float32(448.0)).astype(np.float32))
    with pytest.raises(ValueError):
        O.quantize(w, (300, 256))  # quant.py:37-39


def test_quantize_matches_torch_elementwise():
    """clip(x * (1/scale)) -> fp8 cast: same codes as doing the same steps with torch dtypes."""
    rng = np.random.default_rng(4)
    x = rng.standard_normal((4, 7, 128)).astype(np.float32)
    q, s = O.quantize(x, (1, 128))
    inv = (np.float32(1.0) / s).astype(np.float32)
    scaled = np.clip((x * inv).astype(np.float32), -448, 448)
    np.testing.assert_array_equal(q, _torch_fp8_encode(scaled))
    d = O.dequantize(q, s, (1, 128))
    want = torch.from_numpy(_torch_fp8_decode(q) * s).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(d, want)
    # C row quantiser agrees bit for bit
    lib = clib.load()
    qc = np.empty_like(q)
    sc = np.empty(s.size, dtype=np.float32)
    xf = np.ascontiguousarray(x.reshape(-1, 128))
    lib.lyra_oracle_quantize_rows(xf.ctypes.data, xf.shape[0], 128, qc.ctypes.data, sc.ctypes.data)
    np.testing.assert_array_equal(qc, q)
    np.testing.assert_array_equal(sc, s.reshape(-1))


def test_c_block_quantiser_matches_numpy():
    rng = np.random.default_rng(6)
    w = (rng.standard_normal((3, 512, 256)) * 0.02).astype(np.float32)
    w[1, :256, :128] = 0.0
    for block in ((256, 256), (512, 1), (64, 64), (512, 128)):
        q, s = O.quantize(w, block)
        qc, sc = clib.quantize_blocks(w, block)
        np.testing.assert_array_equal(qc, q)
        np.testing.assert_array_equal(sc, s)
    with pytest.raises(ValueError):
        clib.quantize_blocks(w, (300, 256))


def test_qupdate_writes_one_token():
    rng = np.random.default_rng(5)
    cache = rng.standard_normal((2, 3, 16, 64)).astype(np.float32)
    q, s = O.quantize(cache, (1, 64))
    new = rng.standard_normal((2, 3, 1, 64)).astype(np.float32)
    q2, s2 = O.qupdate(q, s, (1, 64), new, (0, 0, 5, 0))
    qn, sn = O.quantize(new, (1, 64))
    np.testing.assert_array_equal(q2[:, :, 5:6], qn)
    np.testing.assert_array_equal(s2[:, :, 5:6], sn)
    keep = np.ones(16, bool)
    keep[5] = False
    np.testing.assert_array_equal(q2[:, :, keep], q[:, :, keep])
    np.testing.assert_array_equal(s2[:, :, keep], s[:, :, keep])


# ---- the second 1-byte format of the reference's FP8_DTYPES (lyra/nn/quant.py:10): e5m2 -------------------------------
def _torch_e5m2_decode(codes: np.ndarray) -> np.ndarray:
    return torch.from_numpy(codes.astype(np.uint8)).view(torch.float8_e5m2).to(torch.float32).numpy()


def _torch_e5m2_encode(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x.astype(np.float32)).to(torch.float8_e5m2).view(torch.uint8).numpy()


def test_e5m2_decode_all_256_codes_match_torch_and_float16():
    codes = np.arange(256, dtype=np.uint8)
    want = _torch_e5m2_decode(codes)
    got = O.fp8_decode(codes, 2)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
    # the format is the upper byte of IEEE float16: a second, independent definition
    half = (codes.astype(np.uint16) << 8).view(np.float16).astype(np.float32)
    np.testing.assert_array_equal(got[~np.isnan(want)], half[~np.isnan(want)])
    lib = clib.load()
    got_c = np.array([lib.lyra_oracle_fp8_e5m2_to_f32(int(c)) for c in codes], dtype=np.float32)
    np.testing.assert_array_equal(got_c[~np.isnan(want)], want[~np.isnan(want)])
    assert got[0x7B] == 57344.0 and np.isinf(got[0x7C]) and np.isnan(got[0x7D])  # finfo(float8_e5m2).max, then inf / NaN
    assert O.fp8_max(2) == float(torch.finfo(torch.float8_e5m2).max) and O.fp8_max(1) == float(torch.finfo(torch.float8_e4m3fn).max)


def test_e5m2_encode_values_midpoints_and_neighbours_match_torch():
    table = O.fp8_decode(np.arange(0x7C, dtype=np.uint8), 2)  # positive finite codes, ascending
    mids = (table[:-1].astype(np.float64) + table[1:].astype(np.float64)) / 2  # exact ties
    eps = np.float32(1e-3)
    pts = np.concatenate([table, mids.astype(np.float32), np.nextafter(mids.astype(np.float32), np.float32(0)),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9)), table * (1 + eps), table * (1 - eps)])
    pts = np.concatenate([pts, -pts, [0.0, -0.0, 2.0**-17, 2.0**-18, 3 * 2.0**-18, 57343.0, 57344.0]]).astype(np.float32)
    pts = pts[np.abs(pts) <= 57344.0]
    want = _torch_e5m2_encode(pts)
    got = O.fp8_encode(pts, 2)
    np.testing.assert_array_equal(got, want)
    lib = clib.load()
    got_c = np.array([lib.lyra_oracle_f32_to_fp8_e5m2(float(p)) for p in pts], dtype=np.uint8)
    np.testing.assert_array_equal(got_c, want)
    rng = np.random.default_rng(10)
    x = (rng.standard_normal(20000) * rng.choice([1e-5, 1e-3, 1.0, 300.0, 20000.0], 20000)).astype(np.float32)
    x = np.clip(x, -57344, 57344)
    np.testing.assert_array_equal(O.fp8_encode(x, 2), _torch_e5m2_encode(x))


def test_e5m2_quantize_matches_torch_elementwise_and_c():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4, 7, 128)).astype(np.float32)
    x[2, 3] = 0.0
    q, s = O.quantize(x, (1, 128), fmt=2)
    amax = np.abs(x).max(-1, keepdims=True)
    np.testing.assert_array_equal(s[amax > 0], (amax[amax > 0] / np.float32(57344.0)).astype(np.float32))
    assert s[2, 3, 0] == 1.0 and (q[2, 3] == 0).all()
    inv = (np.float32(1.0) / s).astype(np.float32)
    scaled = np.clip((x * inv).astype(np.float32), -57344, 57344)
    np.testing.assert_array_equal(q, _torch_e5m2_encode(scaled))
    d = O.dequantize(q, s, (1, 128), fmt=2)
    want = torch.from_numpy(_torch_e5m2_decode(q) * s).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(d, want)
    qc, sc = clib.quantize_rows(x, fp8_format=2)
    np.testing.assert_array_equal(qc, q)
    np.testing.assert_array_equal(sc, s)
    # round-trip error: half an ulp of 2 mantissa bits (2^-3 relative) in the normal range
    err = np.abs(O.dequantize(q, s, (1, 128), to_bf16=False, fmt=2) - x)
    assert (err <= np.maximum(np.abs(x) * 2.0**-3, s * 2.0**-17) * (1 + 1e-6)).all()
    w = (rng.standard_normal((2, 256, 256)) * 0.02).astype(np.float32)
    for block in ((256, 256), (256, 1), (64, 128)):
        qn, sn = O.quantize(w, block, fmt=2)
        qb, sb = clib.quantize_blocks(w, block, fp8_format=2)
        np.testing.assert_array_equal(qb, qn)
        np.testing.assert_array_equal(sb, sn)


def test_e5m2_operators_of_the_c_oracle_match_numpy():
    """The C attention and matmul read e5m2 codes through the table pinned above: same results as the numpy forms."""
    rng = np.random.default_rng(12)
    B, N, K, S, H = 2, 4, 2, 96, 64
    q = O.bf16_round(rng.standard_normal((B, N, 1, H)).astype(np.float32))
    kq, ks = O.quantize(rng.standard_normal((B, K, S, H)).astype(np.float32), (1, H), fmt=2)
    vq, vs = O.quantize(rng.standard_normal((B, K, S, H)).astype(np.float32), (1, H), fmt=2)
    sinks = rng.standard_normal(N).astype(np.float32)
    pos = np.array([S - 1, 40])
    want = O.decode_attention_reference(q, (kq, ks), (vq, vs), sinks, H**-0.5, 0, pos, fp8_format=2)
    got = clib.decode_attention(O.bf16_bits(q), kq, vq, ks, vs, sinks, pos, None, H**-0.5, 0, fp8_format=2)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6)
    other = clib.decode_attention(O.bf16_bits(q), kq, vq, ks, vs, sinks, pos, None, H**-0.5, 0, fp8_format=1)
    assert np.abs(other - want).max() > 1e-2  # (the format argument is not ignored)
    M, G, Kd, Nd = 12, 3, 64, 32
    lhs = O.bf16_round(rng.standard_normal((M, Kd)).astype(np.float32))
    wq, wsc = O.quantize((rng.standard_normal((G, Kd, Nd)) * 0.05).astype(np.float32), (32, 16), fmt=2)
    sizes = np.array([5, 0, 7], dtype=np.int32)
    want = O.decode_gemm_reference(lhs, (wq, wsc), sizes, block=(32, 16), fp8_format=2)
    got = clib.decode_gemm(O.bf16_bits(lhs), wq, wsc, (32, 16), sizes, None, fp8_format=2)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6)
