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
