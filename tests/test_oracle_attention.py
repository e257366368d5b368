"""Pins the decode-attention oracle (lyra/kernels/decode_attention.py:63-69,263-361).

Independent anchors: torch SDPA / softmax with the sink as one extra key of value 0,
limits in the sink, brute-force window arithmetic over every position, a one-hot
GQA head-mapping probe, and the input vector of the reference's own
tests/test_decode_attention.py:54-65.
"""
import math

import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O


def _rand_case(rng, B, N, K, S, H):
    q = O.bf16_round(rng.standard_normal((B, N, 1, H)).astype(np.float32))
    k = O.bf16_round(rng.standard_normal((B, K, S, H)).astype(np.float32))
    v = O.bf16_round(rng.standard_normal((B, K, S, H)).astype(np.float32))
    sinks = rng.standard_normal(N).astype(np.float32)
    return q, k, v, sinks


def _sdpa_with_sink_key(q, k, v, sinks, sm_scale, sw, pos):
    """Library route: append a key whose logit is the sink and whose value is 0."""
    B, N, _, H = q.shape
    _, K, S, _ = k.shape
    G = N // K
    tq = torch.from_numpy(q).double()  # [B,N,1,H]
    tk = torch.from_numpy(k).double().repeat_interleave(G, dim=1)  # head n -> kv head n // G
    tv = torch.from_numpy(v).double().repeat_interleave(G, dim=1)
    tv = torch.cat([tv, torch.zeros(B, N, 1, H, dtype=torch.float64)], dim=2)
    logits = (tq @ tk.transpose(-1, -2)) * sm_scale  # [B,N,1,S]
    mask = torch.from_numpy(O.visible_mask(pos, sw, S))
    logits = logits.masked_fill(~mask[None, None, None, :], float("-inf"))
    sink_col = torch.from_numpy(sinks).double().reshape(1, N, 1, 1).expand(B, N, 1, 1)
    p = torch.softmax(torch.cat([logits, sink_col], dim=-1), dim=-1)
    return (p @ tv).float().numpy()


@pytest.mark.parametrize("sw,pos,S", [(0, 511, 512), (0, 100, 512), (128, 511, 512), (128, 5, 512), (128, 300, 384), (128, 255, 256), (1, 17, 512)])
def test_attention_equals_softmax_with_extra_sink_key(sw, pos, S):
    rng = np.random.default_rng(10 + sw + pos)
    q, k, v, sinks = _rand_case(rng, 2, 8, 2, S, 64)
    got = O.decode_attention_reference(q, k, v, sinks, 0.125, sw, pos)
    want = _sdpa_with_sink_key(q, k, v, sinks, 0.125, sw, pos)
    np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)


def test_sink_limits_and_closed_form():
    rng = np.random.default_rng(11)
    q, k, v, _ = _rand_case(rng, 1, 4, 2, 128, 32)
    sm = 32**-0.5
    # sink -> -inf: ordinary softmax attention
    got = O.decode_attention_reference(q, k, v, np.full(4, -1e30, np.float32), sm, 0, 127)
    tq, tk, tv = (torch.from_numpy(a) for a in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(
        tq, tk.repeat_interleave(2, 1), tv.repeat_interleave(2, 1), scale=sm
    ).numpy()
    np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)
    # sink -> +inf: all weight goes to the (zero-valued) sink
    got = O.decode_attention_reference(q, k, v, np.full(4, 1e4, np.float32), sm, 0, 127)
    assert np.abs(got).max() == 0.0
    # all keys identical: out = mean(V_vis) * n / (n + exp(sink - s))
    kk = np.broadcast_to(k[:, :, :1], k.shape).copy()
    sinks = np.array([0.3, -0.7, 1.1, 0.0], np.float32)
    pos = 49
    got = O.decode_attention_reference(q, kk, v, sinks, sm, 0, pos)
    n = pos + 1
    for head in range(4):
        s = float(q[0, head, 0] @ kk[0, head // 2, 0]) * sm
        want = v[0, head // 2, :n].mean(0) * n / (n + np.exp(sinks[head] - s))
        np.testing.assert_allclose(got[0, head, 0], want, rtol=2e-5, atol=2e-6)


def test_reference_repo_test_vector():
    """tests/test_decode_attention.py:54-65: q=1, kv=1, sinks=0, scale 1, position 0, H=128.

    The reference asserts only the shape; the closed form is 1/(1+exp(-128)) == 1.0.
    """
    q = np.ones((1, 2, 1, 128), np.float32)
    kv = np.ones((1, 1, 128, 128), np.float32)
    out = O.decode_attention_reference(q, kv, kv, np.zeros(2, np.float32), 1.0, 0, 0)
    assert out.shape == q.shape
    np.testing.assert_array_equal(out, np.ones_like(q))


def test_gqa_head_mapping_one_hot_values():
    B, N, K, S, H = 1, 12, 3, 16, 8
    q = np.zeros((B, N, 1, H), np.float32)
    k = np.zeros((B, K, S, H), np.float32)
    v = np.zeros((B, K, S, H), np.float32)
    for kh in range(K):
        v[0, kh, :, kh] = 1.0  # kv head kh writes only column kh
    out = O.decode_attention_reference(q, k, v, np.full(N, -1e30, np.float32), 1.0, 0, S - 1)
    for n in range(N):
        want = np.zeros(H, np.float32)
        want[n // (N // K)] = 1.0
        np.testing.assert_allclose(out[0, n, 0], want, atol=1e-6)


def test_window_arithmetic_brute_force():
    """decode_window / is_sw / slab start (:63-69, :277-280) against enumeration; bit-exact."""
    lib = clib.load()
    assert O.decode_window(128) == 256 and O.decode_window(1) == 128 and O.decode_window(129) == 256
    assert O.decode_window(130) == 384 and O.decode_window(256) == 384
    assert not O.is_sw(128, 256) and O.is_sw(128, 384) and not O.is_sw(0, 4096)
    for S in (128, 256, 384, 512, 4096):
        for sw in (0, 1, 127, 128, 129, 256):
            assert lib.lyra_oracle_decode_window(sw) == O.decode_window(sw)
            assert bool(lib.lyra_oracle_is_sw(sw, S)) == O.is_sw(sw, S)
            step = 1 if S <= 512 else 37
            for pos in list(range(0, S, step)) + [S - 1]:
                vis = O.visible_mask(pos, sw, S)
                lo, hi = O.visible_range(pos, sw, S)
                want_n = min(sw, pos + 1) if sw > 0 else pos + 1
                assert vis.sum() == want_n == hi - lo + 1
                assert vis[lo] and vis[hi] and (lo == 0 or not vis[lo - 1]) and (hi == S - 1 or not vis[hi + 1])
                if O.is_sw(sw, S):
                    start = O.sliding_start(pos, sw, S)
                    assert lib.lyra_oracle_sliding_start(pos, sw, S) == start
                    wlen = O.decode_window(sw)
                    # the slab is block aligned, inside the cache, and contains every visible key
                    assert start % 128 == 0 and 0 <= start and start + wlen <= S
                    assert start <= lo and hi < start + wlen
                    # first-visible-key formula: floor((pos-sw+1)/128)*128 clipped
                    first = pos - sw + 1
                    assert start == min(max((first // 128) * 128, 0), S - wlen)


def test_slab_path_equals_full_mask_path():
    """sliding_decode reads a slab; the result must equal masking the full cache."""
    rng = np.random.default_rng(12)
    S, sw = 512, 128
    q, k, v, sinks = _rand_case(rng, 1, 4, 2, S, 32)
    for pos in (0, 5, 127, 128, 129, 255, 256, 300, 511):
        assert O.is_sw(sw, S)
        got = O.decode_attention_reference(q, k, v, sinks, 0.2, sw, pos)
        want = _sdpa_with_sink_key(q, k, v, sinks, 0.2, sw, pos)
        np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)


def test_fp8_cache_path_dequantises_first():
    rng = np.random.default_rng(13)
    q, k, v, sinks = _rand_case(rng, 2, 8, 2, 256, 64)
    kq, ks = O.quantize(k, (1, 64))
    vq, vs = O.quantize(v, (1, 64))
    for mode, bf in (("fp32", False), ("ref", True)):
        kd = O.dequantize(kq, ks, (1, 64), to_bf16=bf)
        vd = O.dequantize(vq, vs, (1, 64), to_bf16=bf)
        a = O.decode_attention_reference(q, (kq, ks), (vq, vs), sinks, 0.125, 0, 200, mode=mode)
        b = O.decode_attention_reference(q, kd, vd, sinks, 0.125, 0, 200, mode=mode)
        np.testing.assert_array_equal(a, b)
    # the bf16 rounding points of the JAX code move the result by well under the acceptance tolerance
    f = O.decode_attention_reference(q, (kq, ks), (vq, vs), sinks, 0.125, 0, 200, mode="fp32")
    r = O.decode_attention_reference(q, (kq, ks), (vq, vs), sinks, 0.125, 0, 200, mode="ref")
    assert np.abs(f - r).max() < 1e-2


def test_ragged_positions_are_per_row_scalars():
    rng = np.random.default_rng(14)
    q, k, v, sinks = _rand_case(rng, 3, 4, 2, 256, 32)
    pos = np.array([7, 255, 100])
    got = O.decode_attention_reference(q, k, v, sinks, 0.2, 0, pos)
    for b in range(3):
        one = O.decode_attention_reference(q[b : b + 1], k[b : b + 1], v[b : b + 1], sinks, 0.2, 0, int(pos[b]))
        np.testing.assert_array_equal(got[b : b + 1], one)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("sw", [0, 128])
def test_c_oracle_matches_numpy_oracle(fp8, sw):
    rng = np.random.default_rng(15)
    B, N, K, S, H = 3, 8, 2, 512, 64
    q, k, v, sinks = _rand_case(rng, B, N, K, S, H)
    pos = np.array([511, 3, 260])
    gate = O.bf16_round(2.0 / (1.0 + np.exp(-rng.standard_normal((B, N)))).astype(np.float32))
    if fp8:
        kq, ks = O.quantize(k, (1, H))
        vq, vs = O.quantize(v, (1, H))
        kn, vn = (kq, ks), (vq, vs)
        kc, vc, ksc, vsc = kq, vq, ks[..., 0], vs[..., 0]
    else:
        kn, vn = k, v
        kc, vc, ksc, vsc = O.bf16_bits(k), O.bf16_bits(v), None, None
    for mode in ("fp32", "ref"):
        want = O.decode_attention_reference(q, kn, vn, sinks, H**-0.5, sw, pos, mode=mode, gate=gate)
        got = clib.decode_attention(O.bf16_bits(q), kc, vc, ksc, vsc, sinks, pos, gate, H**-0.5, sw, ref_rounding=(mode == "ref"))
        # summation order differs (einsum vs sequential); "ref" may flip a bf16 ulp
        tol = 2e-5 if mode == "fp32" else 1.6e-2
        np.testing.assert_allclose(got, want, atol=tol, rtol=tol)


# ---- learned exclusive self attention (lyra/model.py:351-363) ----------------------------------------------
def _xsa_case(seed, B=2, N=8, K=2, H=8):
    rng = np.random.default_rng(seed)
    t = rng.standard_normal((B, N, H)).astype(np.float32)
    v = rng.standard_normal((B, K, H)).astype(np.float32)
    alpha = rng.standard_normal(N).astype(np.float32)
    return t, v, alpha


def test_xsa_closed_forms():
    t, v, alpha = _xsa_case(0)
    B, N, H = t.shape
    K = v.shape[1]
    G = N // K
    # alpha = 0: tanh(0) = 0, nothing is removed
    assert np.array_equal(O.xsa(t, v, np.zeros(N, np.float32)), t)
    # unit rows have length 1 (the 1e-10 only matters for a zero row, which stays zero)
    vn = O.unit_rows(v)
    np.testing.assert_allclose(np.sum(vn * vn, -1), 1.0, atol=1e-6)
    assert np.array_equal(O.unit_rows(np.zeros((1, 1, H), np.float32)), np.zeros((1, 1, H), np.float32))
    # t parallel to v^ and tanh(alpha) -> 1: everything is removed
    par = np.repeat(3.0 * vn, G, axis=1)  # head n takes kv head n // G
    out = O.xsa(par, v, np.full(N, 20.0, np.float32))
    assert np.abs(out).max() < 1e-5
    # the orthogonal component is untouched, the parallel one is scaled by 1 - tanh(alpha)
    out = O.xsa(t, v, alpha)
    vg = np.repeat(vn, G, axis=1)
    dot_in, dot_out = np.sum(t * vg, -1), np.sum(out * vg, -1)
    np.testing.assert_allclose(dot_out, dot_in * (1.0 - np.tanh(alpha))[None, :], atol=1e-5)
    np.testing.assert_allclose(out - dot_out[..., None] * vg, t - dot_in[..., None] * vg, atol=1e-5)
    # sign: a positive alpha shrinks the component along v^ (a wrong sign would grow it)
    pos = O.xsa(par, v, np.full(N, 0.5, np.float32))
    assert (np.sum(pos * vg, -1) < np.sum(par * vg, -1)).all()


def test_xsa_scalar_loops_and_head_mapping():
    t, v, alpha = _xsa_case(1, B=2, N=6, K=3, H=8)
    B, N, H = t.shape
    K = v.shape[1]
    G = N // K
    want = np.zeros_like(t)
    for b in range(B):
        for n in range(N):
            k = n // G
            norm2 = sum(float(v[b, k, h]) ** 2 for h in range(H)) + 1e-10
            unit = [float(v[b, k, h]) / math.sqrt(norm2) for h in range(H)]
            coef = sum(float(t[b, n, h]) * unit[h] for h in range(H))
            for h in range(H):
                want[b, n, h] = float(t[b, n, h]) - math.tanh(float(alpha[n])) * coef * unit[h]
    np.testing.assert_allclose(O.xsa(t, v, alpha), want, atol=1e-5)
    # one-hot value rows: kv head k points along axis k, so head n loses exactly its component along axis n // G
    v1 = np.zeros((B, K, H), np.float32)
    for k in range(K):
        v1[:, k, k] = 2.0
    out = O.xsa(t, v1, np.full(N, 20.0, np.float32))
    for n in range(N):
        keep = np.ones(H, bool)
        keep[n // G] = False
        assert np.abs(out[:, n, n // G]).max() < 1e-5
        assert np.array_equal(out[:, n, keep], t[:, n, keep])


def test_xsa_bf16_flow_stays_close_to_float32():
    rng = np.random.default_rng(2)
    t = O.bf16_round(rng.standard_normal((3, 16, 128)).astype(np.float32))
    v = O.bf16_round(rng.standard_normal((3, 4, 128)).astype(np.float32))
    alpha = rng.standard_normal(16).astype(np.float32)
    a, b = O.xsa(t, v, alpha, mode="ref"), O.xsa(t, v, alpha)
    assert np.array_equal(a, O.bf16_round(a))
    assert np.abs(a - b).max() <= 2e-2 + 1e-2 * np.abs(b).max()
