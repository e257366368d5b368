"""Pins the decode-GEMM oracle (decode_gemm.py:368-401, gemm.py:393-400,450-456,1575-1617,
common.py:98-114) and the integer routing helpers (model.py:451-491,557).
"""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O


def test_expert_ids_and_padding_rule():
    np.testing.assert_array_equal(O.expert_ids([2, 0, 3], 5), [0, 0, 2, 2, 2])
    np.testing.assert_array_equal(O.expert_ids([1, 1], 2), [0, 1])
    # rows beyond sum(group_sizes): every group start <= the sum, so the gather lands on G-1
    np.testing.assert_array_equal(O.expert_ids([2, 0, 0], 4), [0, 0, 2, 2])
    np.testing.assert_array_equal(O.expert_ids([1, 0, 1, 0], 4), [0, 2, 3, 3])


def test_normalize_bias_shapes():
    assert O.normalize_bias(None, 3, 8).shape == (3, 1, 8)
    assert O.normalize_bias(np.ones((3, 8)), 3, 8).shape == (3, 1, 8)
    with pytest.raises(ValueError):
        O.normalize_bias(np.ones((3, 2, 8)), 3, 8)


def test_swiglu_closed_forms():
    # zero gate -> 0 whatever the linear half
    assert O.swiglu(np.array([[0.0, 5.0]], np.float32))[0, 0] == 0.0
    # gate clamp at 7 (min only), linear clamp at +-7, +1 shift
    x = np.array([[100.0, 100.0], [100.0, -100.0], [-100.0, 3.0], [2.0, -1.0]], np.float32)
    y = O.swiglu(x)
    sig7 = 1.0 / (1.0 + np.exp(-1.702 * 7.0))
    np.testing.assert_allclose(y[0, 0], (7.0 + 1.0) * 7.0 * sig7, rtol=1e-6)
    np.testing.assert_allclose(y[1, 0], (-7.0 + 1.0) * 7.0 * sig7, rtol=1e-6)
    np.testing.assert_allclose(y[2, 0], (3.0 + 1.0) * -100.0 / (1.0 + np.exp(170.2)), rtol=1e-5, atol=1e-30)
    assert y[3, 0] == 0.0  # lin = -1 -> (lin + 1) = 0
    # first half gates, second half is linear (split, not interleave): common.py:109
    z = O.swiglu(np.array([[1.0, 2.0, 10.0, 20.0]], np.float32))
    sig = lambda g: 1.0 / (1.0 + np.exp(-1.702 * g))
    np.testing.assert_allclose(z[0], [(7.0 + 1) * 1.0 * sig(1.0), (7.0 + 1) * 2.0 * sig(2.0)], rtol=1e-6)
    # against torch's own sigmoid
    rng = np.random.default_rng(0)
    a = (rng.standard_normal((5, 64)) * 4).astype(np.float32)
    t = torch.from_numpy(a)
    g, l = t[:, :32].clamp(max=7.0), t[:, 32:].clamp(-7.0, 7.0)
    np.testing.assert_allclose(O.swiglu(a), ((l + 1) * g * torch.sigmoid(1.702 * g)).numpy(), rtol=2e-6, atol=1e-7)


@pytest.mark.parametrize("sizes,M", [([3, 0, 2, 1], 6), ([0, 0, 4, 0], 4), ([1, 1, 1, 1], 4), ([2, 1, 0, 0], 5)])
def test_grouped_gemm_is_per_group_matmul(sizes, M):
    rng = np.random.default_rng(1)
    G, K, N = len(sizes), 32, 16
    lhs = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    rhs = O.bf16_round(rng.standard_normal((G, K, N)).astype(np.float32))
    bias = rng.standard_normal((G, N)).astype(np.float32)
    got = O.grouped_gemm_reference(lhs, rhs, np.array(sizes), bias=bias)
    want = np.zeros((M, N), np.float32)
    row = 0
    for g, n in enumerate(sizes):
        for _ in range(n):
            want[row] = (torch.from_numpy(lhs[row]).double() @ torch.from_numpy(rhs[g]).double()).float().numpy() + bias[g]
            row += 1
    for r in range(row, M):  # padding rows: zero product + bias of expert G-1
        want[r] = bias[G - 1]
    np.testing.assert_allclose(got, want, atol=1e-5, rtol=1e-5)


def test_brute_force_tiny_with_swiglu():
    rng = np.random.default_rng(2)
    M, G, K, N = 3, 2, 4, 6
    lhs = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    rhs = O.bf16_round(rng.standard_normal((G, K, N)).astype(np.float32))
    sizes = np.array([1, 2])
    got = O.decode_gemm_reference(lhs, rhs, sizes, fused_swiglu=True)
    ids = [0, 1, 1]
    for r in range(M):
        t = [sum(float(lhs[r, k]) * float(rhs[ids[r], k, n]) for k in range(K)) for n in range(N)]
        for j in range(N // 2):
            glu, lin = min(t[j], 7.0), max(-7.0, min(7.0, t[N // 2 + j]))
            want = (lin + 1.0) * glu / (1.0 + np.exp(-1.702 * glu))
            np.testing.assert_allclose(got[r, j], want, rtol=1e-5, atol=1e-6)


def test_fp8_weights_dequantise_to_bf16_first():
    rng = np.random.default_rng(3)
    M, G, K, N = 5, 3, 512, 256
    lhs = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    w = (rng.standard_normal((G, K, N)) * 0.02).astype(np.float32)
    sizes = np.array([2, 0, 3])
    for block in ((256, 256), (K, 1)):
        q, s = O.quantize(w, block)
        wd = O.dequantize(q, s, block, to_bf16=True)
        a = O.decode_gemm_reference(lhs, (q, s), sizes, block=block, mode="ref")
        b = O.grouped_gemm_reference(lhs, wd, sizes, mode="ref")
        np.testing.assert_array_equal(a, b)
        f = O.decode_gemm_reference(lhs, (q, s), sizes, block=block, mode="fp32")
        assert np.abs(f - a).max() < 2e-2
    assert O.default_weight_block(2048, 4096) == (256, 256) and O.default_weight_block(2880, 2880) == (64, 64)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("swiglu", [False, True])
def test_c_oracle_matches_numpy_oracle(fp8, swiglu):
    rng = np.random.default_rng(4)
    M, G, K, N = 9, 4, 512, 256
    lhs = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    w = (rng.standard_normal((G, K, N)) * 0.05).astype(np.float32)
    bias = rng.standard_normal((G, N)).astype(np.float32)
    sizes = np.array([4, 0, 1, 3], np.int32)  # one padding row
    for mode in ("fp32", "ref"):
        if fp8:
            q, s = O.quantize(w, (256, 256))
            want = O.decode_gemm_reference(lhs, (q, s), sizes, block=(256, 256), bias=bias, fused_swiglu=swiglu, mode=mode)
            got = clib.decode_gemm(O.bf16_bits(lhs), q, s, (256, 256), sizes, bias, fused_swiglu=swiglu, ref_rounding=(mode == "ref"))
        else:
            wb = O.bf16_round(w)
            want = O.decode_gemm_reference(lhs, wb, sizes, bias=bias, fused_swiglu=swiglu, mode=mode)
            got = clib.decode_gemm(O.bf16_bits(lhs), O.bf16_bits(wb), None, None, sizes, bias, fused_swiglu=swiglu, ref_rounding=(mode == "ref"))
        tol = 3e-5 if mode == "fp32" else 1.6e-2
        np.testing.assert_allclose(got, want, atol=tol, rtol=tol)


def test_routing_topk_softmax_bincount():
    logits = np.array([[0.1, 2.0, 2.0, -1.0, 0.5], [3.0, -2.0, 0.0, 3.0, 3.0]], np.float32)
    scores, active, groups = O.route_tokens(logits, 3, 5, 1)
    # stable top-k: ties resolve to the lower index (lax.top_k)
    np.testing.assert_array_equal(active.reshape(2, 4), [[1, 2, 4, 5], [0, 3, 4, 5]])
    np.testing.assert_allclose(scores[0, :3], torch.softmax(torch.tensor([2.0, 2.0, 0.5]), 0).numpy(), rtol=1e-6)
    np.testing.assert_array_equal(scores[:, 3], [1.0, 1.0])  # shared expert joins with score 1 (model.py:476)
    np.testing.assert_array_equal(groups, [1, 1, 1, 1, 2, 2])


def test_bpermute_is_stable_counting_sort():
    # input vector of the reference's tests/test_combine.py:13-15
    assignments = np.array([0, 2, 4, 7, 1, 3, 4, 7], np.int32)
    groups = np.bincount(assignments, minlength=8)
    perm, dest = O.bpermute(assignments, groups, 8)
    np.testing.assert_array_equal(perm, np.argsort(assignments, kind="stable"))
    np.testing.assert_array_equal(perm, [0, 4, 1, 5, 2, 6, 3, 7])
    np.testing.assert_array_equal(dest[perm], np.arange(8))
    rng = np.random.default_rng(5)
    for _ in range(20):
        a = rng.integers(0, 6, 40)
        perm, dest = O.bpermute(a, np.bincount(a, minlength=6), 6)
        np.testing.assert_array_equal(perm, np.argsort(a, kind="stable"))
        np.testing.assert_array_equal(np.argsort(perm), dest)


def test_combine_weighted_sum():
    rng = np.random.default_rng(6)
    F, k, C, E = 4, 3, 8, 5
    a = rng.integers(0, E, F * k)
    perm, dest = O.bpermute(a, np.bincount(a, minlength=E), E)
    tokens = rng.standard_normal((F, C)).astype(np.float32)
    rows = tokens[perm // k]  # model.py:521
    scores = rng.random((F, k)).astype(np.float32)
    got = O.combine(rows, scores, dest)
    np.testing.assert_allclose(got, tokens * scores.sum(-1, keepdims=True), rtol=1e-5, atol=1e-6)


def test_rms_norm_and_rotate_against_torch():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    w = rng.standard_normal(64).astype(np.float32)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x), (64,), torch.from_numpy(w), eps=1e-5).numpy()
    np.testing.assert_allclose(O.rms_norm(x, w, 1e-5), want, rtol=2e-6, atol=1e-6)
    cos, sin = O.rope_tables(16, 64)
    assert cos.shape == (16, 32) and cos[0].min() == 1.0 and np.abs(sin[0]).max() == 0.0
    # rotation by angle theta of the pair (x1_i, x2_i) = (x_i, x_{i+H/2}) preserves its norm
    r = O.rotate(x[:1], cos[5], sin[5])
    np.testing.assert_allclose(r[0, :32] ** 2 + r[0, 32:] ** 2, x[0, :32] ** 2 + x[0, 32:] ** 2, rtol=1e-5)
    z = (x[0, :32] + 1j * x[0, 32:]) * np.exp(1j * np.arange(5, 6) * (1.0 / 150000.0 ** (np.arange(0, 64, 2) / 64)))
    np.testing.assert_allclose(r[0, :32], z.real, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r[0, 32:], z.imag, rtol=1e-4, atol=1e-5)


def test_yarn_rope_tables_landmarks():
    """The YaRN branch of the rotary tables (lyra/model.py:164-174) at the gpt-oss setting (variants.py:62-80: base
    150000, scale 32, original length 4096, head dim 64, beta 32, alpha 1), pinned by what the published method fixes:
    the magnitude cos^2 + sin^2 = (0.1 ln(scale) + 1)^2 everywhere; frequencies that turn more than beta times within the
    original length are left alone, those that turn less than alpha times are interpolated (angle / scale), and the
    boundaries fall where i = (H/2) ln(L / (turns 2 pi)) / ln(base): 8.1 and 17.4 here (worked out by hand), so pairs
    0..8 are untouched, 18..31 fully interpolated, and the ones between blend linearly."""
    H, L, scale, base = 64, 4096, 32.0, 150000.0
    cos, sin = O.rope_tables(L, H, rope_base=base, rope_scale=scale, ntk_alpha=1.0, ntk_beta=32.0)
    assert cos.shape == (L * 32, 32)
    conc = 0.1 * np.log(32.0) + 1.0
    np.testing.assert_allclose(cos.astype(np.float64) ** 2 + sin.astype(np.float64) ** 2, conc * conc, rtol=2e-6)
    plain = 1.0 / base ** (np.arange(32) / 32.0)  # radians per position of pair i without scaling
    pos = 1000
    angle = np.arctan2(sin[pos].astype(np.float64), cos[pos].astype(np.float64))  # mod 2 pi
    wrap = lambda a: (a + np.pi) % (2 * np.pi) - np.pi
    np.testing.assert_allclose(wrap(angle[:9] - pos * plain[:9]), 0.0, atol=2e-4)             # untouched
    np.testing.assert_allclose(wrap(angle[18:] - pos * plain[18:] / scale), 0.0, atol=2e-6)   # interpolated
    # between the landmarks the rate lies strictly between the two, falling from one to the other
    rate = np.arctan2(sin[1].astype(np.float64), cos[1].astype(np.float64))  # radians per position (all < pi here)
    share = (rate[9:18] - plain[9:18] / scale) / (plain[9:18] - plain[9:18] / scale)  # 1 = untouched, 0 = interpolated
    assert np.all(share > 0) and np.all(share < 1) and np.all(np.diff(share) < 0)
    np.testing.assert_allclose(np.diff(share), np.diff(share)[0], rtol=1e-3)  # a linear ramp ...
    np.testing.assert_allclose(-1.0 / np.diff(share)[0], 17.39 - 8.09, rtol=2e-3)  # ... as long as the landmarks are apart
    # the host-side tables of the package are the same numbers
    from dataclasses import replace

    from lyra_amd.model import MODEL_VARIANTS, precompute_freq_cis
    cfg = replace(MODEL_VARIANTS["gpt-oss-20b"], seq_len=L)
    assert cfg.rope_scale == scale and cfg.rope_base == base and cfg.head_dim == H
    c2, s2 = precompute_freq_cis(cfg)
    assert np.array_equal(c2, cos) and np.array_equal(s2, sin)


def test_sample_topk_closed_forms():
    """lyra/generate.py:46-53 restated with a caller-supplied uniform number: k = 1 is the argmax whatever the number;
    u -> 0 picks the largest logit, u -> 1 the k-th largest; ties go to the lower index; and over a fine grid of uniform
    numbers the picks are distributed as the softmax of the k largest logits / temperature."""
    rng = np.random.default_rng(4)
    logits = rng.standard_normal((6, 50)).astype(np.float32)
    logits[2, 7] = logits[2, 30] = logits[2].max() + 1.0  # a tie for first place
    u = rng.random(6).astype(np.float32)
    assert (O.sample_topk(logits, u, 1, 0.7) == np.array([np.flatnonzero(r == r.max())[0] for r in logits])).all()
    order = np.argsort(-logits, axis=1, kind="stable")
    assert (O.sample_topk(logits, np.zeros(6, np.float32), 4, 0.8) == order[:, 0]).all()
    assert (O.sample_topk(logits, np.full(6, 0.999999, np.float32), 4, 0.8) == order[:, 3]).all()
    assert O.sample_topk(logits[2:3], np.zeros(1, np.float32), 4, 0.8)[0] == 7  # the lower index of the tied pair
    row = logits[:1]
    grid = ((np.arange(20000) + 0.5) / 20000).astype(np.float32)
    picks = O.sample_topk(np.repeat(row, grid.size, 0), grid, 4, 0.8)
    top = order[0, :4]
    want = torch.softmax(torch.from_numpy(row[0, top] / np.float32(0.8)), 0).numpy()
    got = np.array([(picks == t).mean() for t in top])
    assert set(picks.tolist()) <= set(top.tolist())
    np.testing.assert_allclose(got, want, atol=2e-4)
