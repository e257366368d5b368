"""GPU parity of the HIP decode-attention kernel (through the C ABI) against the CPU oracle.

Tolerance: |got - want| <= 2e-2 + 1e-2*|want| against the fp32 oracle (tests/gpu_util.py); float32
outputs are additionally held to 4e-3.  Index/mask behaviour is checked through outputs that differ
by O(1) if a single key is wrongly included or dropped.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _run(case, sm_scale, sw, pos, *, dtype=torch.bfloat16, gate=None, implementation="pallas", xsa_v=None, xsa_alpha=None,
         ranked=False):
    from lyra_amd.kernels.decode_attention import decode_attention, rank_rows

    q, k, v, sinks = U.attention_torch_inputs(case)
    p = pos if np.ndim(pos) == 0 else torch.from_numpy(np.asarray(pos, dtype=np.int32)).to(U.dev())
    g = None if gate is None else U.t_bf16(gate)
    xv = None if xsa_v is None else U.t_bf16(xsa_v)
    xa = None if xsa_alpha is None else U.t_f32(xsa_alpha)
    order = rank_rows(p) if ranked else None
    out = decode_attention(q, k, v, sinks, sm_scale, sw, p, dtype=dtype, implementation=implementation, gate=g, xsa_v=xv,
                           xsa_alpha=xa, row_order=order)
    torch.cuda.synchronize()
    return U.to_np(out)


def _note(*a):
    print(*a, file=sys.stderr, flush=True)


def test_selftest_layouts_and_conversions():
    from lyra_amd import _lib

    rep = torch.full((8,), -1, dtype=torch.int32, device=U.dev())
    _lib.check(_lib.lib.lyra_selftest(rep.data_ptr(), None), "lyra_selftest")
    torch.cuda.synchronize()
    r = rep.cpu().tolist()
    assert r[:7] == [0] * 7, f"mfma/cvt/cvt_bf16/pack/perm/denorm/rows mismatches: {r}"
    assert r[7] == _lib.ABI_VERSION


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("H,N,K", [(128, 16, 4), (64, 32, 4), (64, 64, 8), (128, 4, 4), (64, 16, 1)])
@pytest.mark.parametrize("sw", [0, 128])
def test_small_shapes_match_oracle(fp8, H, N, K, sw):
    S = 512
    case = U.attention_case(100 + H + N + K, 2, N, K, S, H, fp8=fp8)
    for pos in (511, 130, 5):
        _note(f"attn small fp8={fp8} H={H} N={N} K={K} sw={sw} pos={pos}")
        want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, sw, pos)
        got = _run(case, H**-0.5, sw, pos)
        U.assert_close(got, want, what=f"pos={pos}")
        got32 = _run(case, H**-0.5, sw, pos, dtype=torch.float32)
        U.assert_close(got32, want, atol=4e-3, rtol=4e-3, what=f"f32 pos={pos}")


def test_config1_lyra_small_bf16_global_with_gate():
    """Benchmark configuration 1 (single-sequence attention) at the variants.py shape (16Q/4KV/H=128) and at its literal 32Q/4KV/H=64."""
    for (N, K, H) in ((16, 4, 128), (32, 4, 64)):
        case = U.attention_case(1001, 1, N, K, 512, H, fp8=False)
        rng = np.random.default_rng(7)
        gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((1, N))))).astype(np.float32))
        _note(f"attn cfg1 N={N} K={K} H={H}")
        want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, 511, gate=gate)
        got = _run(case, H**-0.5, 0, 511, gate=gate)
        U.assert_close(got, want, what="cfg1")
        # the kernel rounds like the JAX code: bf16(bf16(attn) * gate)
        ref = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, 511, gate=gate, mode="ref")
        assert np.abs(got - ref).max() <= 2e-2


@pytest.mark.parametrize("S", [1, 3, 31, 33, 100, 257, 1000])
@pytest.mark.parametrize("fp8", [False, True])
def test_odd_cache_lengths_and_every_boundary(S, fp8):
    case = U.attention_case(200 + S, 1, 8, 2, S, 64, fp8=fp8)
    for sw in (0, 1, 7, 128):
        for pos in sorted({0, S // 2, S - 1, min(S - 1, 31), min(S - 1, 32)}):
            _note(f"attn odd S={S} fp8={fp8} sw={sw} pos={pos}")
            want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], 0.125, sw, pos)
            got = _run(case, 0.125, sw, pos)
            U.assert_close(got, want, what=f"S={S} sw={sw} pos={pos}")


def test_window_mask_is_exact_one_key_at_a_time():
    """A single huge-logit key just outside / inside the window flips the output by O(1)."""
    B, N, K, S, H = 1, 4, 1, 640, 64
    rng = np.random.default_rng(3)
    q = np.zeros((B, N, 1, H), np.float32)
    q[..., 0] = 8.0
    k = np.zeros((B, K, S, H), np.float32)
    v = O.bf16_round(rng.standard_normal((B, K, S, H)).astype(np.float32))
    sinks = np.full(N, -30.0, np.float32)
    for sw in (0, 128, 200):
        for pos in (127, 128, 300, 639):
            lo, hi = O.visible_range(pos, sw, S)
            for spike in {lo - 1, lo, hi, hi + 1}:
                if not 0 <= spike < S:
                    continue
                kk = k.copy()
                kk[0, 0, spike, 0] = 16.0  # logit 128*sm_scale: dominates iff visible
                case = {"q": q, "k": kk, "v": v, "sinks": sinks, "fp8": False}
                _note(f"attn mask sw={sw} pos={pos} spike={spike}")
                want = O.decode_attention_reference(q, kk, v, sinks, 1.0, sw, pos)
                got = _run(case, 1.0, sw, pos)
                U.assert_close(got, want, what=f"sw={sw} pos={pos} spike={spike}")
                if lo <= spike <= hi:
                    np.testing.assert_allclose(got[0, 0, 0], v[0, 0, spike], atol=2e-2)


def test_unwritten_cache_beyond_position_is_never_read_into_the_result():
    """Bytes past `position` may be anything (NaN codes, NaN/inf scales)."""
    B, N, K, S, H = 2, 8, 2, 256, 128
    case = U.attention_case(5, B, N, K, S, H, fp8=True)
    pos = np.array([70, 200])
    want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, pos)
    (kq, ks), (vq, vs) = case["k"], case["v"]
    kq, vq, ks, vs = kq.copy(), vq.copy(), ks.copy(), vs.copy()
    for b in range(B):
        kq[b, :, pos[b] + 1 :] = 0x7F
        vq[b, :, pos[b] + 1 :] = 0xFF
        ks[b, :, pos[b] + 1 :] = np.nan
        vs[b, :, pos[b] + 1 :] = np.inf
    dirty = dict(case, k=(kq, ks), v=(vq, vs))
    got = _run(dirty, H**-0.5, 0, pos)
    U.assert_close(got, want, what="dirty tail")
    # the same for a bf16 cache and a sliding window (keys before the window are garbage too)
    case = U.attention_case(6, B, N, K, S, H, fp8=False)
    want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 64, pos)
    kd, vd = case["k"].copy(), case["v"].copy()
    for b in range(B):
        kd[b, :, pos[b] + 1 :] = np.nan
        vd[b, :, pos[b] + 1 :] = np.nan
        kd[b, :, : pos[b] - 63] = np.nan
        vd[b, :, : pos[b] - 63] = np.inf
    got = _run(dict(case, k=kd, v=vd), H**-0.5, 64, pos)
    U.assert_close(got, want, what="dirty head and tail")


def test_sink_extremes_and_no_visible_key():
    B, N, K, S, H = 1, 8, 2, 256, 64
    case = U.attention_case(8, B, N, K, S, H, fp8=True)
    for sink in (-1e30, -float("inf"), 50.0, 1e4):
        c = dict(case, sinks=np.full(N, sink, np.float32))
        want = O.decode_attention_reference(c["q"], c["k"], c["v"], np.full(N, max(sink, -1e30), np.float32), 0.125, 0, 255)
        got = _run(c, 0.125, 0, 255)
        U.assert_close(got, want, what=f"sink={sink}")
    got = _run(case, 0.125, 0, -1)  # nothing cached yet: only the sink, whose value is 0
    assert np.abs(got).max() == 0.0


def test_row_without_visible_keys_in_a_chunked_launch_is_zero():
    """Few (row, kv head) pairs and a long cache: the launch is cut into chunks and merged.  A row whose position is -1 has
    no chunk with a key, so nobody reaches the merge: the output must still be written (zeros: the sink's value), and the
    arrival counters must be left so that the next call works."""
    from lyra_amd import _lib

    B, N, K, S, H = 2, 16, 4, 4096, 128
    assert _lib.lib.lyra_decode_attention_workspace(B, N, K, S, H, 0) > 256  # i.e. chunked
    case = U.attention_case(77, B, N, K, S, H, fp8=True)
    q, k, v, sinks = U.attention_torch_inputs(case)
    L = _lib.lib
    ws = torch.zeros(L.lyra_decode_attention_workspace(B, N, K, S, H, 0), dtype=torch.uint8, device=U.dev())
    for pos in ([-1, 3000], [2500, -1], [4095, 4095]):
        _note(f"attn chunked empty row pos={pos}")
        out = torch.full((B, N, 1, H), float("nan"), dtype=torch.bfloat16, device=U.dev())
        p = torch.tensor(pos, dtype=torch.int32, device=U.dev())
        rc = L.lyra_decode_attention(q.data_ptr(), k.qval.data_ptr(), v.qval.data_ptr(), k.scale.data_ptr(), v.scale.data_ptr(),
                                     sinks.data_ptr(), p.data_ptr(), 1, None, out.data_ptr(), ws.data_ptr(), ws.numel(),
                                     B, N, K, S, H, H**-0.5, 0, _lib.DTYPE_E4M3FN, _lib.DTYPE_BF16, torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "chunked empty row")
        torch.cuda.synchronize()
        got = U.to_np(out)
        want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, np.array(pos))
        for b in range(B):
            if pos[b] < 0:
                assert np.abs(got[b]).max() == 0.0
        U.assert_close(got, want, what=f"pos={pos}")
        assert int(ws[: 1 << 16].count_nonzero()) == 0


def test_split_count_does_not_change_the_result():
    """Partition invariance of the log-sum-exp merge: same keys, different chunking (B changes the plan)."""
    N, K, S, H = 8, 2, 4096, 128
    base = U.attention_case(9, 1, N, K, S, H, fp8=True)
    want = O.decode_attention_reference(base["q"], base["k"], base["v"], base["sinks"], H**-0.5, 0, 4000)
    got1 = _run(base, H**-0.5, 0, 4000)  # B*K = 2 pairs -> many chunks
    rep = 96  # B*K = 192 pairs -> fewer, longer chunks
    big = dict(base, q=np.repeat(base["q"], rep, 0), k=tuple(np.repeat(a, rep, 0) for a in base["k"]), v=tuple(np.repeat(a, rep, 0) for a in base["v"]))
    got2 = _run(big, H**-0.5, 0, 4000)
    U.assert_close(got1, want, what="many chunks")
    for b in (0, 17, rep - 1):
        U.assert_close(got2[b : b + 1], want, what="few chunks")
    assert np.abs(got2[:1] - got1).max() <= 1e-2


@pytest.mark.parametrize("B,N,K,S,H,sw,ragged", [
    (2, 16, 4, 512, 128, 0, False),     # one workgroup per (row, kv head)
    (2, 16, 4, 512, 128, 128, False),   # sliding window
    (3, 32, 8, 4096, 128, 0, True),     # chunked launch: the last workgroup to arrive merges, then the extra step
    (1, 16, 1, 8192, 128, 0, False),    # more chunks than the merge stages in LDS
    (70, 8, 4, 384, 128, 0, True),      # whole rows, longest first
    (40, 64, 8, 384, 64, 0, True),      # ... with 8 wavefronts and 64-wide heads
])
def test_learned_exclusive_self_attention_in_the_epilogue(B, N, K, S, H, sw, ragged):
    """lyra/model.py:351-363 fused behind the gate: t - tanh(alpha) <t, v^> v^ with v^ the new token's unit value row."""
    case = U.attention_case(6000 + B + N, B, N, K, S, H, fp8=True)
    rng = np.random.default_rng(B * 7 + N)
    pos = rng.integers(S // 2, S, B).astype(np.int32) if ragged else np.full(B, S - 1, np.int32)
    if ragged and B > 2:
        pos[1] = -1  # a row that sees only the sink: t = 0 stays 0
    gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((B, N))))).astype(np.float32))
    cur_v = O.bf16_round(rng.standard_normal((B, K, H)).astype(np.float32))
    alpha = rng.standard_normal(N).astype(np.float32)
    unit = O.unit_rows(cur_v, mode="ref")
    p = pos if ragged else int(pos[0])
    _note(f"attn xsa B={B} N={N} K={K} S={S} H={H} sw={sw} ragged={ragged}")
    if B * K * S > (1 << 16):
        (kq, ks), (vq, vs) = case["k"], case["v"]
        t = clib.decode_attention(O.bf16_bits(case["q"]), kq, vq, ks[..., 0], vs[..., 0], case["sinks"], pos, gate, H**-0.5, sw)
    else:
        t = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, sw, pos, gate=gate)
    want = O.xsa(t.reshape(B, N, H), cur_v, alpha).reshape(B, N, 1, H)
    got = _run(case, H**-0.5, sw, p, gate=gate, xsa_v=unit, xsa_alpha=alpha)
    U.assert_close(got, want, what="xsa bf16")
    if ragged and B > 2:
        assert np.all(got[1] == 0)
    got32 = _run(case, H**-0.5, sw, p, gate=gate, xsa_v=unit, xsa_alpha=alpha, dtype=torch.float32)
    U.assert_close(got32, want, atol=6e-3, rtol=6e-3, what="xsa f32")  # (v^ itself is a bf16 array)
    # The attention output over hundreds of random keys is small (~0.05 per element) and what the step removes smaller
    # still, so the bounds above barely see it: compare what the step changed, in float32, with what it should change.
    base32 = _run(case, H**-0.5, sw, p, gate=gate, dtype=torch.float32)
    removed_got, removed_want = base32 - got32, t.reshape(B, N, 1, H) - want
    scale = np.abs(removed_want).max()
    assert scale > 1e-3
    assert np.abs(removed_got - removed_want).max() <= 0.03 * scale, (np.abs(removed_got - removed_want).max(), scale)
    # t parallel to v^ and tanh(alpha) -> 1: the first head of every kv head loses everything
    G = N // K
    par = t.reshape(B, K, G, H)[:, :, 0, :]
    keep = np.abs(par).max(-1) > 0
    unit_par = O.unit_rows(O.bf16_round(par), mode="ref")
    gone = _run(case, H**-0.5, sw, p, gate=gate, xsa_v=unit_par, xsa_alpha=np.full(N, 20.0, np.float32), dtype=torch.float32)
    first = gone.reshape(B, K, G, H)[:, :, 0, :]
    assert np.abs(first[keep]).max() <= 0.02 * np.abs(par[keep]).max()
    # alpha = 0 switches the step off exactly: same bits as the launch without it
    base = _run(case, H**-0.5, sw, p, gate=gate)
    off = _run(case, H**-0.5, sw, p, gate=gate, xsa_v=unit, xsa_alpha=np.zeros(N, np.float32))
    np.testing.assert_array_equal(off, base)
    # the plain-framework path computes the same function
    plain = _run(case, H**-0.5, sw, p, gate=gate, xsa_v=unit, xsa_alpha=alpha, implementation="xla")
    U.assert_close(plain, want, what="xsa plain path")


def test_config4_gpt_oss_shape_ragged_fp8_full_size():
    """Benchmark configuration 4 (gpt-oss attention shape, ragged batch): B=64, 64Q/8KV, H=64, S=4096, L_b ~ U{256..4096}, FP8 cache; global and window 128."""
    B, N, K, S, H = 64, 64, 8, 4096, 64
    case = U.attention_case(1004, B, N, K, S, H, fp8=True)
    rng = np.random.default_rng(1004)
    pos = (rng.integers(256, 4097, B) - 1).astype(np.int32)
    (kq, ks), (vq, vs) = case["k"], case["v"]
    for sw in (0, 128):
        _note(f"attn cfg4 sw={sw}")
        want = clib.decode_attention(O.bf16_bits(case["q"]), kq, vq, ks[..., 0], vs[..., 0], case["sinks"], pos, None, H**-0.5, sw)
        got = _run(case, H**-0.5, sw, pos)
        U.assert_close(got, want, what=f"cfg4 sw={sw}")
    # size-independent property: doubling every V scale doubles the output bit for bit (power-of-two scaling
    # commutes with every rounding in the kernel)
    got2 = _run(dict(case, v=(vq, vs * 2.0)), H**-0.5, 0, pos)
    got1 = _run(case, H**-0.5, 0, pos)
    np.testing.assert_array_equal(got2, got1 * 2.0)


@pytest.mark.parametrize("fp8,H,N,K,B", [(True, 64, 16, 8, 37), (False, 128, 8, 4, 70), (True, 128, 4, 2, 200), (True, 64, 2, 1, 256)])
def test_ragged_rows_longest_first_launch(fp8, H, N, K, B):
    """More (batch row, kv head) pairs than compute units with one position per row: the kernel hands rows out longest
    first.  Equal lengths (rank ties), a row that sees only the sink (position -1), full rows, and the output gate."""
    S = 384
    case = U.attention_case(4000 + B, B, N, K, S, H, fp8=fp8)
    rng = np.random.default_rng(B)
    pos = rng.integers(0, S, B).astype(np.int32)
    pos[: B // 4] = pos[B // 2 : B // 2 + B // 4]  # many ties
    pos[1], pos[B - 1], pos[B // 3] = -1, S - 1, S - 1
    gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((B, N))))).astype(np.float32))
    _note(f"attn sorted fp8={fp8} H={H} N={N} K={K} B={B}")
    want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, pos)
    got = _run(case, H**-0.5, 0, pos)
    U.assert_close(got, want, what="ragged")
    assert np.all(got[1] == 0)
    got_g = _run(case, H**-0.5, 0, pos, gate=gate)
    want_g = want * gate[:, :, None, None]
    U.assert_close(got_g, want_g, what="ragged + gate")


def test_rank_rows_is_the_stable_descending_order():
    from lyra_amd.kernels.decode_attention import rank_rows

    rng = np.random.default_rng(9)
    for B in (1, 2, 63, 64, 65, 300, 1025, 4000):
        pos = rng.integers(-1, 50, B).astype(np.int32)  # many ties
        got = rank_rows(torch.from_numpy(pos).to(U.dev())).cpu().numpy()
        want = np.argsort(-pos.astype(np.int64), kind="stable").astype(np.int32)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("fp8,H,N,K,B", [(True, 64, 16, 8, 37), (False, 128, 8, 4, 70), (True, 128, 4, 2, 200), (True, 64, 2, 1, 300),
                                         (True, 64, 64, 8, 64), (True, 128, 32, 8, 64)])
def test_ragged_rows_dealt_out_by_a_given_order(fp8, H, N, K, B):
    """lyra_decode_attention_ranked: the same cases as the launch that ranks the rows itself, with the order computed
    beforehand; any permutation must give the same output bit for bit (it only changes which workgroup takes which row),
    and a launch the order does not apply to (a window, few pairs) ignores it."""
    from lyra_amd.kernels.decode_attention import decode_attention

    S = 384
    case = U.attention_case(4100 + B, B, N, K, S, H, fp8=fp8)
    rng = np.random.default_rng(B + 1)
    pos = rng.integers(0, S, B).astype(np.int32)
    pos[: B // 4] = pos[B // 2 : B // 2 + B // 4]
    pos[1], pos[B - 1], pos[B // 3] = -1, S - 1, S - 1
    gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((B, N))))).astype(np.float32))
    _note(f"attn ranked fp8={fp8} H={H} N={N} K={K} B={B}")
    want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, pos)
    got = _run(case, H**-0.5, 0, pos, ranked=True)
    U.assert_close(got, want, what="ranked")
    assert np.all(got[1] == 0)
    U.assert_close(_run(case, H**-0.5, 0, pos, gate=gate, ranked=True), want * gate[:, :, None, None], what="ranked + gate")
    got32 = _run(case, H**-0.5, 0, pos, dtype=torch.float32, ranked=True)
    U.assert_close(got32, want, atol=4e-3, rtol=4e-3, what="ranked f32")
    # any other permutation: identical bits
    q, k, v, sinks = U.attention_torch_inputs(case)
    p = torch.from_numpy(pos).to(U.dev())
    perm = torch.from_numpy(rng.permutation(B).astype(np.int32)).to(U.dev())
    other = decode_attention(q, k, v, sinks, H**-0.5, 0, p, implementation="pallas", row_order=perm)
    np.testing.assert_array_equal(U.to_np(other), got)
    # a window: the order is ignored, the result is the plain launch's
    np.testing.assert_array_equal(_run(case, H**-0.5, 128, pos, ranked=True), _run(case, H**-0.5, 128, pos))


def test_ragged_launch_replays_in_a_hip_graph():
    """The whole-row launch captured in a HIP graph: replays follow the positions the caller updates in place between
    them, and every replay equals the eager result for the same positions."""
    from lyra_amd.kernels.decode_attention import decode_attention

    B, N, K, S, H = 70, 8, 4, 384, 128
    case = U.attention_case(4242, B, N, K, S, H, fp8=True)
    q, k, v, sinks = U.attention_torch_inputs(case)
    rng = np.random.default_rng(7)
    pos = torch.from_numpy(rng.integers(0, S, B).astype(np.int32)).to(U.dev())
    out_static = torch.empty_like(q)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out_static.copy_(decode_attention(q, k, v, sinks, H**-0.5, 0, pos, implementation="pallas"))  # warm-up outside the graph
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static.copy_(decode_attention(q, k, v, sinks, H**-0.5, 0, pos, implementation="pallas"))
    for rep in range(3):
        new_pos = rng.integers(-1, S, B).astype(np.int32)
        pos.copy_(torch.from_numpy(new_pos).to(U.dev()))
        _note(f"attn ragged graph replay {rep}")
        graph.replay()
        torch.cuda.synchronize()
        got = U.to_np(out_static)
        eager = U.to_np(decode_attention(q, k, v, sinks, H**-0.5, 0, pos, implementation="pallas"))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(got, eager)
        want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, new_pos)
        U.assert_close(got, want, what=f"replay {rep}")


def test_headline_shape_b64_ctx4096_fp8():
    """B=64, ctx 4096, FP8 cache at the lyra-small shape (16Q/4KV/H=128), all rows full."""
    B, N, K, S, H = 64, 16, 4, 4096, 128
    case = U.attention_case(1000, B, N, K, S, H, fp8=True)
    (kq, ks), (vq, vs) = case["k"], case["v"]
    pos = np.full(B, S - 1, np.int32)
    want = clib.decode_attention(O.bf16_bits(case["q"]), kq, vq, ks[..., 0], vs[..., 0], case["sinks"], pos, None, H**-0.5, 0)
    got = _run(case, H**-0.5, 0, S - 1)
    U.assert_close(got, want, what="headline")
    # permuting the cached keys (with their values and scales) cannot change attention
    perm = np.random.default_rng(1).permutation(S)
    shuf = dict(case, k=(kq[:, :, perm], ks[:, :, perm]), v=(vq[:, :, perm], vs[:, :, perm]))
    got_p = _run(shuf, H**-0.5, 0, S - 1)
    assert np.abs(got_p - got).max() <= 1e-2


# ---- full-size rows held to the float32 bound ------------------------------------------------------------------------
# With N(0,1) keys and values an output element over 4096 keys is ~0.026 in size, which the bf16 acceptance bound
# (2e-2 + 1e-2 |want|) does not resolve: a dropped 32-key tile moves an element by a few 1e-3.  These tests therefore take
# the float32 output of the same launches and hold it to what the kernel's one rounding allows: the probabilities enter
# the second matrix product as bf16 (p_j * v_scale_j, relative error <= 2^-9 each), so an output element may be off by
# 2^-9 * A with A = sum_j p_j |v_j| (the oracle run on the absolute values of the cache gives A); the bound is
# 1e-3 + 2^-8 * A - about 4e-3 for drawn queries.  Once with the drawn queries and once with queries four times as large
# (logits with sigma 4: a handful of keys carry most of the weight, so every single key matters), and a control on the
# host shows that an expected output with one tile left out breaks that bound.
def _f32_bound(case, pos, sw, H):
    (kq, ks), (vq, vs) = case["k"], case["v"]
    a = clib.decode_attention(O.bf16_bits(case["q"]), kq, vq & np.uint8(0x7F), ks[..., 0], vs[..., 0], case["sinks"], pos, None, H**-0.5, sw)
    return 1e-3 + 2.0**-8 * a


def _assert_within(got, want, bound, what):
    got = np.asarray(got, np.float32).reshape(want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    worst = int(np.argmax(err - bound))
    assert (err <= bound).all(), f"{what}: err {err.flat[worst]:.4g} > bound {bound.flat[worst]:.4g} at {worst}: got {got.flat[worst]:.6g} want {want.flat[worst]:.6g}"


def _peaked(case):
    return dict(case, q=O.bf16_round(case["q"] * np.float32(4.0)))


def _oracle_fp8(case, pos, sw, H):
    (kq, ks), (vq, vs) = case["k"], case["v"]
    return clib.decode_attention(O.bf16_bits(case["q"]), kq, vq, ks[..., 0], vs[..., 0], case["sinks"], pos, None, H**-0.5, sw)


def _skipped_tile_breaks_the_bound(case, pos_b, b, H, want_b, bound_b):
    """Negative control, on the host only: the oracle's output for batch row b with one 32-key tile of the visible range
    removed from the cache must violate the float32 bound against the full output."""
    (kq, ks), (vq, vs) = case["k"], case["v"]
    tile = (int(pos_b) // 2) // 32 * 32
    keep = np.r_[0:tile, tile + 32 : kq.shape[2]]
    sub = lambda a: np.ascontiguousarray(a[b : b + 1][:, :, keep])
    short = clib.decode_attention(O.bf16_bits(case["q"][b : b + 1]), sub(kq), sub(vq), sub(ks)[..., 0], sub(vs)[..., 0],
                                  case["sinks"], np.array([pos_b - 32], np.int32), None, H**-0.5, 0)
    err = np.abs(short - want_b)
    assert (err > bound_b).any(), "a skipped tile would pass the float32 bound"
    return float(err.max())


@pytest.mark.parametrize("name,B,N,K,H,ragged", [
    ("headline", 64, 16, 4, 128, False),    # one workgroup per (row, kv head): the launch bench.py times
    ("config 4", 64, 64, 8, 64, True),      # gpt-oss shape, L_b ~ U{256..4096}: the whole-row launch
    ("config 5", 128, 32, 8, 128, False),   # lyra-max layer
])
def test_full_size_rows_float32_bound(name, B, N, K, H, ragged):
    S = 4096
    case = U.attention_case(1100 + B + N, B, N, K, S, H, fp8=True)
    rng = np.random.default_rng(B + N)
    pos = (rng.integers(256, S + 1, B) - 1).astype(np.int32) if ragged else np.full(B, S - 1, np.int32)
    launch_pos = pos if ragged else S - 1
    for label, c in (("drawn", case), ("peaked", _peaked(case))):
        for sw in (0, 128):
            _note(f"attn f32 bound {name} {label} sw={sw}")
            want, bound = _oracle_fp8(c, pos, sw, H), _f32_bound(c, pos, sw, H)
            got = _run(c, H**-0.5, sw, launch_pos, dtype=torch.float32)
            _assert_within(got, want, bound, f"{name} {label} sw={sw} f32")
            if sw == 0:
                b = int(np.argmax(pos))
                moved = _skipped_tile_breaks_the_bound(c, pos[b], b, H, want[b : b + 1], bound[b : b + 1])
                _note(f"   (a skipped tile moves an element by up to {moved:.4f}; bound there {bound[b].max():.4f})")
                if not ragged:  # the same rows through the launch that takes one position per row
                    _assert_within(_run(c, H**-0.5, 0, pos, dtype=torch.float32), want, bound, f"{name} {label} one position per row f32")


@pytest.mark.parametrize("sw", [0, 128])
def test_front_step_launch_at_b64_ctx4096_float32_bound(sw):
    """The launch the decode step runs (QK norm, rotary embedding and cache append inside the attention launch) at the
    headline shape, float32 output against the C oracle fed the q rows and caches the two-launch path leaves."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray, quantize

    B, N, K, S, H = 64, 16, 4, 4096, 128
    dev = U.dev()
    gen = torch.Generator(device=dev)
    gen.manual_seed(77 + sw)
    rng = np.random.default_rng(77)
    width = (N + 2 * K) * H
    for label, amp in (("drawn", 0.58), ("peaked", 2.3)):  # 3 slices of sigma amp: q rows of sigma 1 and 4
        _note(f"attn qkv f32 bound sw={sw} {label}")
        part = torch.randn(3, B, width, device=dev, generator=gen) * amp
        part[:, :, N * H :] *= 0.58 / amp  # (keys and values stay at sigma 1)
        hist_k = torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16)
        hist_v = torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16)
        qk, qv = quantize(hist_k, torch.float8_e4m3fn, (1, H)), quantize(hist_v, torch.float8_e4m3fn, (1, H))
        mk = lambda a: QArray(a.qval.clone(), a.scale.clone(), (1, H))
        ka, va, kb_, vb = mk(qk), mk(qv), mk(qk), mk(qv)
        cos_t, sin_t = O.rope_tables(S, H)
        cos_t, sin_t = U.t_f32(cos_t), U.t_f32(sin_t)
        sinks = rng.standard_normal(N).astype(np.float32)
        pos = torch.tensor(S - 1, dtype=torch.int32, device=dev)
        got = F.attention_qkv(F.Unsummed(part, None, 1.0), None, None, cos_t, sin_t, pos, ka, va, U.t_f32(sinks), H**-0.5, sw,
                              N, K, H, 1e-5, out_dtype=torch.float32)
        assert got is not None
        q = F.qkv_post(F.Unsummed(part.clone(), None, 1.0), None, None, cos_t, sin_t, pos, kb_, vb, N, K, H, 1e-5)
        torch.cuda.synchronize()
        assert torch.equal(ka.qval.view(torch.uint8), kb_.qval.view(torch.uint8)) and torch.equal(va.scale, vb.scale)
        u8 = lambda t: t.view(torch.uint8).cpu().numpy()
        want = clib.decode_attention(O.bf16_bits(U.to_np(q)[:, :, None, :]), u8(kb_.qval), u8(vb.qval), U.to_np(kb_.scale)[..., 0],
                                     U.to_np(vb.scale)[..., 0], sinks, np.full(B, S - 1, np.int32), None, H**-0.5, sw)
        a = clib.decode_attention(O.bf16_bits(U.to_np(q)[:, :, None, :]), u8(kb_.qval), u8(vb.qval) & np.uint8(0x7F), U.to_np(kb_.scale)[..., 0],
                                  U.to_np(vb.scale)[..., 0], sinks, np.full(B, S - 1, np.int32), None, H**-0.5, sw)
        _assert_within(U.to_np(got), want, 1e-3 + 2.0**-8 * a, f"front step {label} sw={sw}")


def test_config5_lyra_max_shape_b128_ctx4096_fp8():
    """Benchmark configuration 5, the attention of one lyra-max layer: B=128, 32Q/8KV, H=128, ctx 4096, FP8 cache, global
    and window 128; then the same batch with one position per row (the whole-row launch) against the shared position."""
    B, N, K, S, H = 128, 32, 8, 4096, 128
    case = U.attention_case(1005, B, N, K, S, H, fp8=True)
    (kq, ks), (vq, vs) = case["k"], case["v"]
    pos = np.full(B, S - 1, np.int32)
    got0 = None
    for sw in (0, 128):
        _note(f"attn cfg5 sw={sw}")
        want = clib.decode_attention(O.bf16_bits(case["q"]), kq, vq, ks[..., 0], vs[..., 0], case["sinks"], pos, None, H**-0.5, sw)
        got = _run(case, H**-0.5, sw, S - 1)
        U.assert_close(got, want, what=f"cfg5 sw={sw}")
        if sw == 0:
            got0 = got
    got_rows = _run(case, H**-0.5, 0, pos)
    assert np.abs(got_rows - got0).max() <= 1e-2


def test_xla_path_and_dispatch_contract():
    from lyra_amd.kernels.decode_attention import decode_attention

    case = U.attention_case(11, 2, 8, 2, 384, 64, fp8=True)
    q, k, v, sinks = U.attention_torch_inputs(case)
    want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], 0.125, 128, 300)
    for impl in ("auto", "pallas", "hip", "xla"):
        out = decode_attention(q, k, v, sinks, 0.125, 128, torch.tensor(300, dtype=torch.int32, device=U.dev()), implementation=impl)
        assert out.shape == q.shape and out.dtype == q.dtype
        U.assert_close(U.to_np(out), want, what=impl)
    # unsupported head_dim: "pallas" raises like common.py:147-151, "auto" falls back to the plain path
    c2 = U.attention_case(12, 1, 4, 2, 64, 32, fp8=False)
    q2, k2, v2, s2 = U.attention_torch_inputs(c2)
    with pytest.raises(ValueError, match="no HIP kernel configuration"):
        decode_attention(q2, k2, v2, s2, 0.2, 0, 63, implementation="pallas")
    out = decode_attention(q2, k2, v2, s2, 0.2, 0, 63, implementation="auto")
    U.assert_close(U.to_np(out), O.decode_attention_reference(c2["q"], c2["k"], c2["v"], c2["sinks"], 0.2, 0, 63), what="fallback")
    # a QArray handed to a dense config (and vice versa) is an error: decode_attention.py:199-200,215-216
    from lyra_amd.kernels.decode_attention import DecodeAttentionConfig, _decode_attention

    with pytest.raises(ValueError, match="requires QArray"):
        _decode_attention(q, k.qval.to(torch.bfloat16), v.qval.to(torch.bfloat16), sinks, 0.125, 0, 3, DecodeAttentionConfig(cache_dtype=torch.float8_e4m3fn), torch.bfloat16)
    with pytest.raises(ValueError, match="received QArray"):
        _decode_attention(q, k, v, sinks, 0.125, 0, 3, DecodeAttentionConfig(), torch.bfloat16)
