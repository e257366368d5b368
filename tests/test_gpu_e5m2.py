"""GPU parity of the decode kernels on the second 1-byte format of the reference's ``FP8_DTYPES`` (lyra/nn/quant.py:10):
float8_e5m2 KV caches and weights.  The reference's operators are generic over the two formats (``is_scaled``,
decode_attention.py:52, decode_gemm.py:83); its serve path only sets e4m3fn (generate.py:36).  The matmul cases live in
tests/test_gpu_gemm.py (kind "e5m2"); here: attention, the cache append and the conversions' self-check.

Tolerances as for e4m3fn: |got - want| <= 2e-2 + 1e-2*|want| against the fp32 oracle on the same codes (bf16 output),
4e-3 for float32 output; appended codes and scales bit for bit.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O
from tests import gpu_util as U

pytestmark = pytest.mark.gpu
E5M2 = 2  # the oracle's format number


def _note(*a):
    print(*a, file=sys.stderr, flush=True)


def _run(case, sm_scale, sw, pos, *, dtype=torch.bfloat16, gate=None, ranked=False):
    from lyra_amd.kernels.decode_attention import decode_attention, rank_rows

    q, k, v, sinks = U.attention_torch_inputs(case)
    assert k.qval.dtype == torch.float8_e5m2
    p = pos if np.ndim(pos) == 0 else torch.from_numpy(np.asarray(pos, dtype=np.int32)).to(U.dev())
    g = None if gate is None else U.t_bf16(gate)
    out = decode_attention(q, k, v, sinks, sm_scale, sw, p, dtype=dtype, implementation="pallas", gate=g,
                           row_order=rank_rows(p) if ranked else None)
    torch.cuda.synchronize()
    return U.to_np(out)


def _want(case, sm_scale, sw, pos):
    return O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], sm_scale, sw, pos, fp8_format=E5M2)


@pytest.mark.parametrize("H,N,K", [(128, 16, 4), (64, 32, 4), (64, 64, 8), (128, 4, 4)])
@pytest.mark.parametrize("sw", [0, 128])
def test_attention_small_shapes_match_oracle(H, N, K, sw):
    S = 512
    case = U.attention_case(300 + H + N + K, 2, N, K, S, H, fp8=True, fmt=E5M2)
    for pos in (511, 130, 5):
        _note(f"e5m2 attn small H={H} N={N} K={K} sw={sw} pos={pos}")
        want = _want(case, H**-0.5, sw, pos)
        U.assert_close(_run(case, H**-0.5, sw, pos), want, what=f"pos={pos}")
        U.assert_close(_run(case, H**-0.5, sw, pos, dtype=torch.float32), want, atol=4e-3, rtol=4e-3, what=f"f32 pos={pos}")


def test_attention_is_not_the_e4m3fn_reading_of_the_same_bytes():
    """Negative control of the format plumbing: the same bytes read as e4m3fn give a different answer by far."""
    H, N, K, S = 64, 8, 2, 256
    case = U.attention_case(77, 2, N, K, S, H, fp8=True, fmt=E5M2)
    want = _want(case, H**-0.5, 0, S - 1)
    got = _run(case, H**-0.5, 0, S - 1)
    U.assert_close(got, want, what="e5m2")
    wrong = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, 0, S - 1, fp8_format=1)
    assert np.abs(got - wrong).max() > 0.05


@pytest.mark.parametrize("S", [1, 3, 33, 257, 1000])
def test_attention_odd_cache_lengths(S):
    """Lengths that are not multiples of 4: per-token scales are fetched one by one."""
    case = U.attention_case(500 + S, 1, 8, 2, S, 64, fp8=True, fmt=E5M2)
    for sw in (0, 7, 128):
        for pos in sorted({0, S // 2, S - 1, min(S - 1, 32)}):
            _note(f"e5m2 attn odd S={S} sw={sw} pos={pos}")
            U.assert_close(_run(case, 0.125, sw, pos), _want(case, 0.125, sw, pos), what=f"S={S} sw={sw} pos={pos}")


@pytest.mark.parametrize("H,N,K,B", [(64, 16, 8, 37), (128, 4, 2, 200)])
def test_attention_ragged_rows_whole_row_launch_and_given_order(H, N, K, B):
    S = 384
    case = U.attention_case(4200 + B, B, N, K, S, H, fp8=True, fmt=E5M2)
    rng = np.random.default_rng(B)
    pos = rng.integers(0, S, B).astype(np.int32)
    pos[1], pos[B - 1] = -1, S - 1
    gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((B, N))))).astype(np.float32))
    _note(f"e5m2 attn ragged H={H} N={N} K={K} B={B}")
    want = _want(case, H**-0.5, 0, pos)
    got = _run(case, H**-0.5, 0, pos)
    U.assert_close(got, want, what="ragged")
    assert np.all(got[1] == 0)
    U.assert_close(_run(case, H**-0.5, 0, pos, gate=gate), want * gate[:, :, None, None], what="ragged + gate")
    ranked = _run(case, H**-0.5, 0, pos, ranked=True)
    U.assert_close(ranked, want, what="ranked")
    U.assert_close(_run(case, H**-0.5, 0, pos, dtype=torch.float32, ranked=True), want, atol=4e-3, rtol=4e-3, what="ranked f32")


def test_attention_full_context_b16_ctx4096():
    """The headline layer shape (16 query / 4 kv heads of 128, 4096 keys) at a batch the C oracle finishes in seconds."""
    B, N, K, S, H = 16, 16, 4, 4096, 128
    case = U.attention_case(9100, B, N, K, S, H, fp8=True, fmt=E5M2)
    (kq, ks), (vq, vs) = case["k"], case["v"]
    _note("e5m2 attn full context")
    for sw in (0, 128):
        want = clib.decode_attention(O.bf16_bits(case["q"]), kq, vq, ks[..., 0], vs[..., 0], case["sinks"], S - 1, None, H**-0.5, sw,
                                     fp8_format=E5M2)
        U.assert_close(_run(case, H**-0.5, sw, S - 1), want, what=f"full sw={sw}")
        U.assert_close(_run(case, H**-0.5, sw, S - 1, dtype=torch.float32), want, atol=4e-3, rtol=4e-3, what=f"full f32 sw={sw}")


@pytest.mark.parametrize("B,N,K,S,H,per_row", [(64, 16, 4, 512, 128, False), (3, 2, 1, 256, 64, True)])
def test_cache_append_quantises_to_e5m2(B, N, K, S, H, per_row):
    """lyra_qkv_post on an e5m2 cache: the value row is appended untouched, so its codes and scale are those of the
    reference quantiser (scale = amax / 57344, lyra/nn/quant.py:68-72) bit for bit; at position 0 without QK norm so is
    the key row.  Nothing but the appended row is written."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray

    _note(f"e5m2 append B{B} N{N} K{K} S{S} H{H} per_row={per_row}")
    dev = U.dev()
    rng = np.random.default_rng(B + S)
    qkv = O.bf16_round(rng.standard_normal((B, (N + 2 * K) * H), dtype=np.float32) * np.exp(rng.standard_normal((B, 1)) * 2).astype(np.float32))
    qkv[0, (N + K) * H : (N + K) * H + H] = 0  # an all-zero value row: scale 1, codes 0
    cos_t, sin_t = O.rope_tables(S, H)
    sentinel = 0x55
    mk = lambda: QArray(torch.full((B, K, S, H), sentinel, dtype=torch.uint8, device=dev).view(torch.float8_e5m2),
                        torch.full((B, K, S, 1), 7.0, dtype=torch.float32, device=dev), (1, H))
    for pos in ((rng.integers(0, S, B).astype(np.int32) if per_row else np.full(B, S - 1, np.int32)), np.zeros(B, np.int32)):
        ck, cv = mk(), mk()
        pos_t = torch.from_numpy(pos).to(dev) if per_row else torch.tensor(int(pos[0]), dtype=torch.int32, device=dev)
        F.qkv_post(U.t_bf16(qkv), None, None, U.t_f32(cos_t), U.t_f32(sin_t), pos_t, ck, cv, N, K, H, 1e-5)
        torch.cuda.synchronize()
        rows = np.arange(B)
        kw = qkv[:, N * H : (N + K) * H].reshape(B, K, H)
        vw = qkv[:, (N + K) * H :].reshape(B, K, H)
        for name, cache, want in (("k", ck, kw), ("v", cv, vw)):
            codes = cache.qval.view(torch.uint8).cpu().numpy()
            scales = cache.scale.cpu().numpy()[..., 0]
            if name == "v" or not pos.any():
                wq, ws = O.quantize(want[:, :, None, :], (1, H), fmt=E5M2)
                assert np.array_equal(codes[rows, :, pos], wq[:, :, 0]), name
                assert np.array_equal(scales[rows, :, pos], ws[:, :, 0, 0]), name
            codes[rows, :, pos] = sentinel
            scales[rows, :, pos] = 7.0
            assert (codes == sentinel).all() and (scales == 7.0).all()


@pytest.mark.parametrize("B,N,K,S,H,qknorm,sw,unsummed,full", [
    (64, 16, 4, 4096, 128, True, 0, True, True),     # the headline layer
    (64, 16, 4, 4096, 128, True, 128, True, True),
    (5, 8, 2, 515, 64, False, 0, False, False),
    (10, 6, 2, 1000, 128, True, 0, True, False),
])
def test_attention_with_the_front_step_equals_the_two_launches(B, N, K, S, H, qknorm, sw, unsummed, full):
    """lyra_decode_attention_qkv on e5m2 caches against lyra_qkv_post(_sum) + lyra_decode_attention: outputs and every byte
    of the caches identical."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.kernels.decode_attention import decode_attention
    from lyra_amd.nn.quant import QArray, quantize

    _note(f"e5m2 attention_qkv B{B} N{N} K{K} S{S} H{H} qknorm={qknorm} sw={sw} unsummed={unsummed}")
    dev = U.dev()
    rng = np.random.default_rng(B * 3 + N + S)
    gen = torch.Generator(device=dev)
    gen.manual_seed(S + B)
    width = (N + 2 * K) * H
    if unsummed:
        part = torch.randn(3, B, width, device=dev, generator=gen) * (1.4 / 3**0.5)
        qkv_a, qkv_b = F.Unsummed(part, None, 1.0), F.Unsummed(part.clone(), None, 1.0)
    else:
        t = (torch.randn(B, width, device=dev, generator=gen) * 2).to(torch.bfloat16)
        qkv_a, qkv_b = t, t.clone()
    qn = U.t_f32((1 + 0.1 * rng.standard_normal(H)).astype(np.float32)) if qknorm else None
    kn = U.t_f32((1 + 0.1 * rng.standard_normal(H)).astype(np.float32)) if qknorm else None
    cos_t, sin_t = O.rope_tables(S, H)
    cos_t, sin_t = U.t_f32(cos_t), U.t_f32(sin_t)
    if full:
        pos = torch.tensor(S - 1, dtype=torch.int32, device=dev)
    else:
        vals = rng.integers(0, S, B)
        vals[0] = S - 1
        pos = torch.from_numpy(np.asarray(vals, dtype=np.int32)).to(dev)
    hist = torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16)
    hist2 = torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16)

    def caches():
        qk, qv = quantize(hist, torch.float8_e5m2, (1, H)), quantize(hist2, torch.float8_e5m2, (1, H))
        return QArray(qk.qval.clone(), qk.scale.clone(), (1, H)), QArray(qv.qval.clone(), qv.scale.clone(), (1, H))

    sinks = U.t_f32(rng.standard_normal(N).astype(np.float32))
    ka, va = caches()
    kb_, vb = caches()
    got = F.attention_qkv(qkv_a, qn, kn, cos_t, sin_t, pos, ka, va, sinks, H**-0.5, sw, N, K, H, 1e-5)
    assert got is not None
    q = F.qkv_post(qkv_b, qn, kn, cos_t, sin_t, pos, kb_, vb, N, K, H, 1e-5)
    want = decode_attention(q[:, :, None, :], kb_, vb, sinks, H**-0.5, sw, pos, implementation="pallas").reshape(B, N * H)
    torch.cuda.synchronize()
    for name, a, b in (("k", ka, kb_), ("v", va, vb)):
        assert torch.equal(a.qval.view(torch.uint8), b.qval.view(torch.uint8)), f"{name} codes differ"
        assert torch.equal(a.scale, b.scale), f"{name} scales differ"
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # and the two-launch result itself against the oracle on the GPU's own cache bytes
    pos_np = pos.cpu().numpy() if pos.ndim else int(pos)
    kq, ks = kb_.qval.view(torch.uint8).cpu().numpy(), kb_.scale.cpu().numpy()
    vq, vs = vb.qval.view(torch.uint8).cpu().numpy(), vb.scale.cpu().numpy()
    ref = clib.decode_attention(O.bf16_bits(U.to_np(q)[:, :, None, :]), kq, vq, ks[..., 0], vs[..., 0], U.to_np(sinks), pos_np, None,
                                H**-0.5, sw, fp8_format=E5M2)
    U.assert_close(U.to_np(want).reshape(B, N, 1, H), ref, what="two launches vs oracle")
