"""GPU parity of the HIP decode GEMM (through the C ABI) against the CPU oracle.

Tolerance: |got - want| <= 2e-2 + 1e-2*|want| against the fp32 oracle on the same dequantised
weights; float32 outputs are held to 2e-3 + 2e-3*|want|.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _note(*a):
    print(*a, file=sys.stderr, flush=True)


def _weights(rng, G, K, N, w_std):
    """N(0, w_std) weights.  Big shapes draw one expert-sized pool and give expert g a shifted window of it
    (i.i.d. within an expert, which is all a parity test needs) to keep generation in seconds."""
    if G * K * N <= (1 << 24):
        return (rng.standard_normal((G, K, N), dtype=np.float32) * np.float32(w_std)).astype(np.float32)
    pool = rng.standard_normal(K * N + 1009 * G, dtype=np.float32) * np.float32(w_std)
    return np.stack([pool[1009 * g : 1009 * g + K * N].reshape(K, N) for g in range(G)])


def _case(seed, M, G, K, N, sizes, *, kind, block=(256, 256), bias=False, w_std=0.02):
    rng = np.random.default_rng(seed)
    lhs = O.bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    w = _weights(rng, G, K, N, w_std)
    c = {"lhs": lhs, "sizes": np.asarray(sizes, np.int32), "kind": kind, "block": block}
    c["bias"] = rng.standard_normal((G, N)).astype(np.float32) if bias else None
    c["fmt"] = 2 if kind == "e5m2" else 1  # the 1-byte format of the codes: e4m3fn unless the case says e5m2
    if kind in ("fp8", "e5m2"):
        c["w"] = clib.quantize_blocks(w, block, fp8_format=c["fmt"])  # bit-identical to O.quantize (tests/test_oracle_formats.py)
        c["kind"] = "fp8"
    else:
        c["w"] = O.bf16_round(w)
    return c


def _want(c, swiglu, big=False):
    # Several groups with scale blocks shorter than K: the kernel dequantises like the reference, f32(code) * scale rounded
    # to bf16 (lyra/nn/quant.py:82-85), so that is the operand the float32 product is taken on.  Everywhere else the
    # scales factor out of the product and are applied to the float32 sums.
    like_reference = c["kind"] == "fp8" and len(c["sizes"]) > 1 and c["block"][0] < c["lhs"].shape[1]
    if big:  # the C restatement (same arithmetic, threaded) for shapes numpy would take minutes on
        if c["kind"] == "fp8":
            q, s = c["w"]
            return clib.decode_gemm(O.bf16_bits(c["lhs"]), q, s, c["block"], c["sizes"], c["bias"], fused_swiglu=swiglu,
                                    dequant_bf16=like_reference, fp8_format=c["fmt"])
        return clib.decode_gemm(O.bf16_bits(c["lhs"]), O.bf16_bits(c["w"]), None, None, c["sizes"], c["bias"], fused_swiglu=swiglu)
    if c["kind"] == "fp8":
        return O.decode_gemm_reference(c["lhs"], c["w"], c["sizes"], block=c["block"], bias=c["bias"], fused_swiglu=swiglu,
                                       dequant_bf16=like_reference, fp8_format=c["fmt"])
    return O.decode_gemm_reference(c["lhs"], c["w"], c["sizes"], bias=c["bias"], fused_swiglu=swiglu)


def _run(c, swiglu, *, out_f32=False, implementation="pallas"):
    from lyra_amd.kernels.decode_gemm import decode_gemm
    from lyra_amd.nn.quant import QArray

    lhs = U.t_bf16(c["lhs"])
    if out_f32:
        lhs = lhs.to(torch.float32)
    if c["kind"] == "fp8":
        q, s = c["w"]
        rhs = QArray(U.t_fp8(q, c["fmt"]), U.t_f32(s), tuple(c["block"]))
        qd = torch.float8_e5m2 if c["fmt"] == 2 else torch.float8_e4m3fn
    else:
        rhs = U.t_bf16(c["w"])
        qd = None
    gs = torch.from_numpy(c["sizes"]).to(U.dev())
    bias = None if c["bias"] is None else U.t_f32(c["bias"])
    out = decode_gemm(lhs, rhs, gs, bias=bias, fused_swiglu=swiglu, quant_dtype=qd, implementation=implementation)
    torch.cuda.synchronize()
    return U.to_np(out)


@pytest.mark.parametrize("kind,block", [("bf16", None), ("fp8", (256, 256)), ("fp8", (512, 1)), ("fp8", (512, 128)), ("fp8", (64, 64)),
                                        ("e5m2", (256, 256)), ("e5m2", (512, 1))])
@pytest.mark.parametrize("swiglu", [False, True])
def test_small_grouped_shapes(kind, block, swiglu):
    M, G, K, N = 11, 4, 512, 512
    sizes = [3, 0, 7, 1]
    c = _case(1, M, G, K, N, sizes, kind=kind, block=block, bias=True, w_std=0.05)
    _note(f"gemm small kind={kind} block={block} swiglu={swiglu}")
    want = _want(c, swiglu)
    U.assert_close(_run(c, swiglu), want, what="bf16 out")
    U.assert_close(_run(c, swiglu, out_f32=True), want, atol=2e-3, rtol=2e-3, what="f32 out")


@pytest.mark.parametrize("sizes,M", [([0, 0, 0, 5], 5), ([5, 0, 0, 0], 5), ([1, 1, 1, 1], 4), ([2, 0, 1, 0], 6), ([0, 0, 0, 0], 3),
                                     ([17, 0, 33, 2], 52), ([70, 1, 0, 9], 80)])
def test_group_layouts_empty_groups_padding_rows_and_many_rows(sizes, M):
    for K in (256, 1024):  # 1024 rows of K are split across workgroups, 256 are not
        for kind, block in (("bf16", None), ("fp8", (256, 256))):
            for swiglu in (False, True):
                c = _case(2, M, 4, K, 256, sizes, kind=kind, block=(256, 256) if block else None, bias=True, w_std=0.05)
                _note(f"gemm groups sizes={sizes} M={M} K={K} kind={kind} swiglu={swiglu}")
                U.assert_close(_run(c, swiglu), _want(c, swiglu), what=f"sizes={sizes} K={K}")


def test_untouched_experts_are_never_read():
    """Weights of experts with no rows may be anything (here NaN codes / NaN scales)."""
    M, G, K, N = 6, 8, 512, 256
    sizes = [0, 4, 0, 0, 2, 0, 0, 0]
    c = _case(3, M, G, K, N, sizes, kind="fp8", block=(256, 256))
    want = _want(c, True)
    q, s = c["w"]
    q, s = q.copy(), s.copy()
    for g, n in enumerate(sizes):
        if n == 0:
            q[g] = 0x7F
            s[g] = np.nan
    got = _run(dict(c, w=(q, s)), True)
    U.assert_close(got, want, what="poisoned idle experts")


@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 512), (2048, 6144), (3072, 2048), (2880, 2816)])
def test_dense_projection_is_the_one_group_case(K, N):
    """quant.dot on [B,1,C] x [C,N] = decode_gemm with G == 1 (lyra-small widths, gpt-oss width 2880)."""
    for M in (1, 8, 64):
        for kind, block in (("fp8", (K, 1)), ("bf16", None)):
            c = _case(4, M, 1, K, N, [M], kind=kind, block=block)
            _note(f"gemm dense K={K} N={N} M={M} kind={kind}")
            swiglu = N % 256 == 0 and N == 6144
            U.assert_close(_run(c, swiglu), _want(c, swiglu, big=True), what=f"dense M={M}")


@pytest.mark.parametrize("kind,block", [("bf16", None), ("fp8", "channel"), ("fp8", (256, 1, 256))])
def test_quant_dot_takes_the_projections_of_a_decode_step_to_the_kernel(kind, block):
    """lyra_amd.nn.quant.dot with the reference's call shapes (lyra/model.py:307-309, 366, 614, 628: [B, 1, C] . [C, N] and
    the [C, 2, Hd] up projection under NN_INNER) against the float32 oracle on the same dequantised weights; "pallas" and
    "auto" must be the HIP kernel (bit-identical to the one-group decode_gemm call), "xla" the torch path."""
    from lyra_amd.kernels.decode_gemm import decode_gemm
    from lyra_amd.nn.quant import QArray, dot, einsum

    NN_INNER = (((2,), (0,)), ((), ()))
    B, C, Hd = 64, 2048, 3072
    rng = np.random.default_rng(61)
    x = O.bf16_round(rng.standard_normal((B, 1, C), dtype=np.float32))
    for shape in ((C, 2560), (C, 2, Hd)):
        w = (rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)).astype(np.float32)
        N = int(np.prod(shape[1:]))
        _note(f"quant.dot {kind} block={block} rhs={shape}")
        if kind == "fp8":
            blk = (C,) + (1,) * (len(shape) - 1) if block == "channel" else ((256, 256) if len(shape) == 2 else block)
            flat_blk = (blk[0], blk[-1])
            q, sc = clib.quantize_blocks(w.reshape(1, C, N), flat_blk)
            rhs = QArray(U.t_fp8(q.reshape(shape)), U.t_f32(sc.reshape((C // blk[0],) + shape[1:-1] + (shape[-1] // blk[-1],))), blk)
            rhs_flat = QArray(rhs.qval.reshape(1, C, N), rhs.scale.reshape(1, C // blk[0], -1), flat_blk)
            want = clib.decode_gemm(O.bf16_bits(x[:, 0]), q, sc, flat_blk, np.array([B], np.int32), None)
        else:
            rhs = U.t_bf16(w)
            rhs_flat = rhs.reshape(1, C, N)
            want = clib.decode_gemm(O.bf16_bits(x[:, 0]), O.bf16_bits(O.bf16_round(w).reshape(1, C, N)), None, None,
                                    np.array([B], np.int32), None)
        xt = U.t_bf16(x)
        got = dot(xt, rhs, dimension_numbers=NN_INNER, implementation="pallas")
        assert tuple(got.shape) == (B, 1) + shape[1:] and got.dtype == torch.bfloat16
        U.assert_close(U.to_np(got).reshape(B, N), want, what="dot bf16")
        got32 = dot(xt, rhs, dimension_numbers=NN_INNER, preferred_element_type=torch.float32, implementation="pallas")
        assert got32.dtype == torch.float32
        U.assert_close(U.to_np(got32).reshape(B, N), want, atol=2e-3, rtol=2e-3, what="dot f32")
        sizes = torch.full((1,), B, dtype=torch.int32, device=U.dev())
        direct = decode_gemm(xt[:, 0], rhs_flat, sizes, quant_dtype=torch.float8_e4m3fn if kind == "fp8" else None, implementation="pallas")
        assert torch.equal(got.reshape(B, N), direct)
        assert torch.equal(dot(xt, rhs, dimension_numbers=NN_INNER), got)  # auto = the kernel
        assert torch.equal(einsum("btc,c" + "jh"[: len(shape) - 1] + "->bt" + "jh"[: len(shape) - 1], xt, rhs), got)
        plain = dot(xt, rhs, dimension_numbers=NN_INNER, implementation="xla")
        U.assert_close(U.to_np(plain).reshape(B, N), want, what="dot plain path")


def _zipf_routing(rng, T, n_routed, k, n_shared):
    p = 1.0 / np.arange(1, n_routed + 1) ** 1.1
    p /= p.sum()
    ids = np.stack([rng.choice(n_routed, size=k, replace=False, p=p) for _ in range(T)])
    if n_shared:
        ids = np.concatenate([ids, np.broadcast_to(np.arange(n_routed, n_routed + n_shared), (T, n_shared))], axis=1)
    return np.bincount(ids.reshape(-1), minlength=n_routed + n_shared).astype(np.int32)


@pytest.mark.parametrize("T,k_routed", [(1, 3), (16, 3), (64, 3), (1, 4), (16, 4), (64, 4)])
def test_config3_moe_medium_shape_zipf_routing(T, k_routed):
    """Benchmark configuration 3 (MoE matmul at lyra-medium widths): width 4096, 31 routed + 1 shared expert, FP8 per-channel
    scales, Zipf(1.1) routing: top-(3+1) as lyra/variants.py has it (4 active experts, one of them shared) and 4 routed
    + the shared expert as the configuration's wording has it."""
    C, Hd, E = 4096, 4096, 32
    rng = np.random.default_rng(1003 + T + 100 * (k_routed - 3))
    sizes = _zipf_routing(rng, T, 31, k_routed, 1)
    M = int(sizes.sum())
    assert M == (k_routed + 1) * T
    up = _case(5, M, E, C, 2 * Hd, sizes, kind="fp8", block=(C, 1))
    _note(f"gemm cfg3 up T={T} M={M} touched={(sizes > 0).sum()}")
    want_up = _want(up, True, big=True)
    got_up = _run(up, True)
    U.assert_close(got_up, want_up, what="up+swiglu")
    down = _case(6, M, E, Hd, C, sizes, kind="fp8", block=(Hd, 1))
    down["lhs"] = O.bf16_round(want_up)
    _note(f"gemm cfg3 down T={T}")
    U.assert_close(_run(down, False), _want(down, False, big=True), what="down")


def test_config5_lyra_max_expert_shape_b128():
    """Benchmark configuration 5, the expert matmuls of one lyra-max MoE layer at B=128: width 4096, 63 routed + 1 shared
    expert, FP8 per-channel scales, top-(3+1) Zipf(1.1) routing: 512 rows, the shared expert holds 128 of them (two row
    blocks)."""
    C, Hd, E = 4096, 4096, 64
    rng = np.random.default_rng(1005)
    sizes = _zipf_routing(rng, 128, 63, 3, 1)
    M = int(sizes.sum())
    assert M == 512 and sizes[63] == 128
    up = _case(15, M, E, C, 2 * Hd, sizes, kind="fp8", block=(C, 1))
    _note(f"gemm cfg5 up M={M} touched={(sizes > 0).sum()}")
    want_up = _want(up, True, big=True)
    U.assert_close(_run(up, True), want_up, what="up+swiglu")
    del up
    down = _case(16, M, E, Hd, C, sizes, kind="fp8", block=(Hd, 1))
    down["lhs"] = O.bf16_round(want_up)
    _note("gemm cfg5 down")
    U.assert_close(_run(down, False), _want(down, False, big=True), what="down")


@pytest.mark.parametrize("kind,block", [("fp8", (512, 1)), ("fp8", (128, 128)), ("bf16", None), ("e5m2", (512, 1))])
def test_down_projection_with_many_units_takes_256_column_units(kind, block):
    """Without SwiGLU and with at least 1.75 rounds of 256-column units (here 34 row blocks x 16 = 544 for 256 workgroups)
    the grouped kernel picks the wider units on the device; the result must not depend on that choice."""
    G, K, N = 32, 512, 4096
    rng = np.random.default_rng(77)
    sizes = rng.integers(1, 9, size=G).astype(np.int32)
    sizes[3], sizes[31] = 70, 129  # two and three row blocks
    M = int(sizes.sum())
    c = _case(21, M, G, K, N, sizes, kind=kind, block=block, bias=True)
    _note(f"gemm many units {kind} {block} M={M}")
    U.assert_close(_run(c, False), _want(c, False, big=True), what=f"many units {kind}")


def test_reference_default_blocks_256_at_small_moe_shape():
    """lyra-small MoE: 15+1 experts, K=2048, up N=4096 with SwiGLU; QArray block (256,256) (model.py:154-156)."""
    rng = np.random.default_rng(8)
    sizes = _zipf_routing(rng, 8, 15, 3, 1)
    M = int(sizes.sum())
    c = _case(9, M, 16, 2048, 4096, sizes, kind="fp8", block=(256, 256), bias=True)
    U.assert_close(_run(c, True), _want(c, True, big=True), what="small up")


def test_linearity_and_row_independence_at_full_size():
    """Size-independent properties at the medium expert shape: out(2x) == 2 out(x) bit for bit (no SwiGLU,
    power-of-two scaling commutes with every rounding), and a row's result does not depend on its neighbours."""
    C, N, E = 4096, 4096, 32
    sizes = np.zeros(E, np.int32)
    sizes[[0, 5, 31]] = [3, 1, 64]
    M = int(sizes.sum())
    c = _case(10, M, E, C, N, sizes, kind="fp8", block=(C, 1))
    a = _run(c, False)
    b = _run(dict(c, lhs=c["lhs"] * 2.0), False)
    np.testing.assert_array_equal(b, a * 2.0)
    solo = np.zeros(E, np.int32)
    solo[31] = 1
    one = _run(dict(c, lhs=c["lhs"][10:11], sizes=solo), False)
    np.testing.assert_allclose(one[0], a[10], atol=1e-2, rtol=1e-2)


def test_quantize_on_the_fly_and_dispatch_contract():
    from lyra_amd.kernels.decode_gemm import decode_gemm
    from lyra_amd.nn.quant import QArray

    rng = np.random.default_rng(11)
    M, G, K, N = 4, 2, 512, 512
    lhs = O.bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    w = (rng.standard_normal((G, K, N)) * 0.05).astype(np.float32)
    sizes = np.array([1, 3], np.int32)
    gs = torch.from_numpy(sizes).to(U.dev())
    # float weights + quant_dtype=fp8: quantised with block (gcd(K,256), gcd(N,256)) first (decode_gemm.py:427-428)
    q, s = O.quantize(O.bf16_round(w), (256, 256))
    want = O.decode_gemm_reference(lhs, (q, s), sizes, block=(256, 256))
    for impl in ("auto", "pallas", "xla"):
        out = decode_gemm(U.t_bf16(lhs), U.t_bf16(w), gs, quant_dtype=torch.float8_e4m3fn, implementation=impl)
        assert out.shape == (M, N) and out.dtype == torch.bfloat16
        U.assert_close(U.to_np(out), want, what=f"on-the-fly {impl}")
    # a QArray without quant_dtype is dequantised to lhs.dtype and multiplied as bf16 (decode_gemm.py:432-434)
    rhs = QArray(U.t_fp8(q), U.t_f32(s), (256, 256))
    out = decode_gemm(U.t_bf16(lhs), rhs, gs, implementation="pallas")
    U.assert_close(U.to_np(out), O.decode_gemm_reference(lhs, (q, s), sizes, block=(256, 256), mode="ref"), what="dequantised")
    # unsupported N (not a multiple of 8): "pallas" raises, "auto" takes the plain path
    w2 = U.t_bf16(w[:, :, :204])
    with pytest.raises(ValueError, match="no HIP kernel configuration"):
        decode_gemm(U.t_bf16(lhs), w2, gs, implementation="pallas")
    out = decode_gemm(U.t_bf16(lhs), w2, gs, implementation="auto")
    U.assert_close(U.to_np(out), O.decode_gemm_reference(lhs, O.bf16_round(w[:, :, :204]), sizes), what="fallback")
    with pytest.raises(ValueError, match="Unsupported bias shape"):
        decode_gemm(U.t_bf16(lhs), U.t_bf16(w), gs, bias=torch.zeros(3, N, device=U.dev()))


@pytest.mark.parametrize("M,K,N,kind,block,swiglu", [
    (100, 1024, 512, "fp8", (256, 256), False),   # two row blocks, scale blocks that change along K
    (200, 1536, 768, "fp8", (1536, 1), True),     # four row blocks (rows past 192 only partly filled), per-channel scales
    (37, 512, 256, "bf16", None, False),          # bf16 weights, one slice of 512 rows
    (64, 4096, 1024, "fp8", (128, 128), False),   # 128-row scale blocks, 8 slices
    (16, 128, 128, "fp8", (128, 1), False),       # the smallest split shape
    (100, 1024, 512, "e5m2", (256, 256), False),  # e5m2 codes: scale blocks that change along K
    (64, 2048, 2048, "e5m2", (2048, 1), True),    # ... per-channel scales, SwiGLU
    (16, 2048, 512, "e5m2", (128, 128), False),   # ... 16-row blocks
])
def test_split_k_dense_variants(M, K, N, kind, block, swiglu):
    """One group with a few MB of weights runs split over K: bias, padding rows (group size < M) and SwiGLU included."""
    sizes = [M - 3]  # the last three rows lie past the group: zero product + bias
    c = _case(6, M, 1, K, N, sizes, kind=kind, block=block, bias=True, w_std=0.05)
    _note(f"gemm split-k M={M} K={K} N={N} kind={kind} block={block} swiglu={swiglu}")
    from lyra_amd import _lib

    assert _lib.lib.lyra_decode_gemm_splits(M, K, N, block[0] if block else 0) >= 1
    U.assert_close(_run(c, swiglu), _want(c, swiglu, big=True), what="split-k")


@pytest.mark.parametrize("G,M,K,N,swiglu", [(64, 300, 1024, 512, True), (64, 300, 1024, 512, False), (200, 256, 256, 256, False)])
def test_many_experts_unit_list(G, M, K, N, swiglu):
    """Many experts, most with a few rows, one with several row blocks, some empty, rows left over at the end."""
    rng = np.random.default_rng(G + M)
    sizes = rng.multinomial(M - 150 - 5, np.ones(G - 1) / (G - 1)).astype(np.int32)
    sizes[::7] = 0
    sizes = np.concatenate([sizes, [150]]).astype(np.int32)  # the last expert is the heavy one
    assert sizes.sum() <= M
    c = _case(8, M, G, K, N, sizes, kind="fp8", block=(K, 1), bias=True, w_std=0.05)
    _note(f"gemm unit list G={G} M={M} swiglu={swiglu} rows={int(sizes.sum())}")
    U.assert_close(_run(c, swiglu), _want(c, swiglu, big=True), what="unit list")


@pytest.mark.parametrize("K,N,swiglu", [(512, 2048, True), (512, 2048, False), (256, 8192, True), (256, 8192, False)])
def test_units_listed_by_cost_over_several_rounds(K, N, swiglu):
    """More (row block, column span) units than one round of workgroups: the row blocks are listed by cost class (full
    blocks and 49-63 rows, 33-48, 17-32, 1-16 rows), the left-over units go to the far-end workgroups and, from four full
    rounds on (the two wider shapes), odd rounds run backwards.  Experts with several full blocks plus a remainder of
    every class, empty experts between them, a heavy expert in the middle of the list and rows left over at the end; the
    result must not depend on any of that."""
    sizes = np.array([3, 0, 200, 64, 0, 33, 17, 16, 1, 48, 49, 0, 32, 130, 5, 63] + [2, 0, 7, 11] * 8, np.int32)
    G, M = sizes.size, int(sizes.sum()) + 6
    c = _case(21, M, G, K, N, sizes, kind="fp8", block=(K, 1), bias=True, w_std=0.05)
    _note(f"gemm cost-ordered unit list G={G} M={M} K={K} N={N} swiglu={swiglu}")
    want = _want(c, swiglu, big=True)
    first = _run(c, swiglu)
    U.assert_close(first, want, what="cost-ordered unit list")
    assert np.array_equal(_run(c, swiglu), first)


@pytest.mark.parametrize("kind,block,swiglu", [
    ("fp8", (2048, 1), True), ("fp8", (2048, 1), False), ("fp8", (256, 256), True), ("bf16", None, False),
    ("e5m2", (2048, 1), True), ("e5m2", (256, 256), False),
])
def test_few_units_are_cut_into_k_slices(kind, block, swiglu):
    """Fewer (row block, column span) units than compute units: every unit is cut along K, the slices meet in the
    workspace and the last workgroup to arrive sums them in K order.  Run three times on one workspace: the arrival
    counters must be back at zero after every launch, and the result must not depend on which workgroup came last."""
    G, M, K, N = 8, 6, 2048, 1024
    sizes = np.array([1, 0, 2, 0, 0, 1, 0, 2], np.int32)
    c = _case(9, M, G, K, N, sizes, kind=kind, block=block, bias=True, w_std=0.05)
    _note(f"gemm k-slices kind={kind} block={block} swiglu={swiglu}")
    want = _want(c, swiglu, big=True)
    first = _run(c, swiglu)
    U.assert_close(first, want, what="k slices")
    for _ in range(2):
        again = _run(c, swiglu)
        assert np.array_equal(again, first), "the sum over K slices depends on arrival order or on stale counters"


@pytest.mark.parametrize("M,K,N,kind,block,swiglu", [
    (64, 4096, 6144, "fp8", (4096, 1), False),   # a q/k/v projection of the 4096-wide variants: slices of 896 rows
    (40, 6144, 4096, "fp8", (6144, 1), False),   # their down projection: 8 slices of 768 rows
    (64, 4096, 4096, "fp8", (256, 256), True),   # scale blocks along K in slices of 1024 rows
    (16, 4096, 2048, "bf16", None, False),       # bf16 weights, two register sets refilled
    (64, 4096, 6144, "e5m2", (4096, 1), False),  # e5m2 codes in the looping variant
    (64, 4096, 4096, "e5m2", (256, 256), True),
])
def test_long_k_slices_of_larger_projections(M, K, N, kind, block, swiglu):
    """One group with tens of MB of weights: K is cut only as far as needed for one round of workgroups, so a slice is
    longer than what is requested up front and the register sets are refilled in a loop."""
    c = _case(10, M, 1, K, N, [M - 1], kind=kind, block=block, bias=True, w_std=0.03)
    _note(f"gemm long k slices M={M} K={K} N={N} kind={kind} block={block} swiglu={swiglu}")
    U.assert_close(_run(c, swiglu), _want(c, swiglu, big=True), what="long k slices")


@pytest.mark.parametrize("M,K,N,block", [(16, 8192, 8192, (1024, 128)), (128, 2048, 32768, (1024, 256)), (16, 12288, 8192, (96, 128))])
def test_scale_blocks_that_send_a_projection_to_the_general_kernel(M, K, N, block):
    """One group of 48-160 MB whose scale blocks do not tile a K slice of the K-split kernel: the general kernel runs, with
    more K slices than the K-split plan has; the workspace must be sized for the launch that runs."""
    from lyra_amd import _lib

    L = _lib.lib
    assert L.lyra_decode_gemm_splits(M, K, N, block[0]) == 0  # not the K-split kernel
    assert L.lyra_decode_gemm_workspace_for(M, 1, K, N, block[0], 0) <= L.lyra_decode_gemm_workspace(M, 1, K, N, 0)
    c = _case(12, M, 1, K, N, [M - 1], kind="fp8", block=block, bias=True, w_std=0.03)
    _note(f"gemm general kernel with scale blocks M={M} K={K} N={N} block={block}")
    U.assert_close(_run(c, False), _want(c, False, big=True), what="general kernel, blocks along K")


@pytest.mark.parametrize("block,swiglu", [((256, 256), True), ((128, 128), False), ((512, 256), False), ((64, 128), True)])
def test_many_experts_with_scale_blocks_along_k(block, swiglu):
    """Scale blocks shorter than K in the unit-list kernel: the accumulators are re-expressed whenever a wavefront's next
    step lies in another block (every 1, 2 or 4 steps depending on block height and on how the wavefronts interleave)."""
    G, M, K, N = 40, 300, 1024, 512
    rng = np.random.default_rng(17)
    sizes = rng.multinomial(M - 70, np.ones(G - 1) / (G - 1)).astype(np.int32)
    sizes = np.concatenate([sizes, [70]]).astype(np.int32)
    c = _case(12, M, G, K, N, sizes, kind="fp8", block=block, bias=True, w_std=0.05)
    _note(f"gemm unit list with k scale blocks block={block} swiglu={swiglu}")
    U.assert_close(_run(c, swiglu), _want(c, swiglu, big=True), what="unit list, k scale blocks")


@pytest.mark.parametrize("M,K,N,kind,block", [(5, 416, 131968, "bf16", None), (64, 416, 131200, "bf16", None), (33, 416, 132096, "fp8", (416, 1)),
                                             (64, 288, 204800, "bf16", None), (17, 480, 131328, "fp8", (96, 128)),
                                             (33, 416, 132096, "e5m2", (416, 1))])
def test_very_wide_projection_one_workgroup_per_compute_unit(M, K, N, kind, block):
    """A single projection with more than 1024 spans of 128 columns (the LM head): one workgroup per compute unit, the
    spans dealt out evenly.  Span counts that do not divide by the number of workgroups, with bias, 1 to 4 row tiles
    (K is chosen so that the plan is neither the one-pass nor the K-slice kernel)."""
    c = _case(31, M, 1, K, N, [M], kind=kind, block=block, bias=True, w_std=0.05)
    _note(f"gemm very wide M={M} K={K} N={N} kind={kind} block={block}")
    want = _want(c, False, big=True)
    U.assert_close(_run(c, False), want, what=f"N={N}")
    U.assert_close(_run(c, False, out_f32=True), want, atol=2e-3, rtol=2e-3, what=f"N={N} f32")


@pytest.mark.parametrize("G,M", [(1, 20), (6, 20)])
def test_zero_and_extreme_block_scales(G, M):
    """Scales a quantiser never produces but a caller may pass: exactly zero (the block must contribute nothing), and
    neighbouring blocks 1e8 apart.  K-split (one group) and unit-list (several groups) kernels."""
    K, N = 1024, 256
    sizes = [M] if G == 1 else [3, 0, 7, 2, 5, 3]
    c = _case(21, M, G, K, N, sizes, kind="fp8", block=(256, 128), bias=True, w_std=0.05)
    q, s = c["w"]
    s = s.copy()
    s[:, 1, :] = 0.0          # second K block of every expert: zero scale
    s[:, 2, 0] *= 1e4         # third block, first column block: large
    s[:, 3, 0] *= 1e-4        # fourth: tiny
    c["w"] = (q, s)
    _note(f"gemm zero / extreme scales G={G}")
    want = _want(c, False, big=True)
    got = _run(c, False)
    assert np.isfinite(got).all()
    U.assert_close(got, want, atol=2e-2 * max(1.0, float(np.abs(want).max()) / 50), what="zero / extreme scales")


@pytest.mark.parametrize("M,G,K,N,kind,block,swiglu,bias", [
    (64, 1, 4096, 2880, "bf16", None, False, True),          # gpt-oss-20b: output projection (64 heads of 64 -> width 2880)
    (64, 1, 2880, 5120, "fp8", (2880, 1), False, True),      # ... its q/k/v projection (whole spans, K = 2880)
    (64, 8, 2880, 5760, "fp8", (2880, 1), True, True),       # ... expert up projection with SwiGLU: 2880 output columns
    (64, 8, 2880, 2880, "fp8", (2880, 1), False, True),      # ... expert down projection
    (64, 8, 2880, 2880, "bf16", None, False, False),
    (300, 8, 2880, 2880, "fp8", (96, 64), False, True),      # several row blocks per expert, scale blocks along K
    (40, 3, 96, 8, "bf16", None, False, False),              # one lane of columns
    (40, 3, 96, 16, "fp8", (32, 8), True, True),             # SwiGLU down to 8 output columns
    (70, 5, 256, 200, "fp8", (64, 8), False, False),
    (33, 1, 512, 72, "fp8", (512, 8), False, True),
    (16, 1, 8192, 8200, "fp8", (8192, 1), False, False),     # large enough for K slices across workgroups + the finish kernel
    (64, 8, 2880, 5760, "e5m2", (2880, 1), True, True),      # e5m2 codes: expert kernel at a width that is not whole spans
    (300, 8, 2880, 2880, "e5m2", (96, 64), False, True),
    (33, 1, 512, 72, "e5m2", (512, 8), False, True),         # ... the general kernel
    (16, 1, 8192, 8200, "e5m2", (8192, 1), False, False),    # ... with K slices across workgroups
])
def test_widths_that_are_not_whole_spans(M, G, K, N, kind, block, swiglu, bias):
    """N % 8 == 0 (N % 16 == 0 with SwiGLU) is enough: in the expert kernel and in the general kernel the lanes past the
    last column of a partly filled 128-column span load nothing and store nothing (the reference's kernel needs
    n % 128 == 0, decode_gemm.py:88, and runs such shapes - all of gpt-oss-20b's, width 2880 - on its XLA path)."""
    rng = np.random.default_rng(M + G + N)
    cuts = np.sort(rng.integers(0, M + 1, G - 1)) if G > 1 else np.zeros(0, np.int64)
    sizes = np.diff(np.concatenate([[0], cuts, [M]])).astype(np.int32)
    if G > 2:
        sizes[1] = 0  # an expert without rows
    _note(f"gemm ragged width M={M} G={G} K={K} N={N} {kind} block={block} swiglu={swiglu} bias={bias} sizes={sizes.tolist()}")
    c = _case(N, M, G, K, N, sizes, kind=kind, block=block, bias=bias, w_std=0.03)
    want = _want(c, swiglu, big=True)
    got = _run(c, swiglu)
    assert got.shape == want.shape == (M, N // 2 if swiglu else N)
    U.assert_close(got, want, what=f"ragged width N={N}")
    got32 = _run(c, swiglu, out_f32=True)
    U.assert_close(got32, want, atol=4e-3, rtol=4e-3, what=f"ragged width N={N}, float32 out")


# ---- span-major weights (lyra_gemm_pack) -------------------------------------------------------------------------------
def _run_packed(c, swiglu, *, out_f32=False, bias=True, row_map=None, rows=None):
    """The case's weights through lyra_gemm_pack and lyra_decode_gemm_ex (the host wrapper lyra_amd.kernels.decode_fused.gemm)."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray

    if c["kind"] == "fp8":
        q, s = c["w"]
        rhs = QArray(U.t_fp8(q, c["fmt"]), U.t_f32(s), tuple(c["block"]))
    else:
        rhs = U.t_bf16(c["w"])
    G = len(c["sizes"])
    packed = F.pack_weights(rhs, glu=swiglu and G > 1)
    gs = torch.from_numpy(c["sizes"]).to(U.dev())
    b = None if (c["bias"] is None or not bias) else U.t_f32(c["bias"])
    out = F.gemm(U.t_bf16(c["lhs"]), packed, gs, fused_swiglu=swiglu, out_f32=out_f32, bias=b)
    torch.cuda.synchronize()
    return U.to_np(out)


def test_span_major_copy_is_the_documented_permutation():
    """lyra_gemm_pack against the layout written in the header, for both layouts, both element sizes and widths that do
    not fill their last span (zeros there)."""
    from lyra_amd.kernels import decode_fused as F

    rng = np.random.default_rng(5)
    for (G, K, N) in ((3, 64, 256), (2, 32, 360), (1, 96, 2880), (2, 32, 5760), (1, 32, 16)):
        for es in (1, 2):
            w = rng.integers(1, 250, (G, K, N)).astype(np.uint8) if es == 1 else rng.integers(1, 60000, (G, K, N)).astype(np.uint16)
            t = torch.from_numpy(w.view(np.int16) if es == 2 else w).to(U.dev())
            t = t.view(torch.bfloat16) if es == 2 else t.view(torch.float8_e4m3fn)
            for glu in (False, True):
                if glu and N % 16:
                    continue
                if es == 1:
                    from lyra_amd.nn.quant import QArray
                    rhs = QArray(t, torch.ones(G, 1, N, device=U.dev()), (K, 1))
                else:
                    rhs = t
                pk = F.pack_weights(rhs, glu=glu)
                torch.cuda.synchronize()
                got = pk.data.cpu().numpy().view(np.uint8 if es == 1 else np.uint16)
                if glu:
                    S, half = (N // 2 + 63) // 64, N // 2
                    want = np.zeros((G, S, K, 128), w.dtype)
                    for s_ in range(S):
                        n = min(64, half - 64 * s_)
                        want[:, s_, :, :n] = w[:, :, 64 * s_ : 64 * s_ + n]
                        want[:, s_, :, 64 : 64 + n] = w[:, :, half + 64 * s_ : half + 64 * s_ + n]
                else:
                    S = (N + 127) // 128
                    want = np.zeros((G, S, K, 128), w.dtype)
                    for s_ in range(S):
                        n = min(128, N - 128 * s_)
                        want[:, s_, :, :n] = w[:, :, 128 * s_ : 128 * s_ + n]
                assert got.size == want.size, (G, K, N, es, glu)
                np.testing.assert_array_equal(got.reshape(want.shape), want, err_msg=f"G{G} K{K} N{N} es{es} glu{glu}")


@pytest.mark.parametrize("kind,block", [("bf16", None), ("fp8", (256, 256)), ("fp8", "channel"), ("fp8", (64, 64)), ("e5m2", "channel")])
@pytest.mark.parametrize("swiglu", [False, True])
@pytest.mark.parametrize("M,G,K,N,sizes", [
    (11, 4, 512, 512, [3, 0, 7, 1]),                    # fewer units than workgroups: units cut into K slices
    (80, 4, 256, 1024, [70, 1, 0, 9]),                  # two row blocks in one group
    (300, 16, 512, 4096, None),                         # several rounds of units (units of two spans), cost-ordered list
    (260, 16, 256, 2048, None),                         # about two rounds of single spans
    (200, 40, 64, 4096, None),                          # 40 row blocks: units of two spans also without SwiGLU
    (300, 16, 64, 8192, None),                          # ... and with it (64 spans of 64 + 64 columns)
    (40, 3, 320, 2880, [20, 0, 20]),                    # a width that fills no whole number of spans (22.5)
    (7, 5, 64, 48, [2, 1, 0, 3, 1]),                    # narrower than one span, padding rows (sum < M is drawn below)
    (100, 8, 2048, 1024, [3, 2, 5, 27, 11, 17, 22, 0]),  # K slices of SwiGLU units with two row tiles: the summed tile is read by
    (23, 3, 2048, 4096, [6, 9, 5]),                     # other threads than wrote it (once a race, found by drawn shapes)
])
def test_span_major_weights_match_oracle_and_row_major_call(kind, block, swiglu, M, G, K, N, sizes):
    """Every grouped-matmul case through the span-major copy: against the oracle at the acceptance bound, float32 output at
    2e-3, and against the row-major call of the same kernel (same products; only the float32 summation order over K may
    differ, so the two agree to a few float32 roundings)."""
    if swiglu and N % 32:
        N = N // 32 * 32
    rng = np.random.default_rng(M + G + N)
    if sizes is None:
        cuts = np.sort(rng.integers(0, M + 1, G - 1))
        sizes = np.diff(np.concatenate([[0], cuts, [M]])).tolist()
        sizes[-1] = min(sizes[-1] + 0, 64 * 3)
        sizes[0] = 64  # a full block first in lhs order, last in the kernel's list
        M = int(sum(sizes)) + 3  # three rows past the last group
    blk = (K, 1) if block == "channel" else block
    if kind != "bf16" and blk is not None and (K % blk[0] or N % blk[1]):
        pytest.skip("block does not tile the shape")
    c = _case(7, M, G, K, N, sizes, kind=kind, block=blk, bias=True, w_std=0.05)
    _note(f"span-major kind={kind} block={blk} swiglu={swiglu} M={M} G={G} K={K} N={N}")
    want = _want(c, swiglu, big=G * K * N > (1 << 22))
    got = _run_packed(c, swiglu)
    U.assert_close(got, want, what="span-major bf16 out")
    got32 = _run_packed(c, swiglu, out_f32=True)
    U.assert_close(got32, want, atol=2e-3, rtol=2e-3, what="span-major f32 out")
    plain32 = _run(c, swiglu, out_f32=True)
    assert np.abs(got32 - plain32).max() <= 1e-4 * max(1.0, np.abs(plain32).max()), np.abs(got32 - plain32).max()


def test_span_major_untouched_experts_are_never_read():
    M, G, K, N = 6, 8, 512, 256
    sizes = [0, 4, 0, 0, 2, 0, 0, 0]
    c = _case(3, M, G, K, N, sizes, kind="fp8", block=(256, 256))
    want = _want(c, True)
    q, s = c["w"]
    q, s = q.copy(), s.copy()
    for g, n in enumerate(sizes):
        if n == 0:
            q[g] = 0x7F
            s[g] = np.nan
    U.assert_close(_run_packed(dict(c, w=(q, s)), True), want, what="poisoned idle experts, span-major")


@pytest.mark.parametrize("kind", ["bf16", "fp8", "e5m2"])
@pytest.mark.parametrize("M,K,N,swiglu", [(64, 2048, 2048, False), (64, 2048, 6144, True), (33, 4096, 2880, False), (8, 2880, 5120, False)])
def test_span_major_dense_projection_runs_split_over_k(kind, M, K, N, swiglu):
    """One group: the K-split kernel reads layout 1 (also under a fused SwiGLU, which its finish step applies); bit-identical
    to the row-major call, whose slices hold the same sums."""
    block = (K, 1) if kind != "bf16" else None
    c = _case(9, M, 1, K, N, [M], kind=kind, block=block, bias=False)
    _note(f"span-major dense kind={kind} M={M} K={K} N={N} swiglu={swiglu}")
    got = _run_packed(c, swiglu, out_f32=True)
    np.testing.assert_array_equal(got, _run(c, swiglu, out_f32=True))
    U.assert_close(got, _want(c, swiglu, big=True), atol=2e-3, rtol=2e-3, what="span-major dense")


@pytest.mark.parametrize("M,K,N,kind,block", [
    (64, 2048, 204800, "bf16", None),        # the LM head: one workgroup per compute unit, 6 or 7 spans each
    (5, 1248, 131968, "bf16", None),         # 1031 spans, one 16-row tile
    (33, 1248, 132096, "fp8", (1248, 1)),    # FP8 with per-column scales
    (17, 1440, 131328, "e5m2", (96, 128)),   # scale blocks along K
    (16, 32768, 8200, "fp8", (32768, 1)),    # K split across workgroups + the finish kernel; a last span that N does not fill
    (40, 262144, 1024, "bf16", None),        # few spans, many K slices
])
def test_span_major_weights_in_the_general_kernel(M, K, N, kind, block):
    """One group whose weights are too large for the K-split kernel (the LM head above all): the general kernel reads
    layout 1 as well - every wavefront one contiguous run of K rows of 128 weights - with results bit-identical to the
    row-major call (same products, same order), logits and tile maxima alike."""
    from lyra_amd import _lib
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray

    c = _case(43, M, 1, K, N, [M - 1], kind=kind, block=block, bias=True, w_std=0.05)
    _note(f"span-major general kernel M={M} K={K} N={N} kind={kind} block={block}")
    assert _lib.lib.lyra_decode_gemm_splits(M, K, N, block[0] if block else 0) == 0, "not a shape of the K-split kernel"
    got = _run_packed(c, False, out_f32=True)
    np.testing.assert_array_equal(got, _run(c, False, out_f32=True))
    U.assert_close(got, _want(c, False, big=True), atol=2e-3, rtol=2e-3, what="span-major general f32")
    U.assert_close(_run_packed(c, False), _want(c, False, big=True), what="span-major general bf16")
    # with the tile maxima (the launch of the LM head inside a decode step)
    if c["kind"] == "fp8":
        rhs = QArray(U.t_fp8(c["w"][0], c["fmt"]), U.t_f32(c["w"][1]), tuple(block))
    else:
        rhs = U.t_bf16(c["w"])
    gs = torch.from_numpy(c["sizes"]).to(U.dev())
    bias = U.t_f32(c["bias"]).reshape(-1)
    plain = F.gemm_tile_max(U.t_bf16(c["lhs"]), rhs, gs, bias=bias)
    packed = F.gemm_tile_max(U.t_bf16(c["lhs"]), F.pack_weights(rhs), gs, bias=bias)
    if plain is None:  # (a plan with K slices leaves no tile maxima, in either layout)
        assert packed is None
    else:
        assert torch.equal(plain[0], packed[0]) and torch.equal(plain[1], packed[1])
        np.testing.assert_array_equal(U.to_np(packed[0]), got)
