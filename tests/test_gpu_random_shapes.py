"""GPU parity of both operators at shapes drawn from a seeded generator (through the C ABI, against the CPU oracle).

The named tests pin the shapes of the model variants; these draws walk the rest of the supported domain - K that is
not a multiple of 128, 1 to 40 groups with empty groups and padding rows, every supported scale-block layout, odd
cache lengths, every head-group count up to 16, windows of any width, one position per row including rows that see
no key - so that every launch plan (one pass, K slices, unit list, general kernel; whole rows, chunks) meets sizes
nobody chose for it.  Tolerance as in the named tests: |got - want| <= 2e-2 + 1e-2*|want| against the fp32 oracle.
Each case is printed before it runs.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import lyra_oracle as O
from tests import gpu_util as U
from tests.test_gpu_attention import _run as run_attention
from tests.test_gpu_gemm import _case as gemm_case, _run as run_gemm, _want as gemm_want

pytestmark = pytest.mark.gpu


def _note(*a):
    print(*a, file=sys.stderr, flush=True)


def _blocks_for(rng, K, N):
    """A supported scale-block layout for a (K, N) weight (lyra_amd/kernels/decode_gemm.py: _scale_layout_supported)."""
    bks = [K] + [b for b in (32, 64, 96, 128, 256, 512) if K % b == 0 and b < K]
    bk = int(rng.choice(bks))
    bns = [b for b in (1, 8, 16, 64, 128, 256) if N % b == 0 and (bk == K or b % 8 == 0)]
    return bk, int(rng.choice(bns))


def _draw_gemm(seed):
    rng = np.random.default_rng(seed)
    swiglu = bool(rng.integers(0, 2))
    G = int(rng.choice([1, 1, 2, 3, 5, 8, 17, 40]))
    K = 32 * int(rng.choice([1, 2, 3, 5, 8, 9, 16, 23, 32, 64, 90]))
    n_unit = 256 if swiglu else 128
    N = n_unit * int(rng.choice([1, 1, 2, 3, 5, 8, 11]))
    while G * K * N > (1 << 23):  # keeps the numpy oracle in fractions of a second
        if G > 2:
            G = max(1, G // 2)
        elif N > n_unit:
            N -= n_unit
        else:
            K = max(32, K // 2 // 32 * 32)
    M = int(rng.choice([1, 2, 7, 16, 17, 33, 64, 65, 130, 300]))
    # group sizes: some groups empty, the sum sometimes short of M (the rest are padding rows)
    cuts = np.sort(rng.integers(0, M + 1, G - 1)) if G > 1 else np.zeros(0, np.int64)
    sizes = np.diff(np.concatenate([[0], cuts, [M]])).astype(np.int32)
    if G > 1:
        sizes[rng.integers(0, G)] = 0
    if rng.integers(0, 3) == 0:
        sizes[-1] = sizes[-1] // 2
    kind = "fp8" if rng.integers(0, 4) else "bf16"
    block = _blocks_for(rng, K, N) if kind == "fp8" else None
    bias = bool(rng.integers(0, 2))
    return dict(M=M, G=G, K=K, N=N, sizes=sizes.tolist(), kind=kind, block=block, bias=bias, swiglu=swiglu)


@pytest.mark.parametrize("seed", range(128))
def test_decode_gemm_at_drawn_shapes(seed):
    d = _draw_gemm(7000 + seed)
    _note(f"gemm draw {seed}: {d}")
    c = gemm_case(seed, d["M"], d["G"], d["K"], d["N"], d["sizes"], kind=d["kind"], block=d["block"], bias=d["bias"], w_std=0.05)
    want = gemm_want(c, d["swiglu"])
    got = run_gemm(c, d["swiglu"])
    U.assert_close(got, want, what=f"draw {seed}")


def _draw_attention(seed):
    rng = np.random.default_rng(seed)
    H = int(rng.choice([64, 128]))
    K = int(rng.choice([1, 2, 3, 4, 8]))
    G = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16]))
    B = int(rng.choice([1, 2, 3, 5, 9, 17, 40, 70]))
    S = int(rng.integers(1, 1500))
    while B * K * S * H > (1 << 23):
        if B > 2:
            B = max(1, B // 2)
        else:
            S = max(1, S // 2)
    sw = int(rng.choice([0, 0, 1, 5, 31, 32, 33, 128, 200, 1000]))
    fp8 = bool(rng.integers(0, 2))
    ragged = bool(rng.integers(0, 2))
    if ragged:
        pos = rng.integers(0, S, B).astype(np.int32)
        if B >= 3:
            pos[rng.integers(0, B)] = -1  # the row sees only its sink
        pos[B - 1] = S - 1
    else:
        pos = int(rng.integers(0, S))
    gate = bool(rng.integers(0, 2))
    f32 = bool(rng.integers(0, 4) == 0)
    return dict(B=B, N=K * G, K=K, S=S, H=H, sw=sw, fp8=fp8, pos=pos, gate=gate, f32=f32)


@pytest.mark.parametrize("seed", range(128))
def test_decode_attention_at_drawn_shapes(seed):
    d = _draw_attention(9000 + seed)
    _note(f"attention draw {seed}: { {k: (v.tolist() if isinstance(v, np.ndarray) else v) for k, v in d.items()} }")
    case = U.attention_case(seed, d["B"], d["N"], d["K"], d["S"], d["H"], fp8=d["fp8"])
    rng = np.random.default_rng(seed)
    gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((d["B"], d["N"]))))).astype(np.float32)) if d["gate"] else None
    sm_scale = d["H"] ** -0.5
    want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], sm_scale, d["sw"], d["pos"])
    if gate is not None:
        want = want * gate[:, :, None, None]
    if d["f32"]:
        # float32 output: held to what the kernel's one rounding allows - the probabilities enter the second product as
        # bf16, so an element may be off by 2^-9 * A with A = sum_j p_j |v_j| (the oracle on the absolute values gives A);
        # a gate adds one bf16 rounding of the result.  (With hundreds of keys this is the flat 4e-3 of the other tests;
        # with a handful of keys nothing averages out and A is the size of a single value.)
        v_abs = (case["v"][0] & np.uint8(0x7F), case["v"][1]) if d["fp8"] else np.abs(case["v"])
        a = O.decode_attention_reference(case["q"], case["k"], v_abs, case["sinks"], sm_scale, d["sw"], d["pos"])
        bound = 1e-3 + 2.0**-8 * a
        if gate is not None:
            bound = bound * gate[:, :, None, None] + 2.0**-8 * np.abs(want)
        got = run_attention(case, sm_scale, d["sw"], d["pos"], gate=gate, dtype=torch.float32)
        err = np.abs(np.asarray(got, np.float32).reshape(want.shape) - want)
        worst = int(np.argmax(err - bound))
        assert np.isfinite(got).all() and (err <= bound).all(), \
            f"draw {seed} f32: err {err.flat[worst]:.4g} > bound {bound.flat[worst]:.4g} at {worst}"
    else:
        got = run_attention(case, sm_scale, d["sw"], d["pos"], gate=gate)
        U.assert_close(got, want, what=f"draw {seed}")
    if isinstance(d["pos"], np.ndarray):
        assert np.all(got[d["pos"] < 0] == 0), "a row that sees no key attends only to its sink, whose value is zero"


@pytest.mark.parametrize("seed", range(24))
def test_fused_step_kernels_at_drawn_shapes(seed):
    """The checks of tests/test_gpu_fused.py (norm + projection, QK norm + RoPE + cache append, routing, combine, argmax,
    top-k sampling) at drawn sizes: widths that are not powers of two, 1 to 300 rows, up to 128 routed experts."""
    from tests import test_gpu_fused as TF

    rng = np.random.default_rng(11000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    B, C, n = int(rng.integers(1, 131)), pick([64, 100, 256, 1000, 2048, 2880, 4096, 8192]), pick([0, 1, 3, 8, 15, 16, 31, 63, 64, 100, 128])
    mode = "none" if n == 0 else pick(["gate", "logits"])
    _note(f"fused draw {seed}: rmsnorm_proj B={B} C={C} n={n} {mode}")
    TF.test_rmsnorm_proj(B, C, n, mode)

    K, G, H = pick([1, 2, 4, 8]), pick([1, 2, 4, 8]), pick([64, 128])
    B, S = int(rng.integers(1, 71)), int(rng.integers(2, 600))
    fp8, qknorm, per_row = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    _note(f"fused draw {seed}: qkv_post B={B} N={K * G} K={K} S={S} H={H} fp8={fp8} qknorm={qknorm} per_row={per_row}")
    TF.test_qkv_post(B, K * G, K, S, H, fp8, qknorm, per_row)

    T, n_routed, n_shared = int(rng.integers(1, 301)), int(rng.integers(2, 129)), int(rng.integers(0, 2))
    k = int(rng.integers(1, min(8, n_routed) + 1))
    _note(f"fused draw {seed}: moe_route T={T} routed={n_routed} shared={n_shared} k={k}")
    TF.test_moe_route(T, n_routed, n_shared, k)

    T, topk, C = int(rng.integers(1, 131)), int(rng.integers(1, 9)), 8 * int(rng.integers(1, 600))
    _note(f"fused draw {seed}: moe_combine T={T} topk={topk} C={C}")
    TF.test_moe_combine(T, topk, C)

    rows, cols = int(rng.integers(1, 131)), int(rng.integers(1, 60000))
    ld = (cols + 3) // 4 * 4 + 4 * int(rng.integers(0, 3))
    _note(f"fused draw {seed}: argmax rows={rows} cols={cols} ld={ld}")
    TF.test_argmax_first_maximum(rows, cols, ld)
    kk, temperature = int(rng.integers(1, 9)), float(rng.choice([0.3, 0.8, 1.0, 1.5]))
    _note(f"fused draw {seed}: sample_topk rows={rows} cols={cols} ld={ld} k={kk} T={temperature}")
    TF.test_sample_topk_matches_oracle(rows, cols, ld, kk, temperature)


def _draw_front_step(seed):
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    H, K, G = pick([64, 128]), pick([1, 2, 4, 8]), pick([1, 2, 3, 4, 8, 16])
    B, S = int(rng.integers(1, 71)), int(rng.integers(2, 1500))
    positions = pick(["full", "ragged", "short", "edges"])
    if positions == "edges":
        B = min(B, 10)
    if positions != "full":
        B = min(B, 256 // K)  # more pairs than compute units with one position per row is the whole-row kernel's case
    return dict(B=B, N=K * G, K=K, S=S, H=H, fp8=bool(rng.integers(0, 2)), qknorm=bool(rng.integers(0, 2)),
                sw=pick([0, 0, 1, 33, 128, 1000]), unsummed=pick([False, False, 1, 2, 3, 4, 5, 7, 8, 9, 12, 16]),
                positions=positions)


@pytest.mark.parametrize("seed", range(32))
def test_attention_front_step_at_drawn_shapes(seed):
    """The attention launch that also does QK norm, rotary embedding and cache append, against the two separate launches
    (outputs and cache bytes identical; tests/test_gpu_fused.py), at drawn head counts, cache lengths and positions."""
    from tests import test_gpu_fused as TF

    d = _draw_front_step(13000 + seed)
    _note(f"front step draw {seed}: {d}")
    TF.test_attention_with_the_front_step_equals_the_two_launches(
        d["B"], d["N"], d["K"], d["S"], d["H"], d["fp8"], d["qknorm"], d["sw"], d["unsummed"], d["positions"])


@pytest.mark.parametrize("seed", range(24))
def test_fused_variants_of_the_matmul_and_the_norm_at_drawn_shapes(seed):
    """The equalities of tests/test_gpu_fused.py - row gather and residual epilogue inside the matmul, K slices summed by
    the consumer, the MoE combine left to the norm behind it - bit for bit at drawn sizes."""
    from tests import test_gpu_fused as TF

    rng = np.random.default_rng(15000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    fp8, swiglu = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    G, K, N = pick([1, 1, 2, 3, 8, 16, 40]), 32 * pick([1, 2, 4, 8, 16, 32, 64]), (256 if swiglu else 128) * pick([1, 2, 3, 8, 16])
    while G * K * N > (1 << 24):
        G = max(1, G // 2)
    M = int(rng.integers(1, 321))
    _note(f"variants draw {seed}: row map / residual fp8={fp8} M={M} G={G} K={K} N={N} swiglu={swiglu}")
    TF.test_gemm_row_map_and_residual_epilogue(fp8, M, G, K, N, swiglu)

    H, Kh, Gq = pick([64, 128]), pick([1, 2, 4]), pick([1, 2, 4])
    if Kh * Gq * H % 256 == 0:  # (the output projection's scale blocks are (256, 256))
        fp8, B, C = bool(rng.integers(0, 2)), int(rng.integers(1, 131)), pick([256, 512, 1024, 2048, 4096])
        _note(f"variants draw {seed}: unsummed fp8={fp8} B={B} C={C} N={Kh * Gq} K={Kh} H={H}")
        TF.test_unsummed_projection_consumers_equal_summed_path(fp8, B, C, Kh * Gq, Kh, H)

    T, topk, gate = int(rng.integers(1, 131)), int(rng.integers(1, 17)), bool(rng.integers(0, 2))
    C, n = 8 * int(rng.integers(8, 600)), pick([1, 7, 15, 16, 32, 64]) if gate else pick([0, 1, 7, 15, 16, 63])
    _note(f"variants draw {seed}: uncombined T={T} topk={topk} C={C} n={n} gate={gate}")
    TF.test_uncombined_moe_layer_end_equals_combine_then_norm(T, topk, C, n, gate)


@pytest.mark.parametrize("seed", range(32))
def test_decode_gemm_at_drawn_widths_that_are_not_whole_spans(seed):
    """As test_decode_gemm_at_drawn_shapes, with N any multiple of 8 (16 with SwiGLU) up to 1500."""
    rng = np.random.default_rng(17000 + seed)
    swiglu = bool(rng.integers(0, 2))
    G = int(rng.choice([1, 1, 2, 3, 5, 8, 17]))
    K = 32 * int(rng.choice([1, 2, 3, 5, 8, 9, 16, 23, 32, 64, 90]))
    step = 16 if swiglu else 8
    N = step * int(rng.integers(1, 1500 // step))
    while G * K * N > (1 << 23):
        G, K = max(1, G // 2), (K if G > 1 else max(32, K // 2 // 32 * 32))
    M = int(rng.choice([1, 2, 7, 16, 17, 33, 64, 65, 130, 300]))
    cuts = np.sort(rng.integers(0, M + 1, G - 1)) if G > 1 else np.zeros(0, np.int64)
    sizes = np.diff(np.concatenate([[0], cuts, [M]])).astype(np.int32)
    if G > 1:
        sizes[rng.integers(0, G)] = 0
    kind = "fp8" if rng.integers(0, 4) else "bf16"
    block = None
    if kind == "fp8":
        bks = [K] + [b for b in (32, 64, 96, 128, 256, 512) if K % b == 0 and b < K]
        bk = int(rng.choice(bks))
        bns = [b for b in (1, 8, 16, 64, 128, 256) if N % b == 0 and (bk == K or b % 8 == 0)]
        block = (bk, int(rng.choice(bns)))
    bias = bool(rng.integers(0, 2))
    _note(f"gemm width draw {seed}: M={M} G={G} K={K} N={N} sizes={sizes.tolist()} {kind} block={block} bias={bias} swiglu={swiglu}")
    c = gemm_case(seed, M, G, K, N, sizes.tolist(), kind=kind, block=block, bias=bias, w_std=0.05)
    U.assert_close(run_gemm(c, swiglu), gemm_want(c, swiglu), what=f"width draw {seed}")
