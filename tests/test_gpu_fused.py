"""GPU parity of the fused decode-step launches (norm+projection, QK norm + RoPE + cache append, routing, combine,
matmul with row gather / residual epilogue) against the oracle's restatement of the reference's model code.

Integer results (top-k choice, group sizes, permutations, FP8 codes of unchanged inputs) are bit-exact; bf16 results
may differ from the float32 oracle by one bf16 rounding (|d| <= 2^-7 relative), float32 ones by accumulation order.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import lyra_oracle as O
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, file=sys.stderr, flush=True)


def _bf16_close(got, want, what, update=None):
    """Equal up to one bf16 step of a float32 oracle value rounded to bf16.

    `update`: where the value is residual + update and the update went through two bf16 roundings of its own (the
    weighted sum, then the sum times the residual scale), a different order of the float32 additions behind the sum can
    move the first rounding by one step and with it the second by up to two steps of the update - more than a step of
    the result where residual and update nearly cancel.  That much is allowed on top."""
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    err = np.abs(got - O.bf16_round(want.copy()))
    bound = np.abs(want) * 2.0**-7 + 1e-30
    if update is not None:
        bound = bound + np.abs(np.asarray(update, np.float32)) * 2.0**-6
    assert (err <= bound).all(), f"{what}: {int((err > bound).sum())} values off by more than one bf16 step, max {err.max()}"
    assert (err == 0).mean() > 0.97, f"{what}: only {(err == 0).mean():.3f} bit-identical"


@pytest.mark.parametrize("B,C,n,mode", [(64, 2048, 16, "gate"), (5, 256, 7, "logits"), (64, 2048, 15, "logits"), (3, 4096, 63, "logits"),
                                        (7, 2048, 0, "none"), (2, 4096, 32, "gate")])
def test_rmsnorm_proj(B, C, n, mode):
    from lyra_amd.kernels import decode_fused as F

    _say(f"rmsnorm_proj B{B} C{C} n{n} {mode}")
    rng = np.random.default_rng(B * 131 + C + n)
    x = O.bf16_round(rng.standard_normal((B, C), dtype=np.float32) * 3)
    scale = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    proj = (rng.standard_normal((C, n)) / np.sqrt(C)).astype(np.float32) if n else None
    bias = rng.standard_normal(n).astype(np.float32) if mode == "logits" else None
    h, y = F.rmsnorm_proj(U.t_bf16(x), U.t_f32(scale), 1e-5, None if proj is None else U.t_f32(proj),
                          None if bias is None else U.t_f32(bias), gate=mode == "gate")
    want_h = O.rms_norm(x, scale, 1e-5)
    _bf16_close(U.to_np(h), want_h, "h")
    if n:
        hn = U.to_np(h)  # the projection must consume the bf16-rounded row
        logits = hn.astype(np.float64) @ proj.astype(np.float64) + (0 if bias is None else bias)
        if mode == "gate":
            _bf16_close(U.to_np(y), (2.0 / (1.0 + np.exp(-logits))).astype(np.float32), "gate")
        else:
            np.testing.assert_allclose(U.to_np(y), logits, atol=2e-5, rtol=1e-5)
    else:
        assert y is None


@pytest.mark.parametrize("B,V,C,n", [(64, 1000, 2048, 16), (7, 33, 256, 0), (5, 204800, 2048, 16)])
def test_embedding_gather_inside_the_first_norm(B, V, C, n):
    """lyra_rmsnorm_proj_embed: rows table[tokens] (lyra/model.py:747) normalised like lyra_rmsnorm_proj's, bit for bit;
    token ids outside [0, V) are clamped into the table (the rule stated in the header) instead of being read."""
    from lyra_amd.kernels import decode_fused as F

    _say(f"embed B{B} V{V} C{C} n{n}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(V + B)
    table = torch.randn(V, C, generator=g, device=dev).to(torch.bfloat16)
    scale = 1 + 0.1 * torch.randn(C, generator=g, device=dev)
    proj = torch.randn(C, n, generator=g, device=dev) / C**0.5 if n else None
    ids = torch.randint(0, V, (B,), generator=g, device=dev, dtype=torch.int32)
    ids[0], ids[-1] = 0, V - 1
    bad = ids.clone()
    bad[1], bad[2], bad[3] = -1, V, 2**31 - 1  # padding, one past the end, garbage
    for tokens in (ids, bad):
        h, y, x = F.embed_rmsnorm_proj(table, tokens, scale, 1e-5, proj, None, gate=True)
        rows = table[tokens.long().clamp(0, V - 1)]
        h2, y2 = F.rmsnorm_proj(rows, scale, 1e-5, proj, None, gate=True)
        assert torch.equal(x, rows) and torch.equal(h, h2)
        assert (y is None and y2 is None) or torch.equal(y, y2)


@pytest.mark.parametrize("B,N,K,S,H,fp8,qknorm,per_row", [
    (64, 16, 4, 512, 128, True, True, False),
    (3, 2, 1, 256, 64, True, True, True),
    (5, 8, 8, 128, 64, False, False, True),
    (4, 16, 4, 300, 128, False, True, False),
    (2, 4, 2, 64, 128, True, False, False),
])
def test_qkv_post(B, N, K, S, H, fp8, qknorm, per_row):
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray

    _say(f"qkv_post B{B} N{N} K{K} S{S} H{H} fp8={fp8} qknorm={qknorm} per_row={per_row}")
    rng = np.random.default_rng(B + N * 7 + S)
    qkv = O.bf16_round(rng.standard_normal((B, (N + 2 * K) * H), dtype=np.float32) * 2)
    qkv[0, N * H : N * H + H] = 0  # an all-zero key row: scale 1, codes 0
    qn = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32) if qknorm else None
    kn = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32) if qknorm else None
    cos_t, sin_t = O.rope_tables(S, H)
    pos = rng.integers(0, S, B).astype(np.int32) if per_row else np.full(B, S - 1, np.int32)
    pos_t = torch.from_numpy(pos).to(U.dev()) if per_row else torch.tensor(S - 1, dtype=torch.int32, device=U.dev())
    dev = U.dev()
    sentinel = 0x55
    if fp8:
        mk = lambda: QArray(torch.full((B, K, S, H), sentinel, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn),
                            torch.full((B, K, S, 1), 7.0, dtype=torch.float32, device=dev), (1, H))
    else:
        mk = lambda: torch.full((B, K, S, H), 7.0, dtype=torch.bfloat16, device=dev)
    ck, cv = mk(), mk()
    q = F.qkv_post(U.t_bf16(qkv), None if qn is None else U.t_f32(qn), None if kn is None else U.t_f32(kn), U.t_f32(cos_t),
                   U.t_f32(sin_t), pos_t, ck, cv, N, K, H, 1e-5)
    torch.cuda.synchronize()

    qw, kw, vw = np.split(qkv, [N * H, (N + K) * H], axis=-1)
    qw, kw, vw = qw.reshape(B, N, H), kw.reshape(B, K, H), vw.reshape(B, K, H)
    if qknorm:
        qw, kw = O.bf16_round(O.rms_norm(qw, qn, 1e-5)), O.bf16_round(O.rms_norm(kw, kn, 1e-5))
    cos, sin = cos_t[pos][:, None, :], sin_t[pos][:, None, :]
    qw, kw = O.rotate(qw, cos, sin), O.rotate(kw, cos, sin)
    got_q = U.to_np(q)
    # norm and rotation each round to bf16 once: allow two bf16 steps on q against the float32 chain
    assert np.abs(got_q - qw).max() <= np.abs(qw).max() * 2.0**-6
    assert (got_q == O.bf16_round(qw.copy())).mean() > 0.9

    rows = np.arange(B)
    for name, cache, want in (("k", ck, O.bf16_round(kw.copy())), ("v", cv, vw)):
        if fp8:
            codes = cache.qval.view(torch.uint8).cpu().numpy()
            scales = cache.scale.cpu().numpy()[..., 0]
            got_codes, got_scale = codes[rows, :, pos], scales[rows, :, pos]  # [B,K,H], [B,K]
            if name == "v":  # V is appended untouched: codes and scales are those of the reference quantiser, bit for bit
                wq, ws = O.quantize(want[:, :, None, :], (1, H))
                assert np.array_equal(got_codes, wq[:, :, 0]) and np.array_equal(got_scale, ws[:, :, 0, 0])
            else:  # K went through norm + RoPE (one bf16 step of slack): self-consistent quantisation of the GPU's own row
                deq = O.fp8_e4m3fn_decode(got_codes) * got_scale[..., None]
                np.testing.assert_allclose(deq, want, atol=np.abs(want).max() * 0.07, rtol=0.07)
                amax = np.abs(deq).max(-1)
                np.testing.assert_allclose(got_scale, np.where(amax > 0, amax / 448, 1.0), rtol=2e-2)
            # nothing but the appended row was written
            codes[rows, :, pos] = sentinel
            scales[rows, :, pos] = 7.0
            assert (codes == sentinel).all() and (scales == 7.0).all()
        else:
            arr = cache.float().cpu().numpy()
            got = arr[rows, :, pos]
            if name == "v":
                assert np.array_equal(got, want)
            else:
                assert np.abs(got - want).max() <= np.abs(want).max() * 2.0**-6
            arr[rows, :, pos] = 7.0
            assert (arr == 7.0).all()


def test_qkv_post_key_codes_bit_exact_at_position_zero():
    """At position 0 the rotation is the identity (cos 1, sin 0) and without QK norm the key row reaches the
    quantiser unchanged: its codes and scale must equal the reference quantiser's bit for bit."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray

    B, N, K, S, H = 9, 4, 2, 32, 128
    rng = np.random.default_rng(11)
    qkv = O.bf16_round(rng.standard_normal((B, (N + 2 * K) * H), dtype=np.float32) * np.exp(rng.standard_normal((B, 1)) * 3).astype(np.float32))
    cos_t, sin_t = O.rope_tables(S, H)
    dev = U.dev()
    mk = lambda: QArray(torch.zeros((B, K, S, H), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn),
                        torch.ones((B, K, S, 1), dtype=torch.float32, device=dev), (1, H))
    ck, cv = mk(), mk()
    q = F.qkv_post(U.t_bf16(qkv), None, None, U.t_f32(cos_t), U.t_f32(sin_t), torch.tensor(0, dtype=torch.int32, device=dev), ck, cv,
                   N, K, H, 1e-5)
    assert np.array_equal(U.to_np(q).reshape(B, -1), qkv[:, : N * H])
    k = qkv[:, N * H : (N + K) * H].reshape(B, K, 1, H)
    wq, ws = O.quantize(k, (1, H))
    assert np.array_equal(ck.qval.view(torch.uint8)[:, :, 0].cpu().numpy(), wq[:, :, 0])
    assert np.array_equal(ck.scale[:, :, 0, 0].cpu().numpy(), ws[:, :, 0, 0])


@pytest.mark.parametrize("H,fp8", [(128, True), (64, False)])
def test_qkv_post_hands_over_unit_value_rows(H, fp8):
    """The new token's value rows scaled to unit length (lyra/model.py:353-354), taken before cache quantisation; a zero
    row stays zero (the 1e-10 under the root); rows whose position lies outside the cache are handed over all the same."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray

    B, N, K, S = 7, 4, 2, 16
    rng = np.random.default_rng(12)
    qkv = O.bf16_round(rng.standard_normal((B, (N + 2 * K) * H), dtype=np.float32) * np.exp(rng.standard_normal((B, 1)) * 3).astype(np.float32))
    qkv[2, (N + K) * H : (N + K + 1) * H] = 0.0
    cos_t, sin_t = O.rope_tables(S, H)
    dev = U.dev()
    if fp8:
        mk = lambda: QArray(torch.zeros((B, K, S, H), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn),
                            torch.ones((B, K, S, 1), dtype=torch.float32, device=dev), (1, H))
    else:
        mk = lambda: torch.zeros((B, K, S, H), dtype=torch.bfloat16, device=dev)
    pos = torch.tensor([0, 3, 15, 16, -1, 7, 8], dtype=torch.int32, device=dev)
    _say(f"qkv_post unit rows H{H} fp8={fp8}")
    q, vn = F.qkv_post(U.t_bf16(qkv), None, None, U.t_f32(cos_t), U.t_f32(sin_t), pos, mk(), mk(), N, K, H, 1e-5, unit_v=True)
    torch.cuda.synchronize()
    v = qkv[:, (N + K) * H :].reshape(B, K, H)
    want = O.unit_rows(v, mode="ref")
    got = U.to_np(vn)
    assert np.abs(got - want).max() <= 2.0**-8  # one bf16 step at magnitude <= 1 (rsqrt vs 1/sqrt)
    assert (got == want).mean() > 0.9
    assert np.all(got[2, 0] == 0)
    np.testing.assert_allclose(np.sum(got.astype(np.float64) ** 2, -1)[np.abs(v).max(-1) > 0], 1.0, atol=2e-2)


@pytest.mark.parametrize("T,n_routed,n_shared,k", [(64, 15, 1, 3), (5, 7, 1, 1), (128, 31, 1, 3), (33, 63, 1, 3), (16, 8, 0, 2), (1, 15, 1, 3),
                                                   (256, 15, 1, 3), (300, 15, 1, 3), (250, 127, 1, 3), (3, 128, 0, 8)])
def test_moe_route(T, n_routed, n_shared, k):
    from lyra_amd.kernels import decode_fused as F

    _say(f"moe_route T{T} routed{n_routed} shared{n_shared} k{k}")
    rng = np.random.default_rng(T + n_routed)
    logits = rng.standard_normal((T, n_routed)).astype(np.float32)
    logits[0, :] = 0.25  # all tied: the lowest indices win
    if T > 2:
        logits[2, 1::2] = logits[2, 0]  # ties with the maximum candidate
    scores, groups, row_map, dest = F.moe_route(U.t_f32(logits), n_routed, n_shared, k)
    w_scores, w_active, w_groups = O.route_tokens(logits, k, n_routed, n_shared)
    w_perm, w_dest = O.bpermute(w_active, w_groups, n_routed + n_shared)
    assert np.array_equal(groups.cpu().numpy(), w_groups)
    assert np.array_equal(dest.cpu().numpy(), w_dest)
    assert np.array_equal(row_map.cpu().numpy(), w_perm // (k + n_shared))
    np.testing.assert_allclose(scores.cpu().numpy(), w_scores, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("T,topk,C", [(64, 4, 2048), (3, 2, 256), (17, 4, 4096)])
def test_moe_combine(T, topk, C):
    from lyra_amd.kernels import decode_fused as F

    rng = np.random.default_rng(T)
    rows = O.bf16_round(rng.standard_normal((T * topk, C), dtype=np.float32))
    x = O.bf16_round(rng.standard_normal((T, C), dtype=np.float32))
    scores = rng.random((T, topk)).astype(np.float32)
    dest = rng.permutation(T * topk).astype(np.int32)
    rs = 0.1767766952966369
    out = F.moe_combine(U.t_bf16(rows), U.t_f32(scores), torch.from_numpy(dest).to(U.dev()), U.t_bf16(x), rs)
    t = O.bf16_round(O.combine(rows, scores, dest))
    t = O.bf16_round(t * np.float32(rs))
    want = x + t
    _bf16_close(U.to_np(out), want, "combine", update=t)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("M,G,K,N,swiglu", [(64, 1, 2048, 2048, False), (256, 16, 2048, 4096, True), (48, 8, 1024, 2048, False),
                                              (320, 40, 512, 4096, False)])  # the last: enough units for the 256-column ones
def test_gemm_row_map_and_residual_epilogue(fp8, M, G, K, N, swiglu):
    """The fused variants must equal the plain kernel composed with the torch ops they replace, bit for bit."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import quantize

    _say(f"gemm_ex fp8={fp8} M{M} G{G} K{K} N{N} swiglu={swiglu}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(M + G)
    tokens = max(1, M // 4)
    x = torch.randn(tokens, K, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(G, K, N, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    if fp8:
        w = quantize(w, torch.float8_e4m3fn, (K, 1))
    row_map = torch.randint(0, tokens, (M,), generator=g, device=dev, dtype=torch.int32)
    sizes = torch.zeros(G, dtype=torch.int32, device=dev)
    cuts = torch.sort(torch.randint(0, M + 1, (G - 1,), generator=g, device=dev)).values if G > 1 else torch.zeros(0, dtype=torch.int64, device=dev)
    bounds = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), cuts, torch.full((1,), M, dtype=torch.int64, device=dev)])
    sizes.copy_((bounds[1:] - bounds[:-1]).to(torch.int32))
    plain = F.gemm(x[row_map.long()].contiguous(), w, sizes, fused_swiglu=swiglu)
    gathered = F.gemm(x, w, sizes, rows=M, row_map=row_map, fused_swiglu=swiglu)
    assert torch.equal(plain, gathered)
    NO = plain.shape[1]
    res = torch.randn(M, NO, generator=g, device=dev).to(torch.bfloat16)
    scale = 0.1767766952966369
    fused = F.gemm(x, w, sizes, rows=M, row_map=row_map, fused_swiglu=swiglu, residual=res, out_scale=scale)
    assert torch.equal(fused, res + plain * scale)
    scaled = F.gemm(x, w, sizes, rows=M, row_map=row_map, fused_swiglu=swiglu, out_scale=scale)
    assert torch.equal(scaled, plain * scale)


@pytest.mark.parametrize("fp8", [False, True])
def test_fused_model_matches_unfused(fp8):
    """Whole decode step: the fused launches against the same step built from torch ops around the two kernels."""
    from dataclasses import replace

    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights, model_apply

    cfg = replace(MODEL_VARIANTS["dev"], sliding_window=128, use_sdpa_output_gate=True, seq_len=512)
    if fp8:
        cfg = apply_inference_overrides(cfg, fp8=True, fp8_attn=True)
    dev = U.dev()
    w = init_weights(cfg, dev, seed=3)
    B, S, start = 5, 512, 300
    outs = []
    for fused in (True, False):
        c = replace(cfg, fused_glue=fused)
        cache = init_cache(c, B, S, dev)
        cache.pos.fill_(start)
        tok = torch.arange(B, device=dev) * 7 + 1
        steps = []
        for _ in range(2):
            logits, _ = model_apply(tok, w, cache, c)
            steps.append(U.to_np(logits[:, : cfg.vocab_size]))
            tok = logits.argmax(-1)
        outs.append(steps)
    for a, b in zip(*outs):
        U.assert_close(a, b, atol=3e-2, rtol=2e-2, what="fused vs unfused logits")


@pytest.mark.parametrize("rows,cols,ld", [(64, 201088, 204800), (3, 1000, 1024), (1, 7, 8), (5, 4097, 4100), (130, 50000, 50000)])
def test_argmax_first_maximum(rows, cols, ld):
    from lyra_amd.kernels import decode_fused as F

    _say(f"argmax rows{rows} cols{cols} ld{ld}")
    g = torch.Generator(device=U.dev())
    g.manual_seed(rows + cols)
    x = torch.randn(rows, ld, generator=g, device=U.dev())
    x[:, cols:] = 100.0  # padding columns must not win
    x[0, : min(cols, 5)] = 50.0  # ties: the first index wins
    if rows > 1:
        x[1, :cols] = float("-inf")  # a fully masked row picks index 0
    if rows > 2:
        x[2, cols - 1] = 60.0  # the last valid column
    for _ in range(2):  # twice: the arrival counters must be back at zero
        got = F.argmax(x, cols).cpu().numpy()
        want = torch.argmax(x[:, :cols], dim=-1).cpu().numpy()
        want[0] = 0
        if rows > 1:
            want[1] = 0
        assert np.array_equal(got, want)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("B,C,N,K,H", [(64, 2048, 16, 4, 128), (5, 256, 2, 1, 64)])
def test_unsummed_projection_consumers_equal_summed_path(fp8, B, C, N, K, H):
    """Handing the K slices of a dense projection to the next kernel must give bit for bit what summing them first gives."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray, quantize

    _say(f"unsummed fp8={fp8} B{B} C{C}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(B + C)
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g, device=dev) * std).to(torch.bfloat16)
    width = (N + 2 * K) * H
    w_qkv, w_out = rnd(1, C, width, std=0.03), rnd(1, N * H, C, std=0.03)
    if fp8:
        w_qkv, w_out = quantize(w_qkv, torch.float8_e4m3fn, (C, 1)), quantize(w_out, torch.float8_e4m3fn, (min(N * H, 256), 256))
    one = torch.full((1,), B, dtype=torch.int32, device=dev)
    h, x = rnd(B, C), rnd(B, C)
    S = 64
    cos_t, sin_t = (U.t_f32(t) for t in O.rope_tables(S, H))
    qn = torch.ones(H, device=dev) * 1.1
    pos = torch.tensor(7, dtype=torch.int32, device=dev)
    mk = lambda: QArray(torch.zeros((B, K, S, H), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn),
                        torch.ones((B, K, S, 1), dtype=torch.float32, device=dev), (1, H))
    # q/k/v projection -> QK norm, RoPE, cache append
    un = F.gemm_unsummed(h, w_qkv, one)
    assert un is not None and un.partials.shape[1:] == (B, width)
    ck1, cv1, ck2, cv2 = mk(), mk(), mk(), mk()
    q1 = F.qkv_post(un, qn, qn, cos_t, sin_t, pos, ck1, cv1, N, K, H, 1e-5)
    q2 = F.qkv_post(F.gemm(h, w_qkv, one), qn, qn, cos_t, sin_t, pos, ck2, cv2, N, K, H, 1e-5)
    assert torch.equal(q1, q2)
    assert torch.equal(ck1.qval.view(torch.uint8), ck2.qval.view(torch.uint8)) and torch.equal(cv1.scale, cv2.scale)
    # output projection -> residual update -> next norm (+ router logits)
    t = rnd(B, N * H)
    un = F.gemm_unsummed(t, w_out, one)
    assert un is not None
    un.residual, un.scale = x, 0.1767766952966369
    scale = torch.rand(C, generator=g, device=dev) + 0.5
    router = torch.randn(C, 7, generator=g, device=dev) * 0.05
    h1, y1, x1 = F.rmsnorm_proj(un, scale, 1e-5, router, None)
    x2 = F.gemm(t, w_out, one, residual=x, out_scale=0.1767766952966369)
    h2, y2 = F.rmsnorm_proj(x2, scale, 1e-5, router, None)
    assert torch.equal(x1, x2) and torch.equal(h1, h2) and torch.equal(y1, y2)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("B,C,N,K,H,sw", [(64, 2880, 64, 8, 64, 0), (64, 2880, 64, 8, 64, 128), (5, 256, 2, 1, 64, 0), (8, 2048, 16, 4, 128, 0)])
def test_biased_projections_left_unsummed_equal_the_summed_path(fp8, B, C, N, K, H, sw):
    """Projections with a bias of their own (gpt-oss variants, lyra/model.py:310-313, 367-368): handing the K slices and
    the bias to the consumer - the attention launch with the front step, the norm kernel - must give bit for bit what the
    matmul's epilogue (bias added to the bf16 result, in bf16) followed by the consumer on the summed form gives."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import QArray, quantize

    _say(f"biased unsummed fp8={fp8} B{B} C{C} N{N} K{K} H{H} sw{sw}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(B + C + sw)
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g, device=dev) * std).to(torch.bfloat16)
    width = (N + 2 * K) * H
    w_qkv, w_out = rnd(1, C, width, std=0.03), rnd(1, N * H, C, std=0.03)
    if fp8:
        w_qkv, w_out = quantize(w_qkv, torch.float8_e4m3fn, (C, 1)), quantize(w_out, torch.float8_e4m3fn, (N * H, 1))
    b_qkv = rnd(width, std=0.5).to(torch.float32)  # (bf16 values as float32, what the epilogue takes)
    b_out = rnd(C, std=0.5).to(torch.float32)
    one = torch.full((1,), B, dtype=torch.int32, device=dev)
    h, x = rnd(B, C), rnd(B, C)
    S = 256
    cos_t, sin_t = (U.t_f32(t) for t in O.rope_tables(S, H))
    pos = torch.tensor(77, dtype=torch.int32, device=dev)
    sinks = torch.randn(N, generator=g, device=dev)

    def caches():
        kv = []
        for _ in range(2):
            c = rnd(B, K, S, H)
            kv.append(quantize(c, torch.float8_e4m3fn, (1, H)) if fp8 else c)
        return kv

    g.manual_seed(99)
    ck1, cv1 = caches()
    g.manual_seed(99)
    ck2, cv2 = caches()
    # q/k/v projection -> front step of the attention launch
    un = F.gemm_unsummed(h, w_qkv, one)
    assert un is not None
    un.bias = b_qkv
    a1 = F.attention_qkv(un, None, None, cos_t, sin_t, pos, ck1, cv1, sinks, H**-0.5, sw, N, K, H, 1e-5)
    summed = F.gemm(h, w_qkv, one, bias=b_qkv.reshape(1, -1), bias_after_cast=True)
    a2 = F.attention_qkv(summed, None, None, cos_t, sin_t, pos, ck2, cv2, sinks, H**-0.5, sw, N, K, H, 1e-5)
    assert a1 is not None and a2 is not None and torch.equal(a1, a2)
    raw = lambda c: c.qval.view(torch.uint8) if isinstance(c, QArray) else c.view(torch.int16)
    assert torch.equal(raw(ck1), raw(ck2)) and torch.equal(raw(cv1), raw(cv2))
    if fp8:
        assert torch.equal(ck1.scale, ck2.scale) and torch.equal(cv1.scale, cv2.scale)
    # output projection -> residual update -> next norm
    t = rnd(B, N * H)
    un = F.gemm_unsummed(t, w_out, one)
    assert un is not None
    un.residual, un.scale, un.bias = x, 0.1767766952966369, b_out
    scale = torch.rand(C, generator=g, device=dev) + 0.5
    h1, _, x1 = F.rmsnorm_proj(un, scale, 1e-5)
    x2 = F.gemm(t, w_out, one, bias=b_out.reshape(1, -1), bias_after_cast=True, residual=x, out_scale=0.1767766952966369)
    h2, _ = F.rmsnorm_proj(x2, scale, 1e-5)
    assert torch.equal(x1, x2) and torch.equal(h1, h2)


@pytest.mark.parametrize("T,topk,C,n,gate", [(64, 4, 2048, 16, True), (64, 4, 2048, 15, False), (3, 2, 256, 0, False), (17, 16, 4096, 7, False)])
def test_uncombined_moe_layer_end_equals_combine_then_norm(T, topk, C, n, gate):
    """Leaving the combine step of a MoE layer to the norm that follows must give bit for bit what combining first gives,
    and the combined row itself is checked against the oracle."""
    from lyra_amd.kernels import decode_fused as F

    _say(f"uncombined T{T} topk{topk} C{C} n{n}")
    dev = U.dev()
    rng = np.random.default_rng(T * 31 + topk)
    rows_np = O.bf16_round(rng.standard_normal((T * topk, C), dtype=np.float32))
    x_np = O.bf16_round(rng.standard_normal((T, C), dtype=np.float32))
    scores_np = rng.random((T, topk)).astype(np.float32)
    dest_np = rng.permutation(T * topk).astype(np.int32)
    rows, x, scores, dest = U.t_bf16(rows_np), U.t_bf16(x_np), U.t_f32(scores_np), torch.from_numpy(dest_np).to(dev)
    rs = 0.1767766952966369
    g = torch.Generator(device=dev)
    g.manual_seed(T)
    scale = torch.rand(C, generator=g, device=dev) + 0.5
    proj = torch.randn(C, n, generator=g, device=dev) * 0.05 if n else None
    bias = torch.randn(n, generator=g, device=dev) if (n and not gate) else None
    h1, y1, x1 = F.rmsnorm_proj(F.Uncombined(rows, scores, dest, x, rs), scale, 1e-5, proj, bias, gate=gate)
    x2 = F.moe_combine(rows, scores, dest, x, rs)
    h2, y2 = F.rmsnorm_proj(x2, scale, 1e-5, proj, bias, gate=gate)
    assert torch.equal(x1, x2) and torch.equal(h1, h2)
    assert (y1 is None and y2 is None) or torch.equal(y1, y2)
    t = O.bf16_round(O.bf16_round(O.combine(rows_np, scores_np, dest_np)) * np.float32(rs))
    _bf16_close(U.to_np(x1), x_np + t, "combined row", update=t)


@pytest.mark.parametrize("rows,cols,ld,k,temperature", [(64, 201088, 204800, 4, 0.8), (3, 1000, 1024, 8, 1.5), (130, 5000, 5000, 1, 0.3),
                                                        (1, 201088, 204800, 4, 0.8), (5, 7, 8, 4, 1.0)])
def test_sample_topk_matches_oracle(rows, cols, ld, k, temperature):
    """lyra/generate.py:46-53 with temperature > 0: the drawn column must be the oracle's for the same uniform numbers
    (rows whose uniform number lies within 1e-5 of a CDF boundary are not compared: expf differs in the last bit).  Ties
    between logits are planted, the padding beyond `cols` holds larger values that must be ignored, and the call is
    repeated on the same workspace."""
    from lyra_amd.kernels import decode_fused as F

    rng = np.random.default_rng(rows * 7 + k)
    x = rng.standard_normal((rows, ld)).astype(np.float32)
    x[:, cols:] = 50.0
    if cols > 40:
        x[0, 11] = x[0, 37] = 9.0  # a tie for first place: index 11 first
    u = rng.random(rows).astype(np.float32)
    u[0] = 0.0
    xt, ut = torch.from_numpy(x).to(U.dev()), torch.from_numpy(u).to(U.dev())
    want = O.sample_topk(x[:, :cols], u, k, temperature)
    kk = min(k, cols)
    order = np.argsort(-x[:, :cols], axis=1, kind="stable")[:, :kk]
    top = np.take_along_axis(x[:, :cols], order, 1) / np.float32(temperature)
    cdf = np.cumsum(np.exp(top - top[:, :1]), axis=1)
    cdf = cdf / cdf[:, -1:]
    safe = np.abs(cdf - u[:, None]).min(axis=1) > 1e-5
    assert safe.mean() > 0.9
    for _ in range(2):
        got = U.to_np(F.sample_topk(xt, ut, k, temperature, cols))
        assert (got < cols).all() and (got >= 0).all()
        assert (got[safe] == want[safe]).all(), np.flatnonzero(got != want)
    if cols > 40:
        assert got[0] == 11


def test_sample_token_draws_from_the_topk_softmax():
    """sample_token on the device path: over many draws the tokens of one row are distributed as the softmax of its 4
    largest logits / temperature, and nothing outside the top 4 is ever drawn."""
    from dataclasses import replace

    from lyra_amd.generate import sample_token
    from lyra_amd.model import MODEL_VARIANTS

    cfg = replace(MODEL_VARIANTS["dev"], sample_topk=4, sample_temperature=0.8, implementation="pallas")
    rng = np.random.default_rng(3)
    row = rng.standard_normal(cfg.padded_vocab_size).astype(np.float32)
    row[cfg.vocab_size:] = -np.inf
    logits = torch.from_numpy(np.repeat(row[None], 4096, 0)).to(U.dev())
    gen = torch.Generator(device=U.dev())
    gen.manual_seed(11)
    picks = np.concatenate([U.to_np(sample_token(logits, cfg, gen)) for _ in range(8)])
    top = np.argsort(-row[: cfg.vocab_size], kind="stable")[:4]
    assert set(picks.tolist()) <= set(top.tolist())
    want = torch.softmax(torch.from_numpy(row[top] / np.float32(0.8)), 0).numpy()
    got = np.array([(picks == t).mean() for t in top])
    np.testing.assert_allclose(got, want, atol=0.015)  # 32768 draws: ~4 standard errors


def test_sampler_with_its_own_generator_follows_the_documented_stream():
    """lyra_sample_topk_rng: the uniform number of row r at draw count c is the splitmix64 formula of the header; the launch
    then equals lyra_sample_topk fed those numbers, and leaves count + 1 behind - also when replayed from a graph."""
    from lyra_amd.kernels import decode_fused as F

    M64 = (1 << 64) - 1

    def splitmix(z):
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
        return z ^ (z >> 31)

    def uniforms(seed, count, rows):
        return np.array([(splitmix(seed ^ (((count + 1) * 0x9E3779B97F4A7C15) & M64) ^ (((r + 1) * 0xD1B54A32D192ED03) & M64)) >> 40) * 2.0**-24
                         for r in range(rows)], np.float32)

    dev = U.dev()
    rows, cols = 37, 5000
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    logits = torch.randn(rows, cols, generator=g, device=dev) * 3
    seed = 0x1234567890ABCDEF
    state = F.rng_state(dev, seed)
    for count in range(3):
        got = F.sample_topk(logits, state, 4, 0.8)
        want = F.sample_topk(logits, torch.from_numpy(uniforms(seed, count, rows)).to(dev), 4, 0.8)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"draw {count}"
        assert state.cpu().tolist() == [seed, count + 1]
    # every draw differs from the one before somewhere, and the picks follow the top-4 softmax over many draws
    row = torch.randn(cols, generator=g, device=dev) * 2
    many = row[None].repeat(4096, 1).contiguous()
    picks = torch.cat([F.sample_topk(many, state, 4, 0.8) for _ in range(4)]).cpu().numpy()
    top = np.argsort(-U.to_np(row), kind="stable")[:4]
    want_p = torch.softmax(torch.from_numpy(U.to_np(row)[top] / np.float32(0.8)), 0).numpy()
    np.testing.assert_allclose(np.array([(picks == t).mean() for t in top]), want_p, atol=0.02)
    # replayed from a graph: the count moves on by one per replay
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        F.sample_topk(logits, state, 4, 0.8, out=out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    start = state.cpu().tolist()[1]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        F.sample_topk(logits, state, 4, 0.8, out=out)
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        want = F.sample_topk(logits, torch.from_numpy(uniforms(seed, start + rep, rows)).to(dev), 4, 0.8)
        assert torch.equal(out, want) and state.cpu().tolist()[1] == start + rep + 1


def _tile_maxima(x: torch.Tensor) -> torch.Tensor:
    """Maximum of every 128-column tile of every row (the last tile may be short), as lyra_decode_gemm_tile_max leaves them."""
    rows, n = x.shape
    pad = torch.full((rows, (n + 127) // 128 * 128), float("-inf"), device=x.device)
    pad[:, :n] = x
    return pad.view(rows, -1, 128).amax(dim=2).contiguous()


@pytest.mark.parametrize("rows,cols,ld,case", [(64, 201088, 201088, "random"), (64, 201000, 201088, "random"), (3, 1000, 1024, "random"),
                                               (1, 7, 8, "random"), (5, 4097, 4104, "random"), (130, 50000, 50048, "random"),
                                               (4, 201088, 201088, "flat"), (6, 3000, 3072, "sparse")])
def test_tile_samplers_equal_the_full_samplers(rows, cols, ld, case):
    """lyra_argmax_tiles / lyra_sample_topk_tiles, which read a row's tile maxima and a few tiles, must return what
    lyra_argmax / lyra_sample_topk / lyra_sample_topk_rng return from the whole row: random logits with planted ties and a
    fully masked row, `cols` that cuts a tile, "flat" rows (every logit equal or one of two values: more tiles qualify than
    a workgroup lists) and "sparse" rows (fewer finite values than k)."""
    from lyra_amd.kernels import decode_fused as F

    _say(f"tile samplers rows{rows} cols{cols} ld{ld} {case}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(rows + cols)
    x = torch.randn(rows, ld, generator=g, device=dev)
    if case == "flat":
        x[0] = 1.5
        x[1] = torch.where(torch.rand(ld, generator=g, device=dev) < 0.5, 2.0, 1.0)
        x[2, ::128] = 7.0  # one equal maximum in every tile
    elif case == "sparse":
        x[:] = float("-inf")
        x[0, 5] = 1.0
        x[1, 129], x[1, 2999] = 2.0, 2.5
        x[2, 100], x[2, 101], x[2, 102] = 0.5, 0.5, 0.25
        x[4, :] = torch.randn(ld, generator=g, device=dev)
    else:
        x[0, : min(cols, 5)] = 50.0  # ties: the first index wins
        if rows > 1:
            x[1, :cols] = float("-inf")
        if rows > 2:
            x[2, cols - 1] = 60.0  # the last valid column
    x[:, cols:] = 100.0  # padding columns must not win (their tiles' maxima say 100)
    tm = _tile_maxima(x)
    u = torch.rand(rows, generator=g, device=dev)
    for _ in range(2):
        assert torch.equal(F.argmax(x, cols, tile_max=tm), F.argmax(x, cols))
        for k, temp in ((4, 0.8), (1, 0.3), (8, 1.5)):
            assert torch.equal(F.sample_topk(x, u, k, temp, cols, tile_max=tm), F.sample_topk(x, u, k, temp, cols)), (k, temp)
    a, b = F.rng_state(dev, 77), F.rng_state(dev, 77)
    for draw in range(3):
        assert torch.equal(F.sample_topk(x, a, 4, 0.8, cols, tile_max=tm), F.sample_topk(x, b, 4, 0.8, cols)), draw
    torch.cuda.synchronize()
    assert a.cpu().tolist() == b.cpu().tolist() == [77, 3]


@pytest.mark.parametrize("M,K,N,fp8,mask", [(64, 2048, 201088, False, True), (5, 1024, 200008, False, False), (17, 512, 400000, True, True)])
def test_lm_head_leaves_tile_maxima(M, K, N, fp8, mask):
    """lyra_decode_gemm_tile_max: the logits are bit for bit lyra_decode_gemm_ex's, the tile maxima are theirs, and
    sample_token with them (model.py hangs them on the logits tensor) picks what it picks without."""
    from dataclasses import replace

    from lyra_amd.generate import sample_token
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.model import MODEL_VARIANTS
    from lyra_amd.nn.quant import quantize

    _say(f"lm head tile max M{M} K{K} N{N} fp8={fp8}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(M + N)
    h = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(1, K, N, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    if fp8:
        w = quantize(w, torch.float8_e4m3fn, (K, 1))
    vocab = N - 40
    bias = None
    if mask:
        bias = torch.zeros(N, device=dev)
        bias[vocab:] = float("-inf")
    one = torch.full((1,), M, dtype=torch.int32, device=dev)
    got = F.gemm_tile_max(h, w, one, bias=bias)
    assert got is not None
    logits, tm = got
    want = F.gemm(h, w, one, out_f32=True, bias=bias)
    assert torch.equal(logits, want)
    assert torch.equal(tm, _tile_maxima(want))
    cfg = replace(MODEL_VARIANTS["dev"], vocab_size=vocab, sample_topk=4, sample_temperature=0.8, implementation="pallas")
    plain = logits.clone()
    logits.tile_max = (tm, logits._version)
    for c in (cfg, replace(cfg, sample_temperature=0.0)):
        a, b = F.rng_state(dev, 5), F.rng_state(dev, 5)
        gen_a, gen_b = torch.Generator(device=dev), torch.Generator(device=dev)
        gen_a.manual_seed(3), gen_b.manual_seed(3)
        assert torch.equal(sample_token(logits, c, gen_a), sample_token(plain, c, gen_b))
    logits[0, 3] = 1e9  # written to since: the maxima are stale and must not be used
    assert int(sample_token(logits, replace(cfg, sample_temperature=0.0))[0]) == 3
    # a small projection goes to other kernels: no tile maxima
    ws = (torch.randn(1, 256, 1024, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    assert F.gemm_tile_max(h[:, :256].contiguous(), ws, one) is None


@pytest.mark.parametrize("B,N,K,S,H,fp8,qknorm,sw,unsummed,positions", [
    (64, 16, 4, 4096, 128, True, True, 0, True, "full"),        # headline shape: one workgroup per (row, kv head)
    (64, 16, 4, 4096, 128, True, True, 128, True, "full"),      # sliding layer
    (8, 16, 4, 4096, 128, True, True, 0, True, "ragged"),       # chunked launch: only one chunk holds the new key
    (8, 16, 4, 4096, 128, True, True, 128, True, "ragged"),
    (3, 8, 2, 300, 64, True, False, 0, False, "short"),         # positions inside the tiles requested before the append
    (5, 8, 8, 515, 64, False, True, 0, True, "short"),
    (4, 32, 2, 700, 128, False, False, 33, False, "ragged"),    # 16 query heads per kv head, bf16 cache
    (10, 6, 2, 1000, 128, True, True, 0, True, "edges"),        # tile and chunk boundaries, first row, outside the cache
    (70, 4, 4, 200, 64, True, True, 0, True, "ragged"),         # 280 pairs, one position per row: the whole-row kernel's case, refused
    (64, 32, 8, 4096, 128, True, True, 0, True, "full"),        # lyra-medium: 512 pairs, two workgroups per compute unit
    (64, 64, 8, 4096, 64, True, False, 0, False, "full"),       # gpt-oss shape: 8 query heads per kv head, head width 64
    (64, 64, 8, 4096, 64, True, False, 128, False, "full"),
    # more query heads per kv head than wavefronts AND more slices than one request holds: every head needs both requests
    (4, 16, 2, 300, 64, True, True, 0, 5, "short"),
    (3, 32, 2, 515, 128, True, True, 0, 8, "ragged"),
    (2, 16, 1, 200, 128, False, True, 33, 12, "ragged"),
    (6, 24, 3, 400, 64, True, False, 128, 8, "edges"),
    (5, 32, 2, 1000, 64, False, False, 0, 12, "ragged"),
    (9, 8, 1, 260, 128, True, True, 0, 5, "short"),
    (8, 16, 4, 4096, 128, True, True, 0, 8, "ragged"),          # lyra-small at a small batch: the planner's 8 slices
])
def test_attention_with_the_front_step_equals_the_two_launches(B, N, K, S, H, fp8, qknorm, sw, unsummed, positions):
    """lyra_decode_attention_qkv against lyra_qkv_post(_sum) followed by lyra_decode_attention on copies of the same
    caches: outputs and every byte of the caches must be identical.  `unsummed`: False = the summed bf16 projection,
    True = 3 float32 slices, a number = that many slices."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.kernels.decode_attention import decode_attention
    from lyra_amd.nn.quant import QArray, quantize

    _say(f"attention_qkv B{B} N{N} K{K} S{S} H{H} fp8={fp8} qknorm={qknorm} sw={sw} unsummed={unsummed} {positions}")
    dev = U.dev()
    rng = np.random.default_rng(B * 3 + N + S)
    gen = torch.Generator(device=dev)
    gen.manual_seed(S + B)
    width = (N + 2 * K) * H
    if unsummed:
        n_slices = 3 if unsummed is True else int(unsummed)
        part = torch.randn(n_slices, B, width, device=dev, generator=gen) * (1.4 / n_slices**0.5)
        qkv_a, qkv_b = F.Unsummed(part, None, 1.0), F.Unsummed(part.clone(), None, 1.0)
    else:
        t = (torch.randn(B, width, device=dev, generator=gen) * 2).to(torch.bfloat16)
        qkv_a, qkv_b = t, t.clone()
    qn = U.t_f32((1 + 0.1 * rng.standard_normal(H)).astype(np.float32)) if qknorm else None
    kn = U.t_f32((1 + 0.1 * rng.standard_normal(H)).astype(np.float32)) if qknorm else None
    cos_t, sin_t = O.rope_tables(S, H)
    cos_t, sin_t = U.t_f32(cos_t), U.t_f32(sin_t)
    if positions == "full":
        pos = torch.tensor(S - 1, dtype=torch.int32, device=dev)
    else:
        if positions == "short":
            vals = rng.integers(0, 130, B)
        elif positions == "edges":
            vals = np.array([0, S - 1] + [31, 32, 127, 128, 255, 256, S, -1][: max(0, B - 2)])[:B]
        else:
            vals = rng.integers(0, S, B)
            vals[0] = S - 1
        pos = torch.from_numpy(np.asarray(vals, dtype=np.int32)).to(dev)
    hist = torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16)
    hist2 = torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16)

    def caches():
        if fp8:
            qk, qv = quantize(hist, torch.float8_e4m3fn, (1, H)), quantize(hist2, torch.float8_e4m3fn, (1, H))
            return QArray(qk.qval.clone(), qk.scale.clone(), (1, H)), QArray(qv.qval.clone(), qv.scale.clone(), (1, H))
        return hist.clone(), hist2.clone()

    sinks = U.t_f32(rng.standard_normal(N).astype(np.float32))
    gate = (2 * torch.sigmoid(torch.randn(B, N, device=dev, generator=gen))).to(torch.bfloat16)
    ka, va = caches()
    kb_, vb = caches()
    got = F.attention_qkv(qkv_a, qn, kn, cos_t, sin_t, pos, ka, va, sinks, H**-0.5, sw, N, K, H, 1e-5, gate=gate)
    if positions == "ragged" and sw == 0 and B * K > 256:
        assert got is None  # the whole-row kernel's case: the caller runs the two launches
        return
    assert got is not None
    q = F.qkv_post(qkv_b, qn, kn, cos_t, sin_t, pos, kb_, vb, N, K, H, 1e-5)
    want = decode_attention(q[:, :, None, :], kb_, vb, sinks, H**-0.5, sw, pos, gate=gate, implementation="pallas").reshape(B, N * H)
    torch.cuda.synchronize()
    for name, a, b in (("k", ka, kb_), ("v", va, vb)):
        if fp8:
            assert torch.equal(a.qval.view(torch.uint8), b.qval.view(torch.uint8)), f"{name} codes differ"
            assert torch.equal(a.scale, b.scale), f"{name} scales differ"
        else:
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"{name} cache differs"
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), \
        f"outputs differ in {(got != want).sum().item()} of {got.numel()} values, max {(got.float() - want.float()).abs().max().item()}"
    # a second call on the same caches (the row is appended again, identically) must give the same result
    got2 = F.attention_qkv(qkv_a, qn, kn, cos_t, sin_t, pos, ka, va, sinks, H**-0.5, sw, N, K, H, 1e-5, gate=gate)
    assert torch.equal(got2.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("M,K,N", [(64, 2048, 2048),    # K-split kernel + finish kernel
                                    (64, 2880, 5120),    # one-pass kernel (K not a multiple of 128)
                                    (64, 4096, 2880),    # general kernel (a width that is not whole spans)
                                    (5, 8192, 8200),     # general kernel, K split across workgroups + finish kernel
                                    (130, 512, 136)])
def test_gemm_bias_after_the_cast(fp8, M, K, N):
    """bias_after_cast: bf16(bf16(x @ w) + bias), then the scale / residual epilogue - bit for bit what the plain matmul
    followed by the bf16 torch ops of lyra/model.py:366-373 gives."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import quantize

    _say(f"gemm bias after cast fp8={fp8} M{M} K{K} N{N}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(M + N)
    x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(1, K, N, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    if fp8:
        w = quantize(w, torch.float8_e4m3fn, (K, 1))
    one = torch.full((1,), M, dtype=torch.int32, device=dev)
    bias = torch.randn(N, generator=g, device=dev).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g, device=dev).to(torch.bfloat16)
    b32 = bias.to(torch.float32).reshape(1, N).contiguous()
    plain = F.gemm(x, w, one)
    got = F.gemm(x, w, one, bias=b32, bias_after_cast=True)
    assert torch.equal(got, plain + bias)
    scale = 0.1767766952966369
    got = F.gemm(x, w, one, bias=b32, bias_after_cast=True, residual=res, out_scale=scale)
    assert torch.equal(got, res + (plain + bias) * scale)
    # and the float32 bias of the operator itself is something else: added before the cast
    pre = F.gemm(x, w, one, bias=b32)
    assert not torch.equal(pre, plain + bias)
    U.assert_close(U.to_np(pre), U.to_np(plain).astype(np.float32) + U.to_np(bias), atol=2e-2, rtol=1e-2, what="bias in float32")


def _tile16(x: torch.Tensor):
    """Row-major [rows, cols] bf16 -> Tiled16 (the documented layout, built with torch ops)."""
    from lyra_amd.kernels import decode_fused as F

    rows, cols = x.shape
    rb = (rows + 15) // 16
    pad = torch.zeros(rb * 16, cols, dtype=x.dtype, device=x.device)
    pad[:rows] = x
    data = pad.reshape(rb, 16, cols // 32, 32).permute(0, 2, 1, 3).contiguous().reshape(-1)
    return F.Tiled16(data, rows, cols)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("M,G,K,N,swiglu,gather", [(300, 16, 512, 4096, True, True), (300, 16, 2048, 2048, False, False),
                                                     (11, 4, 512, 512, True, True), (130, 3, 320, 2880, False, False),
                                                     (256, 16, 2048, 4096, True, True),
                                                     # one group: the K-split projections (their finish step writes the tiles)
                                                     (67, 1, 2048, 6144, True, False), (67, 1, 3072, 2048, False, False),
                                                     (36, 1, 2880, 5120, False, False), (131, 1, 4096, 4096, False, False)])
def test_expert_matmul_reads_and_writes_activations_in_tiles(fp8, M, G, K, N, swiglu, gather):
    """LYRA_LHS_TILED16 / LYRA_OUT_TILED16 of lyra_decode_gemm_ex: activations in tiles of 16 rows x 32 columns in, and out.  Only
    addresses change, so the result is the row-major call's bit for bit - with the token gather, with span-major weights,
    and with rows past the last group."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.nn.quant import quantize

    _say(f"tiled activations fp8={fp8} M{M} G{G} K{K} N{N} swiglu={swiglu} gather={gather}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(M + N)
    rng = np.random.default_rng(M + K)
    cuts = np.sort(rng.integers(0, M - 2, G - 1))
    sizes = np.diff(np.concatenate([[0], cuts, [M - 3]])).astype(np.int32)  # three rows past the last group
    sizes[int(np.argmax(sizes))] += 0
    gs = torch.from_numpy(sizes).to(dev)
    tokens = 64 if gather else M
    x = torch.randn(tokens, K, generator=g, device=dev).to(torch.bfloat16)
    row_map = torch.randint(0, tokens, (M,), generator=g, device=dev, dtype=torch.int32) if gather else None
    w = (torch.randn(G, K, N, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    if fp8:
        w = quantize(w, torch.float8_e4m3fn, (K, 1))
    bias = torch.randn(G, N, generator=g, device=dev)
    kw = dict(rows=M, row_map=row_map, fused_swiglu=swiglu, bias=bias)
    want = F.gemm(x, w, gs, **kw)
    got_in = F.gemm(_tile16(x), w, gs, **kw)
    assert torch.equal(got_in, want), "tiled input"
    NO = N // 2 if swiglu else N
    if NO % 32 == 0:
        got_out = F.gemm(_tile16(x), w, gs, out_tiled=True, **kw)
        assert isinstance(got_out, F.Tiled16) and torch.equal(got_out.untiled(), want), "tiled output"
        packed = F.pack_weights(w, glu=swiglu and G > 1)
        got_pk = F.gemm(_tile16(x), packed, gs, out_tiled=True, **kw)
        assert torch.equal(got_pk.untiled(), F.gemm(x, packed, gs, **kw)), "tiled, span-major weights"
    if G == 1 and not swiglu and N % 128 == 0:  # the unsummed slices of a projection, from tiled rows
        a, b = F.gemm_unsummed(x[:M], w, gs), F.gemm_unsummed(_tile16(x[:M]), w, gs)
        assert (a is None) == (b is None) and (a is None or torch.equal(a.partials, b.partials))


@pytest.mark.parametrize("B,C,n", [(64, 2048, 15), (5, 256, 7), (128, 4096, 63), (33, 2880, 32)])
def test_norm_writes_its_rows_in_tiles(B, C, n):
    from lyra_amd.kernels import decode_fused as F

    _say(f"tiled norm B{B} C{C} n{n}")
    dev = U.dev()
    g = torch.Generator(device=dev)
    g.manual_seed(B + C)
    x = (torch.randn(B, C, generator=g, device=dev) * 3).to(torch.bfloat16)
    scale = 1 + 0.1 * torch.randn(C, generator=g, device=dev)
    proj = torch.randn(C, n, generator=g, device=dev) / C**0.5
    h, y = F.rmsnorm_proj(x, scale, 1e-5, proj, None)
    ht, yt = F.rmsnorm_proj(x, scale, 1e-5, proj, None, tiled=True)
    assert isinstance(ht, F.Tiled16) and torch.equal(ht.untiled(), h) and torch.equal(yt, y)
    # ... and when the row is first formed from unsummed slices
    part = torch.randn(3, B, C, generator=g, device=dev)
    h2, _, x2 = F.rmsnorm_proj(F.Unsummed(part, x, 0.25), scale, 1e-5, proj, None)
    h2t, _, x2t = F.rmsnorm_proj(F.Unsummed(part, x, 0.25), scale, 1e-5, proj, None, tiled=True)
    assert torch.equal(h2t.untiled(), h2) and torch.equal(x2t, x2)
