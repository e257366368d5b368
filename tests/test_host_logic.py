"""Host-side mirror of the reference's plugin interface on CPU tensors: QArray arithmetic, dispatch contract, the
plain-framework ("xla") paths of both operators and the decode-step driver, each against the oracle."""
from dataclasses import replace

import numpy as np
import pytest
import torch

from oracle import decode_step as D
from oracle import lyra_oracle as O


def _bf16(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16)


def test_quantize_dequantize_bit_exact_with_oracle():
    from lyra_amd.nn.quant import QArray, dequantize, qupdate, quantize

    rng = np.random.default_rng(7)
    x = O.bf16_round(rng.standard_normal((2, 3, 8, 64), dtype=np.float32) * 5)
    x[0, 0, 0] = 0
    q = quantize(_bf16(x), torch.float8_e4m3fn, (1, 64))
    oq, osc = O.quantize(x, (1, 64))
    assert np.array_equal(q.qval.view(torch.uint8).numpy(), oq) and np.array_equal(q.scale.numpy(), osc)
    assert q.scale.shape == (2, 3, 8, 1) and q.block == (1, 64) and q.dtype == torch.float8_e4m3fn and q.shape == (2, 3, 8, 64)
    assert np.array_equal(dequantize(q, torch.bfloat16).float().numpy(), O.dequantize(oq, osc, (1, 64)))
    w = O.bf16_round(rng.standard_normal((2, 512, 256), dtype=np.float32) * 0.05)
    qw = quantize(_bf16(w), torch.float8_e4m3fn, (256, 256))
    ow, ows = O.quantize(w, (256, 256))
    assert np.array_equal(qw.qval.view(torch.uint8).numpy(), ow) and np.array_equal(qw.scale.numpy(), ows) and qw.scale.shape == (2, 2, 1)
    # functional update of one token, inputs untouched (quant.py:89-98)
    new = O.bf16_round(rng.standard_normal((2, 3, 1, 64), dtype=np.float32))
    before = q.qval.view(torch.uint8).clone()
    upd = qupdate(q, _bf16(new), (0, 0, 5, 0))
    assert torch.equal(q.qval.view(torch.uint8), before) and isinstance(upd, QArray)
    nq, ns = O.quantize(new, (1, 64))
    assert np.array_equal(upd.qval.view(torch.uint8)[:, :, 5].numpy(), nq[:, :, 0]) and np.array_equal(upd.scale[:, :, 5].numpy(), ns[:, :, 0])
    with pytest.raises(ValueError):
        quantize(q, torch.float8_e4m3fn, (1, 32))
    with pytest.raises(ValueError):
        quantize(_bf16(x), torch.bfloat16, (1, 64))


def test_quantize_to_e5m2_bit_exact_with_oracle():
    """The host-side producer of QArrays with dtype=float8_e5m2 (the other member of FP8_DTYPES, lyra/nn/quant.py:10)."""
    from lyra_amd.nn.quant import dequantize, quantize

    rng = np.random.default_rng(5)
    x = O.bf16_round((rng.standard_normal((3, 256, 128)) * np.exp(rng.standard_normal((3, 1, 1)) * 3)).astype(np.float32))
    for block in ((1, 128), (256, 1), (64, 64)):
        qa = quantize(torch.from_numpy(x), torch.float8_e5m2, block)
        wq, ws = O.quantize(x, block, fmt=2)
        assert np.array_equal(qa.qval.view(torch.uint8).numpy(), wq)
        assert np.array_equal(qa.scale.numpy(), ws)
        assert np.array_equal(dequantize(qa, torch.bfloat16).float().numpy(), O.dequantize(wq, ws, block, fmt=2))


def test_dispatch_contract():
    from lyra_amd.kernels.common import dispatch_kernel

    calls = []
    k = lambda: calls.append("kernel") or torch.zeros(1)
    r = lambda: calls.append("reference") or torch.zeros(1)
    common = dict(shape="s", tiling="t", kernel=k, reference=r)
    dispatch_kernel("op", implementation="auto", config=object(), **common)
    dispatch_kernel("op", implementation="pallas", config=object(), **common)
    dispatch_kernel("op", implementation="xla", config=object(), **common)
    dispatch_kernel("op", implementation="auto", config=None, **common)
    assert calls == ["kernel", "kernel", "reference", "reference"]
    with pytest.raises(ValueError, match="no HIP kernel configuration supports inputs"):
        dispatch_kernel("op", implementation="pallas", config=None, **common)
    with pytest.raises(ValueError):
        dispatch_kernel("op", implementation="cuda", config=None, **common)


def test_operator_selectors_are_decode_only():
    from lyra_amd.kernels.op import Mode, attn_op, gmm_op

    assert attn_op(Mode.DECODE, "xla").keywords == {"implementation": "xla"}
    assert gmm_op(Mode.DECODE, "auto").func.__name__ == "decode_gemm"
    for mode in Mode:
        if mode is not Mode.DECODE:
            with pytest.raises((ValueError, NotImplementedError)):
                attn_op(mode, "auto")


@pytest.mark.parametrize("fp8,sw", [(False, 0), (True, 0), (True, 128)])
def test_decode_attention_plain_path_on_cpu_matches_oracle(fp8, sw):
    from lyra_amd.kernels.decode_attention import decode_attention
    from lyra_amd.nn.quant import QArray

    rng = np.random.default_rng(3)
    B, N, K, S, H = 2, 8, 2, 384, 64
    q = O.bf16_round(rng.standard_normal((B, N, 1, H), dtype=np.float32))
    k = O.bf16_round(rng.standard_normal((B, K, S, H), dtype=np.float32))
    v = O.bf16_round(rng.standard_normal((B, K, S, H), dtype=np.float32))
    sinks = rng.standard_normal(N).astype(np.float32)
    pos = 300
    if fp8:
        (kq, ks), (vq, vs) = O.quantize(k, (1, H)), O.quantize(v, (1, H))
        kt = QArray(torch.from_numpy(kq).view(torch.float8_e4m3fn), torch.from_numpy(ks), (1, H))
        vt = QArray(torch.from_numpy(vq).view(torch.float8_e4m3fn), torch.from_numpy(vs), (1, H))
        want = O.decode_attention_reference(q, (kq, ks), (vq, vs), sinks, H**-0.5, sw, pos, mode="fp32")
    else:
        kt, vt = _bf16(k), _bf16(v)
        want = O.decode_attention_reference(q, k, v, sinks, H**-0.5, sw, pos, mode="fp32")
    got = decode_attention(_bf16(q), kt, vt, torch.from_numpy(sinks), H**-0.5, sw, torch.tensor(pos, dtype=torch.int32), implementation="auto")
    assert got.shape == (B, N, 1, H) and got.dtype == torch.bfloat16
    np.testing.assert_allclose(got.float().numpy(), want, atol=2e-2, rtol=1e-2)
    with pytest.raises(ValueError):  # CPU tensors have no HIP kernel
        decode_attention(_bf16(q), kt, vt, torch.from_numpy(sinks), H**-0.5, sw, torch.tensor(pos, dtype=torch.int32), implementation="pallas")


@pytest.mark.parametrize("fp8", [False, True])
def test_decode_gemm_plain_path_on_cpu_matches_oracle(fp8):
    from lyra_amd.kernels.decode_gemm import decode_gemm
    from lyra_amd.nn.quant import quantize

    rng = np.random.default_rng(4)
    sizes = np.asarray([3, 0, 2, 4], np.int32)
    M, K, N = 11, 128, 256  # two rows past the last group
    lhs = O.bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    w = O.bf16_round((rng.standard_normal((4, K, N)) * 0.05).astype(np.float32))
    bias = rng.standard_normal((4, N)).astype(np.float32)
    if fp8:
        wq = quantize(_bf16(w), torch.float8_e4m3fn, (128, 256))
        got = decode_gemm(_bf16(lhs), wq, torch.from_numpy(sizes), bias=torch.from_numpy(bias), fused_swiglu=True,
                          quant_dtype=torch.float8_e4m3fn, implementation="xla")
        want = O.decode_gemm_reference(lhs, O.quantize(w, (128, 256)), sizes, block=(128, 256), bias=bias, fused_swiglu=True, mode="fp32")
    else:
        got = decode_gemm(_bf16(lhs), _bf16(w), torch.from_numpy(sizes), bias=torch.from_numpy(bias), fused_swiglu=True, implementation="xla")
        want = O.decode_gemm_reference(lhs, w, sizes, bias=bias, fused_swiglu=True, mode="fp32")
    assert got.shape == (M, N // 2) and got.dtype == torch.bfloat16
    np.testing.assert_allclose(got.float().numpy(), want, atol=2e-2, rtol=1e-2)


def test_routing_and_permutation_match_oracle():
    from lyra_amd.model import MODEL_VARIANTS, MoEWeights, bpermute, route_tokens

    cfg = MODEL_VARIANTS["lyra-small"]
    rng = np.random.default_rng(9)
    T, C = 12, 64
    x = O.bf16_round(rng.standard_normal((T, C), dtype=np.float32))
    router = (rng.standard_normal((C, cfg.n_routed_experts)) * 0.2).astype(np.float32)
    rbias = rng.standard_normal(cfg.n_routed_experts).astype(np.float32)
    w = MoEWeights(router=torch.from_numpy(router), router_bias=torch.from_numpy(rbias), mlp_up=None, mlp_down=None, norm_scale=None)
    scores, active, groups = route_tokens(_bf16(x), w, cfg)
    logits = x @ router + rbias
    o_scores, o_active, o_groups = O.route_tokens(logits, cfg.n_active_routed_experts, cfg.n_routed_experts, cfg.n_shared_experts)
    assert np.array_equal(active.numpy(), o_active) and np.array_equal(groups.numpy(), o_groups)
    np.testing.assert_allclose(scores.numpy(), o_scores, atol=1e-6)
    perm, dest = bpermute(active)
    o_perm, o_dest = O.bpermute(o_active, o_groups, cfg.n_experts)
    assert np.array_equal(perm.numpy(), o_perm) and np.array_equal(dest.numpy(), o_dest)


@pytest.mark.parametrize("fp8", [False, True, "e5m2"])
def test_decode_step_driver_on_cpu_matches_oracle(fp8):
    """model_apply with the plain-framework operators on CPU tensors: the same op sequence as the oracle's decode step
    ("e5m2": FP8 weights and cache in the other format of FP8_DTYPES, lyra/nn/quant.py:10)."""
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights, model_apply

    cfg = replace(MODEL_VARIANTS["dev"], implementation="xla", seq_len=128, use_sdpa_output_gate=True, sliding_window=128)
    if fp8:
        cfg = apply_inference_overrides(cfg, fp8=True)
    if fp8 == "e5m2":
        cfg = replace(cfg, gemm_dtype=torch.float8_e5m2)
    dev = torch.device("cpu")
    w = init_weights(cfg, dev, seed=1)
    cache = init_cache(cfg, 2, 128, dev)
    cache.pos.fill_(0)
    wn, cn = D.weights_to_numpy(w, cfg), D.cache_to_numpy(cache)
    tokens = np.asarray([[3, 900], [17, 5]])
    for s in range(2):
        got, _ = model_apply(torch.from_numpy(tokens[s]), w, cache, cfg)
        want = D.decode_step(tokens[s], wn, cn, s, cfg)
        assert np.isneginf(got[:, cfg.vocab_size :].numpy()).all()
        np.testing.assert_allclose(got[:, : cfg.vocab_size].numpy(), want[:, : cfg.vocab_size], atol=6e-2, rtol=2e-2)
    assert int(cache.pos) == 2


def test_decode_step_driver_with_exclusive_self_attention_and_biases_on_cpu_matches_oracle():
    """The model options of the larger variants (use_learned_xsa, lyra/variants.py:38) and of the gpt-oss shapes (biases on
    q/k/v, the output projection and the MLPs, no shared expert, no QK norm, YaRN tables; variants.py:62-80) through the
    plain-framework operators: same op sequence as the oracle's decode step."""
    from lyra_amd.model import MODEL_VARIANTS, init_cache, init_weights, model_apply

    dev = torch.device("cpu")
    base = replace(MODEL_VARIANTS["dev"], implementation="xla", seq_len=64, sliding_window=16)
    cases = {
        "xsa": replace(base, use_learned_xsa=True, use_sdpa_output_gate=True),
        "gpt-oss-like": replace(base, use_qk_norm=False, use_qkv_bias=True, use_attn_out_bias=True, use_mlp_bias=True,
                                n_shared_experts=0, n_active_experts=2, rope_scale=4.0, mlp_map=("moe", "dense", "moe", "moe")),
    }
    for name, cfg in cases.items():
        w = init_weights(cfg, dev, seed=2)
        assert (w.layers[0].attn.xsa_alpha is not None) == cfg.use_learned_xsa
        cache = init_cache(cfg, 2, 64, dev)
        cache.pos.fill_(0)
        wn, cn = D.weights_to_numpy(w, cfg), D.cache_to_numpy(cache)
        tokens = np.asarray([[3, 900], [17, 5], [4, 4]])
        for s in range(3):
            got, _ = model_apply(torch.from_numpy(tokens[s]), w, cache, cfg)
            want = D.decode_step(tokens[s], wn, cn, s, cfg)
            np.testing.assert_allclose(got[:, : cfg.vocab_size].numpy(), want[:, : cfg.vocab_size], atol=6e-2, rtol=2e-2, err_msg=name)
        # the options are not no-ops: the same weights without them give different logits
        first = D.decode_step(tokens[0], wn, D.cache_to_numpy(init_cache(cfg, 2, 64, dev)), 0, cfg)
        for lw in w.layers:
            lw.attn.xsa_alpha = lw.attn.qkv_bias = lw.attn.out_bias = None
            lw.mlp.mlp_up_bias = lw.mlp.mlp_down_bias = None
        other, _ = model_apply(torch.from_numpy(tokens[0]), w, init_cache(cfg, 2, 64, dev), cfg)
        assert np.abs(other[:, : cfg.vocab_size].numpy() - first[:, : cfg.vocab_size]).max() > 0.05, name


def test_oracle_decode_step_skeleton_is_pinned_by_what_the_model_structure_fixes():
    """oracle/decode_step.py is a composition of pinned pieces; the composition itself is pinned here by consequences of the
    model's structure (lyra/model.py:284-374, 734-793) that do not depend on how the step is written down:
      * with every output projection and every down projection zero, every layer adds nothing: the residual stream stays
        the embedding rows through all layers, and the logits are the final norm of those rows times the unembedding
        (torch), -inf beyond the vocabulary;
      * the step writes, at the position it is given, the new token's keys - normalised, then rotated by that position -
        and its values as projected (torch, complex rotation), and touches no other cache row;
      * at position 0 with zero sinks' weight removed (sink logit -1e4) a token attends only to itself: the attention
        output is its own value row whatever q and k are, so the first layer's contribution is out_proj(gate * v)."""
    from lyra_amd.model import MODEL_VARIANTS, init_cache, init_weights

    dev = torch.device("cpu")
    cfg = replace(MODEL_VARIANTS["dev"], implementation="xla", seq_len=64, sliding_window=16, use_sdpa_output_gate=True)
    w = init_weights(cfg, dev, seed=5)
    for lw in w.layers:  # make the attention weights large enough that every piece matters
        lw.attn.qkv = (lw.attn.qkv.float() * 8).to(torch.bfloat16)
    tokens = np.asarray([11, 700, 42])
    B, C, H, N, K = 3, cfg.n_embd, cfg.head_dim, cfg.n_attn_heads, cfg.n_kv_heads
    bf = lambda t: t.to(torch.bfloat16).float()

    # 1. layers that add nothing
    wn = D.weights_to_numpy(w, cfg)
    for lw in wn["layers"]:
        lw["attn"]["out"] = np.zeros_like(lw["attn"]["out"])
        lw["mlp"]["mlp_down"] = np.zeros_like(lw["mlp"]["mlp_down"])
    cn = D.cache_to_numpy(init_cache(cfg, B, 64, dev))
    hidden = []
    logits = D.decode_step(tokens, wn, cn, 7, cfg, hidden_out=hidden)
    emb = bf(w.emb.float()[torch.from_numpy(tokens)])
    assert len(hidden) == cfg.n_layers + 1
    for h in hidden:
        assert np.array_equal(h, emb.numpy())
    normed = bf(torch.nn.functional.rms_norm(emb, (C,), w.norm_scale.float(), eps=cfg.norm_eps))
    want = normed @ w.unemb_t.float().reshape(C, -1)
    np.testing.assert_allclose(logits[:, : cfg.vocab_size], want[:, : cfg.vocab_size].numpy(), rtol=1e-4, atol=1e-4)
    assert np.isneginf(logits[:, cfg.vocab_size :]).all()

    # 2. what the step writes into the cache (layer 0), and only there
    wn = D.weights_to_numpy(w, cfg)
    cn = D.cache_to_numpy(init_cache(cfg, B, 64, dev))
    before_k = cn["k"][0].copy()
    pos = 9
    D.decode_step(tokens, wn, cn, pos, cfg)
    a = w.layers[0].attn
    hn = bf(torch.nn.functional.rms_norm(emb, (C,), a.norm_scale.float(), eps=cfg.norm_eps))
    qkv = bf(hn @ a.qkv.float()[0])
    k_new = qkv[:, N * H : (N + K) * H].reshape(B, K, H)
    v_new = qkv[:, (N + K) * H :].reshape(B, K, H)
    if cfg.use_qk_norm:
        k_new = bf(torch.nn.functional.rms_norm(k_new, (H,), a.knorm_scale.float(), eps=cfg.norm_eps))
    rate = 1.0 / cfg.rope_base ** (np.arange(0, H, 2) / H)
    z = (k_new[..., : H // 2].numpy() + 1j * k_new[..., H // 2 :].numpy()) * np.exp(1j * pos * rate)
    k_rot = bf(torch.from_numpy(np.concatenate([z.real, z.imag], -1).astype(np.float32)))
    np.testing.assert_allclose(cn["k"][0][:, :, pos], k_rot.numpy(), rtol=2e-2, atol=2e-3)  # (one bf16 step of slack)
    assert np.array_equal(cn["v"][0][:, :, pos], v_new.numpy())
    untouched = np.ones(64, bool)
    untouched[pos] = False
    assert np.array_equal(cn["k"][0][:, :, untouched], before_k[:, :, untouched])

    # 3. a lone token attends to itself
    wn = D.weights_to_numpy(w, cfg)
    for lw in wn["layers"]:
        lw["attn"]["sinks"] = np.full_like(lw["attn"]["sinks"], -1e4)
    wn["layers"] = wn["layers"][:1]
    wn["layers"][0]["mlp"]["mlp_down"] = np.zeros_like(wn["layers"][0]["mlp"]["mlp_down"])
    one_layer = replace(cfg, n_layers=1, mlp_map=cfg.mlp_map[:1])
    cn = D.cache_to_numpy(init_cache(one_layer, B, 64, dev))
    hidden = []
    D.decode_step(tokens, wn, cn, 0, one_layer, hidden_out=hidden)
    gate = bf(2 * torch.sigmoid(hn @ a.sdpa_gate.float()))  # [B, N]
    G = N // K
    own = bf(bf(v_new.repeat_interleave(G, dim=1)) * gate[:, :, None]).reshape(B, N * H)
    contrib = bf(bf(own @ a.out.float()[0]) * one_layer.residual_scale)
    np.testing.assert_allclose(hidden[1], bf(emb + contrib).numpy(), rtol=2e-2, atol=2e-2)
    assert np.abs(contrib.numpy()).max() > 0.05  # (the contribution is not lost in that tolerance)


def test_sampling():
    from lyra_amd.generate import sample_token
    from lyra_amd.model import MODEL_VARIANTS

    logits = torch.tensor([[0.0, 3.0, 3.0, -1.0], [5.0, 1.0, 0.0, 4.9]])
    greedy = replace(MODEL_VARIANTS["dev"], sample_temperature=0.0)
    assert sample_token(logits, greedy).tolist() == [1, 0]  # ties: lowest index
    cfg = replace(MODEL_VARIANTS["dev"], sample_temperature=0.8, sample_topk=2)
    g = torch.Generator().manual_seed(0)
    draws = torch.stack([sample_token(logits, cfg, g) for _ in range(200)])
    assert set(draws[:, 0].tolist()) <= {1, 2} and set(draws[:, 1].tolist()) <= {0, 3}
    assert len(set(draws[:, 0].tolist())) == 2


@pytest.mark.parametrize("fp8", [False, True])
def test_cache_append_outside_the_cache_writes_nothing(fp8):
    """cache_update with the position on the device: a row inside the cache is written (quantised for an FP8 cache), a
    position at or beyond its length, or below zero, leaves every byte as it was (the HIP kernels that append do the same)."""
    from lyra_amd.model import LayerCache, cache_update
    from lyra_amd.nn.quant import QArray, dequantize, quantize

    B, K, S, H = 2, 3, 8, 16
    g = torch.Generator().manual_seed(5)
    hist = [torch.randn(B, K, S, H, generator=g).to(torch.bfloat16) for _ in range(2)]
    new = [torch.randn(B, K, 1, H, generator=g).to(torch.bfloat16) for _ in range(2)]

    def fresh():
        if fp8:
            return LayerCache(*(quantize(h, torch.float8_e4m3fn, (1, H)) for h in hist))
        return LayerCache(*(h.clone() for h in hist))

    def raw(c):
        return [(a.qval.view(torch.uint8).clone(), a.scale.clone()) if isinstance(a, QArray) else (a.clone(),) for a in (c.k, c.v)]

    before = raw(fresh())
    for pos in (-1, S, S + 100):
        c = cache_update(fresh(), new[0], new[1], torch.tensor(pos, dtype=torch.int32))
        for got, want in zip(raw(c), before):
            assert all(torch.equal(a, b) for a, b in zip(got, want)), f"position {pos} changed the cache"
    for pos in (0, 5, S - 1):
        c = cache_update(fresh(), new[0], new[1], torch.tensor(pos, dtype=torch.int32))
        for arr, n, (old, *_) in zip((c.k, c.v), new, before):
            row = dequantize(arr, torch.float32)[:, :, pos] if isinstance(arr, QArray) else arr[:, :, pos].float()
            assert torch.allclose(row, n[:, :, 0].float(), atol=0.08 if fp8 else 0, rtol=0.07 if fp8 else 0)
            now = arr.qval.view(torch.uint8) if isinstance(arr, QArray) else arr
            keep = [i for i in range(S) if i != pos]
            assert torch.equal(now[:, :, keep], old[:, :, keep])


def test_quant_dot_and_einsum_on_the_plain_path():
    """lyra/nn/quant.py:106-113 on CPU tensors (the torch path): dequantise-if-QArray, then the contraction lax.dot_general
    describes; output axes are batch, lhs free, rhs free; output dtype is preferred_element_type or lhs.dtype."""
    from lyra_amd.nn.quant import dequantize, dot, einsum, quantize

    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 1, 64, generator=g).to(torch.bfloat16)
    w = (torch.randn(64, 2, 48, generator=g) * 0.1).to(torch.bfloat16)
    nn_inner = (((2,), (0,)), ((), ()))
    want = torch.einsum("btc,cjh->btjh", x.float(), w.float())
    got = dot(x, w, dimension_numbers=nn_inner)
    assert got.shape == (3, 1, 2, 48) and got.dtype == torch.bfloat16
    assert (got.float() - want).abs().max() <= 2e-2
    got32 = dot(x, w, dimension_numbers=nn_inner, preferred_element_type=torch.float32)
    assert got32.dtype == torch.float32 and (got32 - want).abs().max() <= 1e-5
    # a QArray weight is dequantised to the activation dtype first (quant.py:101-103)
    qw = quantize(w, torch.float8_e4m3fn, (32, 1, 16))
    assert qw.scale.shape == (2, 2, 3)
    want_q = torch.einsum("btc,cjh->btjh", x.float(), dequantize(qw, torch.bfloat16).float())
    assert (dot(x, qw, dimension_numbers=nn_inner, preferred_element_type=torch.float32) - want_q).abs().max() <= 1e-5
    assert torch.equal(dot(x[:, 0], qw.__class__(qw.qval[:, 0], qw.scale[:, 0], (32, 16))), dot(x, qw)[:, 0, 0])
    # default dimension numbers: last axis of lhs with first axis of rhs
    assert torch.equal(dot(x, w), got)
    # a contraction with a batch axis: [b, t, c] . [b, c, n] over c, batched over b
    wb = torch.randn(3, 64, 5, generator=g).to(torch.bfloat16)
    got_b = dot(x, wb, dimension_numbers=(((2,), (1,)), ((0,), (0,))), preferred_element_type=torch.float32)
    assert got_b.shape == (3, 1, 5)
    assert (got_b - torch.einsum("btc,bcn->btn", x.float(), wb.float())).abs().max() <= 1e-5
    # einsum: the projection pattern is dot; anything else is torch.einsum on the dequantised weight
    assert torch.equal(einsum("btc,cjh->btjh", x, qw), dot(x, qw))
    sc = torch.rand(3, 2, generator=g)
    rows = torch.randn(3, 2, 7, generator=g)
    assert torch.allclose(einsum("fkc,fk->fc", rows, sc), (rows * sc[:, :, None]).sum(1))  # lyra/model.py:557
    # the kernel cannot be asked for on CPU tensors
    with pytest.raises(ValueError, match="no HIP kernel"):
        dot(x, w, implementation="pallas")
