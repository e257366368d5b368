"""GPU parity of the decode-step driver (lyra_amd.model) against the CPU restatement of the reference's
model_apply in decode mode (oracle/decode_step.py).  Logits pass through every layer in bf16, so the bound is
looser than for a single kernel: |got - want| <= 6e-2 + 2e-2*|want| on float32 logits of magnitude ~1.
"""
import sys
from dataclasses import replace

import numpy as np
import pytest
import torch

from oracle import decode_step as D
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _run_steps(cfg, B, S, steps, start, use_c=False):
    from lyra_amd.model import init_cache, init_weights, model_apply

    dev = U.dev()
    w = init_weights(cfg, dev, seed=3)
    cache = init_cache(cfg, B, S, dev)
    rng = np.random.default_rng(5)
    # a synthetic history: every cached row below `start` holds N(0,1) keys/values
    from lyra_amd.nn.quant import QArray, quantize

    # (seeded: top-1 routing is a discontinuous function of the activations, so an unlucky history can put a router
    # logit pair within bf16 noise of a tie and send one token to a different expert than the float32-exact oracle)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2024)
    for layer in cache.layers:
        for name in ("k", "v"):
            hist = torch.randn(B, cfg.n_kv_heads, start, cfg.head_dim, device=dev, generator=gen).to(torch.bfloat16)
            dst = getattr(layer, name)
            if isinstance(dst, QArray):
                q = quantize(hist, dst.dtype, dst.block)
                dst.qval.view(torch.uint8)[:, :, :start] = q.qval.view(torch.uint8)
                dst.scale[:, :, :start] = q.scale
            else:
                dst[:, :, :start] = hist
    cache.pos.fill_(start)
    wn = D.weights_to_numpy(w, cfg)
    cn = D.cache_to_numpy(cache)
    tokens = rng.integers(0, cfg.vocab_size, (steps, B))
    for s in range(steps):
        print(f"model step {s} pos {start + s}", file=sys.stderr, flush=True)
        got, _ = model_apply(torch.from_numpy(tokens[s]).to(dev), w, cache, cfg)
        torch.cuda.synchronize()
        want = D.decode_step(tokens[s], wn, cn, start + s, cfg, use_c=use_c)
        g, t = U.to_np(got), want
        assert np.isneginf(g[:, cfg.vocab_size :]).all()
        U.assert_close(g[:, : cfg.vocab_size], t[:, : cfg.vocab_size], atol=6e-2, rtol=2e-2, what=f"step {s}")
        # the appended cache row must dequantise to the oracle's qupdate row (inputs differ by bf16 rounding
        # upstream, so codes may move by one step: compare values, and most codes must be identical)
        for l in (0, cfg.n_layers - 1):
            ck = cache.layers[l].k
            if isinstance(ck, QArray):
                from oracle import lyra_oracle as O

                kq = ck.qval.view(torch.uint8)[:, :, start + s].cpu().numpy()
                ks = ck.scale[:, :, start + s].float().cpu().numpy()
                oq, osc = cn["k"][l][0][:, :, start + s], cn["k"][l][1][:, :, start + s]
                fmt = 2 if ck.qval.dtype == torch.float8_e5m2 else 1
                step = 0.16 if fmt == 2 else 0.08  # one code step: 2 mantissa bits for e5m2, 3 for e4m3fn
                np.testing.assert_allclose(O.fp8_decode(kq, fmt) * ks, O.fp8_decode(oq, fmt) * osc, atol=step, rtol=step)
                if l == 0:
                    assert (kq == oq).mean() > 0.8  # the rest sits one FP8 step away (checked by value above)
    assert int(cache.pos.item()) == start + steps


@pytest.mark.parametrize("fp8", [False, True, "e5m2"])
def test_dev_model_decode_steps_match_oracle(fp8):
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides

    cfg = MODEL_VARIANTS["dev"]
    cfg = replace(cfg, sliding_window=128, use_sdpa_output_gate=True, seq_len=512, implementation="pallas")
    if fp8:
        cfg = apply_inference_overrides(cfg, fp8=True, fp8_attn=True)
    if fp8 == "e5m2":  # every FP8 array of the model (weights, cache) in the other format of FP8_DTYPES
        cfg = replace(cfg, gemm_dtype=torch.float8_e5m2)
    _run_steps(cfg, B=3, S=512, steps=3, start=200)


def test_dev_model_per_channel_scales_and_graph_replay():
    from lyra_amd.generate import GraphedDecoder
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights, model_apply

    cfg = apply_inference_overrides(replace(MODEL_VARIANTS["dev"], implementation="pallas"), fp8=True, fp8_attn=True, per_channel=True)
    _run_steps(cfg, B=2, S=256, steps=2, start=40)
    # the captured graph replays the same step: identical logits on identical inputs, replay after replay
    dev = U.dev()
    w = init_weights(cfg, dev, seed=3)
    cache = init_cache(cfg, 2, 256, dev)
    cache.pos.fill_(17)
    tok = torch.tensor([5, 9], device=dev)
    eager, _ = model_apply(tok, w, cache, cfg)
    eager = eager.clone()
    cache.pos.fill_(17)
    dec = GraphedDecoder(w, cache, cfg, batch=2)
    dec.tokens.copy_(tok)
    for _ in range(3):
        cache.pos.fill_(17)
        dec.tokens.copy_(tok)  # (the step replaces its tokens by the ones it drew)
        nxt = dec.step()
        torch.cuda.synchronize()
        assert torch.equal(dec.logits[:, : cfg.vocab_size], eager[:, : cfg.vocab_size])
        assert torch.equal(nxt.long(), eager.argmax(-1))
        assert int(cache.pos.item()) == 18  # the sampler moved the position on


def test_chained_replays_equal_eager_generate_calls_token_for_token():
    """lyra/generate.py:64-85: every drawn token is the next step's input at the next position.  Four replays of the
    captured step, chained on the device with no host work between them (the sampler writes the tokens where the next
    step's first kernel reads them and advances the position), against four eager generate() calls."""
    from lyra_amd.generate import GraphedDecoder, generate
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights

    cfg = apply_inference_overrides(replace(MODEL_VARIANTS["dev"], implementation="pallas", sample_temperature=0.0, seq_len=256),
                                    fp8=True, fp8_attn=True, per_channel=True)
    dev = U.dev()
    w = init_weights(cfg, dev, seed=3)
    B, start, n = 5, 30, 4
    first = torch.tensor([5, 9, 700, 1, 33], device=dev, dtype=torch.int32)

    def history(cache):
        gen = torch.Generator(device=dev)
        gen.manual_seed(11)
        from lyra_amd.nn.quant import quantize

        for layer in cache.layers:
            for dst in (layer.k, layer.v):
                hist = torch.randn(B, cfg.n_kv_heads, start, cfg.head_dim, device=dev, generator=gen).to(torch.bfloat16)
                q = quantize(hist, dst.dtype, dst.block)
                dst.qval.view(torch.uint8)[:, :, :start] = q.qval.view(torch.uint8)
                dst.scale[:, :, :start] = q.scale
        cache.pos.fill_(start)
        return cache

    eager_cache = history(init_cache(cfg, B, 256, dev))
    tok, want = first, []
    for _ in range(n):
        tok, eager_cache = generate(tok, w, eager_cache, cfg)
        want.append(tok.clone())
    want = torch.stack(want)
    assert int(eager_cache.pos.item()) == start + n

    cache = history(init_cache(cfg, B, 256, dev))
    dec = GraphedDecoder(w, cache, cfg, batch=B)
    dec.tokens.copy_(first)
    got = dec.decode(n)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert int(cache.pos.item()) == start + n
    # the appended cache rows are the same bits either way
    for a, b in zip(cache.layers, eager_cache.layers):
        assert torch.equal(a.k.qval.view(torch.uint8)[:, :, start : start + n], b.k.qval.view(torch.uint8)[:, :, start : start + n])
        assert torch.equal(a.v.scale[:, :, start : start + n], b.v.scale[:, :, start : start + n])


def _layer_by_layer(cfg, w, cache, pos_value, layer_inputs, margins, margin):
    """Runs every layer of the fused driver on the oracle's input of that layer (layer_inputs[l]; the last entry is the
    output of the last layer) and returns the worst relative error || got - want || / || want || of a row of a layer's
    output.  The cache row at pos_value is rewritten by each layer."""
    from lyra_amd import model as M
    from lyra_amd.kernels import decode_fused as F

    dev = U.dev()
    pos = torch.tensor(pos_value, dtype=torch.int32, device=dev)
    cos_t, sin_t = M._rope_tables(cfg, dev)
    ones = torch.ones(cfg.n_embd, dtype=torch.float32, device=dev)
    moe_seen = 0
    worst = 0.0
    for idx, layer in enumerate(w.layers):
        x = U.t_bf16(layer_inputs[idx])
        h, _ = M.attention_apply_fused(x, layer.attn, idx, pos, cos_t, sin_t, cache.layers[idx], cfg)
        ok = np.ones(x.shape[0], bool)
        if isinstance(layer.mlp, M.MoEWeights):
            h = M.moe_apply_fused(h, layer.mlp, cfg)
            ok = margins[moe_seen] > margin
            moe_seen += 1
        else:
            h = M.dense_mlp_apply_fused(h, layer.mlp, cfg)
        if isinstance(h, (F.Unsummed, F.Uncombined)):
            h = F.rmsnorm_proj(h, ones, cfg.norm_eps)[2]
        torch.cuda.synchronize()
        got, want = U.to_np(h), layer_inputs[idx + 1]
        rel = np.linalg.norm(got - want, axis=-1) / np.linalg.norm(want, axis=-1)
        worst = max(worst, float(rel[ok].max()))
    return worst


def _full_width_parity(cfg, B, S, start, steps, *, min_clear, moe_layers, hidden_tol, layer_tol=0.01, logit_atol=0.12, margin=0.03, without=None):
    """Whole decode steps of a model at its real widths against the CPU restatement (threaded C contractions; every
    operator exact in float32 on its bf16 / FP8 inputs and rounded to bf16 once at its output, which is what the kernels do:
    the reference's plain-JAX path also rounds the dequantised cache, the dequantised weights and the logits q.k to bf16
    inside the operators, and that alone moves a layer's output by 0.9 %).

    Top-k routing is discontinuous and random-init router logits lie close together, so the router bias of every expert is
    drawn from N(0,1) to spread them, and a row whose last selected / first unselected logits are within ``margin`` of each
    other in any MoE layer of any step so far is not compared (bf16 noise upstream can flip such a row to another expert,
    in the kernels as in either CPU restatement); at least ``min_clear`` rows must remain.  For those rows:
      * layer by layer (first step): every layer is run on the residual stream the oracle had at its input, and its output
        must match the oracle's output of that layer: || got - want || / || want || <= layer_tol per row.  One layer adds a
        handful of bf16 roundings (measured 0.002-0.004); a missing or wrong term of any layer is an order of magnitude more.
      * end to end, the residual stream after the last layer: relative error <= hidden_tol per row.  bf16 rounding noise is
        amplified from layer to layer (an activation that rounds the other way moves its element by 0.4-0.8 %), so after 16
        layers two correct implementations sit 0.025-0.03 apart; the bound is 1.5 times that.
      * float32 logits: | got - want | <= logit_atol + 0.03 |want| for every entry of the vocabulary (the error of a logit
        is the error of the final hidden row times an unembedding column: normal with sigma ~0.024 at 16 layers, and the
        largest of 1.6 million entries lies near 5 sigma), mean < 0.025;
      * the greedy token agrees wherever the oracle's two best logits are further apart than twice the bound.
    ``without``: a function that takes a term out of the weights (say, zeroes xsa_alpha).  The layer-by-layer check is then
    repeated with it and must fail: the control that shows the bound notices that term."""
    from lyra_amd.model import init_cache, init_weights, model_apply
    from lyra_amd.nn.quant import QArray, quantize

    dev = U.dev()
    w = init_weights(cfg, dev, seed=3)
    bias_gen = torch.Generator(device=dev)
    bias_gen.manual_seed(77)
    for lw in w.layers:
        if getattr(lw.mlp, "router_bias", None) is not None:
            lw.mlp.router_bias.copy_(torch.randn(lw.mlp.router_bias.shape, device=dev, generator=bias_gen))
    cache = init_cache(cfg, B, S, dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2024)
    for layer in cache.layers:
        for name in ("k", "v"):
            hist = torch.randn(B, cfg.n_kv_heads, start, cfg.head_dim, device=dev, generator=gen).to(torch.bfloat16)
            dst = getattr(layer, name)
            if isinstance(dst, QArray):
                q = quantize(hist, dst.dtype, dst.block)
                dst.qval.view(torch.uint8)[:, :, :start] = q.qval.view(torch.uint8)
                dst.scale[:, :, :start] = q.scale
            else:
                dst[:, :, :start] = hist
    cache.pos.fill_(start)
    wn = D.weights_to_numpy(w, cfg)
    cn = D.cache_to_numpy(cache)
    tokens = np.random.default_rng(5).integers(0, cfg.vocab_size, (steps, B))
    clear = np.ones(B, bool)  # rows whose routing was unambiguous in every step so far (the cache carries a flip forward)
    for s in range(steps):
        print(f"full-width {cfg.name} step {s} pos {start + s}", file=sys.stderr, flush=True)
        hidden = []
        got, _ = model_apply(torch.from_numpy(tokens[s]).to(dev), w, cache, cfg, hidden_out=hidden)
        torch.cuda.synchronize()
        margins, want_hidden = [], []
        want = D.decode_step(tokens[s], wn, cn, start + s, cfg, use_c=True, router_margins=margins, hidden_out=want_hidden,
                             inner="fp32")
        assert len(margins) == moe_layers
        clear &= np.min(np.stack(margins), axis=0) > margin
        print("router margins (min over layers):", np.min(np.stack(margins), axis=0), file=sys.stderr, flush=True)
        assert clear.sum() >= min_clear, f"too few rows with unambiguous routing: {clear}"
        print(f"step {s}: {int(clear.sum())} of {B} rows compared ({B - int(clear.sum())} left out for a routing margin <= {margin}; "
              f"at least {min_clear} required)", file=sys.stderr, flush=True)
        if s == 0:
            worst = _layer_by_layer(cfg, w, cache, start, want_hidden, margins, margin)
            print(f"layer by layer: worst relative error of a layer output {worst:.5f} (bound {layer_tol})", file=sys.stderr, flush=True)
            assert worst <= layer_tol
            if without is not None:
                undo = without(w)
                broken = _layer_by_layer(cfg, w, cache, start, want_hidden, margins, margin)
                undo()
                print(f"layer by layer with the term taken out: {broken:.5f}", file=sys.stderr, flush=True)
                assert broken > 2 * layer_tol, "the bound would not notice the term"
                _layer_by_layer(cfg, w, cache, start, want_hidden, margins, margin)  # leaves the cache rows as they were
        hg, hw = U.to_np(hidden[0]), want_hidden[-1]
        rel = np.linalg.norm(hg - hw, axis=-1) / np.linalg.norm(hw, axis=-1)
        print(f"residual stream, relative error per row: max {rel[clear].max():.4f} (bound {hidden_tol})", file=sys.stderr, flush=True)
        assert (rel[clear] <= hidden_tol).all(), rel
        g, t = U.to_np(got)[:, : cfg.vocab_size], want[:, : cfg.vocab_size]
        assert np.isneginf(U.to_np(got)[:, cfg.vocab_size :]).all() and np.isfinite(g).all()
        err = np.abs(g[clear] - t[clear])
        print(f"logits: max err {err.max():.4f}, mean {err.mean():.5f}", file=sys.stderr, flush=True)
        U.assert_close(g[clear], t[clear], atol=logit_atol, rtol=0.03, what=f"{cfg.name} step {s}")
        assert err.mean() < 0.025
        top2 = np.sort(t[clear], axis=-1)[:, -2:]
        decided = (top2[:, 1] - top2[:, 0]) > 2 * (logit_atol + 0.03 * np.abs(top2[:, 1]))
        assert (g[clear].argmax(-1) == t[clear].argmax(-1))[decided].all()
    assert int(cache.pos.item()) == start + steps


def test_config2_lyra_small_b8_ctx4096_decode_steps_match_oracle():
    """Benchmark configuration 2 at its literal size: the full lyra-small decode step (16 layers alternating window 128 and
    global, C=2048, 16Q/4KV heads of 128, 15+1 experts, vocabulary 204800), B=8, a cache of 4096 rows with 4094 of them
    history, FP8 cache with per-row scales, FP8 weights with one scale per output channel; two steps, the second one
    writing the last row of the cache."""
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides

    cfg = apply_inference_overrides(replace(MODEL_VARIANTS["lyra-small"], implementation="pallas"), fp8=True, fp8_attn=True,
                                    per_channel=True)
    _full_width_parity(cfg, B=8, S=4096, start=4094, steps=2, min_clear=6, moe_layers=4, hidden_tol=0.045)


def test_reference_serve_path_blocks_256_bf16_attention_weights():
    """What the reference's `--fp8` serve path sets (lyra/generate.py:31-38): FP8 cache and FP8 MLP / expert weights with the
    default (256, 256) scale blocks, attention projections left in bf16.  lyra-small widths, 4 layers (one of them MoE)."""
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, interleaved_moe

    cfg = replace(MODEL_VARIANTS["lyra-small"], implementation="pallas", n_layers=4, mlp_map=interleaved_moe(layers=4, every=4, first=4),
                  vocab_size=8000, padded_vocab_size=8192)
    cfg = apply_inference_overrides(cfg, fp8=True)
    assert cfg.quantize_mlp and cfg.quantize_cache and not cfg.quantize_attn and not cfg.per_channel_scales
    _full_width_parity(cfg, B=16, S=1024, start=700, steps=2, min_clear=12, moe_layers=1, hidden_tol=0.02)


@pytest.mark.parametrize("S,start", [(1024, 900), (64, 2)])
def test_width_4096_step_with_exclusive_self_attention_63_experts_b128(S, start):
    """The widths of lyra-max (C=4096, 32Q/8KV heads of 128, dense hidden 8192, 63 routed + 1 shared experts of hidden 4096,
    learned exclusive self attention with non-zero alpha, output gate) at B=128 on two layers - one dense, one MoE - with a
    small vocabulary: the fused driver path of benchmark configuration 5 against the CPU restatement.  With a long history
    the new token's own value row is a small part of the attention output; with two cached tokens it is a large part, and
    there the check must fail when alpha is zeroed."""
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides

    cfg = replace(MODEL_VARIANTS["lyra-max"], implementation="pallas", n_layers=2, mlp_map=("dense", "moe"), vocab_size=4000,
                  padded_vocab_size=4096)
    assert cfg.use_learned_xsa and cfg.n_routed_experts == 63
    cfg = apply_inference_overrides(cfg, fp8=True, fp8_attn=True, per_channel=True)

    def without_xsa(w):
        kept = [lw.attn.xsa_alpha for lw in w.layers]
        assert all(float(a.abs().min()) > 0 for a in kept)
        for lw in w.layers:
            lw.attn.xsa_alpha = torch.zeros_like(lw.attn.xsa_alpha)

        def undo():
            for lw, a in zip(w.layers, kept):
                lw.attn.xsa_alpha = a
        return undo

    _full_width_parity(cfg, B=128, S=S, start=start, steps=2, min_clear=96, moe_layers=1, hidden_tol=0.03,
                       without=without_xsa if start < 10 else None)


def test_graphed_decoder_samples_inside_the_graph():
    """Temperature / top-k sampling recorded into the HIP graph: every replay draws fresh uniform numbers, every drawn
    token is one of the row's 4 largest logits, and replays on identical inputs do not all draw the same tokens."""
    from lyra_amd.generate import GraphedDecoder
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights

    cfg = apply_inference_overrides(replace(MODEL_VARIANTS["dev"], implementation="pallas", sample_topk=4, sample_temperature=0.8),
                                    fp8=True, fp8_attn=True, per_channel=True)
    dev = U.dev()
    w = init_weights(cfg, dev, seed=3)
    cache = init_cache(cfg, 8, 256, dev)
    cache.pos.fill_(9)
    dec = GraphedDecoder(w, cache, cfg, batch=8, greedy=False)
    dec.tokens.copy_(torch.arange(8, device=dev) + 3)
    draws = []
    for _ in range(12):
        cache.pos.fill_(9)
        dec.tokens.copy_(torch.arange(8, device=dev) + 3)
        nxt = dec.step()
        torch.cuda.synchronize()
        top4 = torch.topk(dec.logits[:, : cfg.vocab_size], 4, dim=-1).indices
        assert (nxt.long()[:, None] == top4).any(-1).all()
        draws.append(U.to_np(nxt).copy())
    assert len({d.tobytes() for d in draws}) > 1


@pytest.mark.parametrize("fp8", [False, True])
def test_gpt_oss_like_variant_width_not_a_multiple_of_128_with_biases(fp8):
    """The options of gpt-oss-20b (lyra/variants.py:62-80: biases on q/k/v, the output projection and the MLPs, no shared
    expert, no QK norm, YaRN tables) at a width that is not a multiple of 128 (320; gpt-oss-20b's is 2880): the fused driver
    takes such a model too - its matmuls through the general kernel, the biases the reference adds to a bf16 result added
    the same way - and must match the oracle step by step, match the plain-operator driver, and replay from a HIP graph."""
    from lyra_amd.generate import GraphedDecoder
    from lyra_amd.model import MODEL_VARIANTS, _fused_supported, apply_inference_overrides, init_cache, init_weights, model_apply

    cfg = replace(MODEL_VARIANTS["dev"], implementation="pallas", n_embd=320, n_attn_heads=4, n_kv_heads=2, seq_len=128,
                  sliding_window=32, use_qk_norm=False, use_qkv_bias=True, use_attn_out_bias=True, use_mlp_bias=True,
                  n_shared_experts=0, n_active_experts=2, rope_scale=4.0, mlp_map=("moe", "dense", "moe", "moe"),
                  sample_temperature=0.0)
    if fp8:
        cfg = apply_inference_overrides(cfg, fp8=True, fp8_attn=True, per_channel=True)
    dev = U.dev()
    assert _fused_supported(init_weights(cfg, dev, seed=3), cfg)
    _run_steps(cfg, B=5, S=128, steps=3, start=40)

    # fused driver against the plain-operator driver on the same weights and history (both on the HIP operators)
    w = init_weights(cfg, dev, seed=3)
    tok = torch.tensor([3, 900, 17, 5, 4], device=dev)
    outs = []
    for fused in (True, False):
        c = replace(cfg, fused_glue=fused)
        cache = init_cache(c, 5, 128, dev)
        cache.pos.fill_(0)
        steps, t = [], tok
        for _ in range(3):
            logits, _ = model_apply(t, w, cache, c)
            steps.append(U.to_np(logits[:, : cfg.vocab_size]))
            t = logits.argmax(-1)
        outs.append(steps)
    for a, b in zip(*outs):
        U.assert_close(a, b, atol=3e-2, rtol=2e-2, what="fused vs plain-operator logits")

    # ... and the captured step chains tokens like the eager one
    cache = init_cache(cfg, 5, 128, dev)
    cache.pos.fill_(0)
    dec = GraphedDecoder(w, cache, cfg, batch=5)
    dec.tokens.copy_(tok.to(torch.int32))
    got = dec.decode(3)
    torch.cuda.synchronize()
    assert got.shape == (3, 5) and int(cache.pos.item()) == 3
    assert torch.equal(got[0].cpu(), torch.from_numpy(outs[0][0].argmax(-1)).to(torch.int32))


def test_width_2880_step_of_gpt_oss_20b_with_biases_32_experts_b64():
    """The widths and options of gpt-oss-20b (lyra/variants.py:62-80: C=2880, 64Q/8KV heads of 64, 32 routed experts of
    hidden 2880 and no shared one, 4 per token, biases on every projection, no QK norm, YaRN tables) at B=64 on two layers
    with a small vocabulary: every projection width but q/k/v's is 22.5 spans of 128 columns.  The fused driver against the
    CPU restatement, layer by layer and end to end."""
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides

    cfg = replace(MODEL_VARIANTS["gpt-oss-20b"], implementation="pallas", n_layers=2, mlp_map=("moe", "moe"), vocab_size=4000,
                  padded_vocab_size=4096, seq_len=1024)
    assert cfg.n_embd == 2880 and cfg.expert_hidden == 2880 and cfg.use_qkv_bias and cfg.use_mlp_bias and cfg.n_shared_experts == 0
    cfg = apply_inference_overrides(cfg, fp8=True, fp8_attn=True, per_channel=True)
    _full_width_parity(cfg, B=64, S=1024, start=700, steps=2, min_clear=40, moe_layers=2, hidden_tol=0.03)


def test_config5_lyra_max_full_depth_b128_ctx4096():
    """Benchmark configuration 5 at its literal size: lyra-max, 32 layers (2 dense + 30 MoE with 63 + 1 experts), width 4096,
    B=128, a cache of 4096 rows, FP8 weights and cache (about 135 GB resident).  Two eager steps and the same two steps
    replayed from a captured graph: finite logits, the same tokens, bit-identical appended cache rows; and the first two
    and last two layers, each run on the residual stream the GPU itself had at that layer's input, against the CPU
    restatement of that layer (teacher forced, so the CPU side stays at four layers)."""
    import time

    from lyra_amd import model as M
    from lyra_amd.generate import GraphedDecoder, generate
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.model import MODEL_VARIANTS, ModelWeights, apply_inference_overrides, init_cache, init_weights
    from lyra_amd.nn.quant import QArray

    dev = U.dev()
    free, _ = torch.cuda.mem_get_info()
    if free < 170e9:
        pytest.skip(f"needs ~150 GB of free device memory, {free / 1e9:.0f} GB are free")
    B, S, start, n = 128, 4096, 4094, 2
    cfg = apply_inference_overrides(replace(MODEL_VARIANTS["lyra-max"], implementation="pallas", sample_temperature=0.0), fp8=True,
                                    fp8_attn=True, per_channel=True)
    assert cfg.n_layers == 32 and cfg.n_routed_experts == 63 and cfg.use_learned_xsa
    t0 = time.perf_counter()
    w = init_weights(cfg, dev, seed=3)
    bias_gen = torch.Generator(device=dev)
    bias_gen.manual_seed(77)
    for lw in w.layers:  # (spread the router logits: random-init ones lie within bf16 noise of each other)
        if getattr(lw.mlp, "router_bias", None) is not None:
            lw.mlp.router_bias.copy_(torch.randn(lw.mlp.router_bias.shape, device=dev, generator=bias_gen))
    cache = init_cache(cfg, B, S, dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1005)
    for layer in cache.layers:  # history: random finite FP8 codes with scales of N(0,1) rows
        for arr in (layer.k, layer.v):
            codes = torch.randint(0, 0x78, arr.qval.shape, generator=gen, device=dev, dtype=torch.uint8)
            signs = torch.randint(0, 2, arr.qval.shape, generator=gen, device=dev, dtype=torch.uint8) << 7
            arr.qval.view(torch.uint8).copy_(codes | signs)
            arr.scale.copy_(torch.rand(arr.scale.shape, generator=gen, device=dev) * 0.004 + 0.006)
    torch.cuda.synchronize()
    print(f"config 5: model and caches built in {time.perf_counter() - t0:.0f} s", file=sys.stderr, flush=True)
    first = torch.randint(0, cfg.vocab_size, (B,), generator=gen, device=dev, dtype=torch.int32)

    def appended():
        rows = []
        for layer in cache.layers:
            for arr in (layer.k, layer.v):
                rows.append(arr.qval.view(torch.uint8)[:, :, start : start + n].clone())
                rows.append(arr.scale[:, :, start : start + n].clone())
        return rows

    # ---- eager ----
    cache.pos.fill_(start)
    tok, eager_tokens = first, []
    for s_ in range(n):
        print(f"config 5: eager step {s_}", file=sys.stderr, flush=True)
        logits, _ = M.model_apply(tok, w, cache, cfg)
        assert torch.isfinite(logits[:, : cfg.vocab_size]).all() and torch.isneginf(logits[:, cfg.vocab_size :]).all()
        tok = F.argmax(logits, cfg.vocab_size)
        eager_tokens.append(tok.clone())
    torch.cuda.synchronize()
    assert int(cache.pos.item()) == start + n
    eager_rows = appended()
    # ---- the same two steps from a captured graph ----
    cache.pos.fill_(start)
    dec = GraphedDecoder(w, cache, cfg, batch=B)
    dec.tokens.copy_(first)
    t1 = time.perf_counter()
    drawn = dec.decode(n)
    torch.cuda.synchronize()
    print(f"config 5: {n} graph replays in {(time.perf_counter() - t1) * 1e3:.1f} ms", file=sys.stderr, flush=True)
    assert int(cache.pos.item()) == start + n
    for s_ in range(n):
        assert torch.equal(drawn[s_], eager_tokens[s_]), f"tokens of step {s_} differ between the graph and eager calls"
    for a, b in zip(appended(), eager_rows):
        assert torch.equal(a, b), "appended cache rows differ between the graph and eager calls"
    del dec
    # ---- layers 0, 1, 30, 31 on the GPU's own inputs against the CPU restatement of the layer ----
    pos = torch.tensor(start, dtype=torch.int32, device=dev)
    cos_t, sin_t = M._rope_tables(cfg, dev)
    ones = torch.ones(cfg.n_embd, dtype=torch.float32, device=dev)
    h = w.emb[first.long()]
    inputs, outputs = {}, {}
    check = (0, 1, cfg.n_layers - 2, cfg.n_layers - 1)
    for idx, layer in enumerate(w.layers):
        if idx in check:
            inputs[idx] = U.to_np(h)
        h, _ = M.attention_apply_fused(h, layer.attn, idx, pos, cos_t, sin_t, cache.layers[idx], cfg)
        h = M.moe_apply_fused(h, layer.mlp, cfg) if isinstance(layer.mlp, M.MoEWeights) else M.dense_mlp_apply_fused(h, layer.mlp, cfg)
        if isinstance(h, (F.Unsummed, F.Uncombined)):
            h = F.rmsnorm_proj(h, ones, cfg.norm_eps)[2]
        if idx in check:
            outputs[idx] = U.to_np(h)
    torch.cuda.synchronize()
    for idx in check:
        t2 = time.perf_counter()
        one_layer = ModelWeights(emb=torch.zeros(1, 8, device=dev), unemb_t=torch.zeros(1, cfg.n_embd, 8, dtype=torch.bfloat16, device=dev),
                                 norm_scale=ones, layers=[w.layers[idx]])
        wn = D.weights_to_numpy(one_layer, cfg)
        wn["emb"] = inputs[idx]
        lc = cache.layers[idx]
        cn = {"k": [(lc.k.qval.view(torch.uint8).cpu().numpy(), lc.k.scale.float().cpu().numpy())],
              "v": [(lc.v.qval.view(torch.uint8).cpu().numpy(), lc.v.scale.float().cpu().numpy())]}
        cfg1 = replace(cfg, vocab_size=8, padded_vocab_size=8)  # (the residual scales depend on the depth: all 32 layers stay configured)
        margins, hidden = [], []
        D.decode_step(np.arange(B), wn, cn, start, cfg1, use_c=True, router_margins=margins, hidden_out=hidden, inner="fp32",
                      layer_offset=idx)
        want, got = hidden[-1], outputs[idx]
        ok = np.ones(B, bool) if not margins else margins[0] > 0.03
        assert ok.sum() >= 96, f"layer {idx}: too few rows with unambiguous routing"
        rel = np.linalg.norm(got - want, axis=-1) / np.linalg.norm(want, axis=-1)
        print(f"config 5: layer {idx} ({cfg.mlp_map[idx]}): worst relative error {rel[ok].max():.5f} over {ok.sum()} rows, "
              f"CPU side {time.perf_counter() - t2:.0f} s", file=sys.stderr, flush=True)
        assert rel[ok].max() <= 0.01, f"layer {idx}: {rel[ok].max()}"
        del wn, cn
