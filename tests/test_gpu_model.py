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


def _run_steps(cfg, B, S, steps, start):
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
        want = D.decode_step(tokens[s], wn, cn, start + s, cfg)
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
                np.testing.assert_allclose(O.fp8_e4m3fn_decode(kq) * ks, O.fp8_e4m3fn_decode(oq) * osc, atol=0.08, rtol=0.08)
                if l == 0:
                    assert (kq == oq).mean() > 0.8  # the rest sits one FP8 step away (checked by value above)
    assert int(cache.pos.item()) == start + steps


@pytest.mark.parametrize("fp8", [False, True])
def test_dev_model_decode_steps_match_oracle(fp8):
    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides

    cfg = MODEL_VARIANTS["dev"]
    cfg = replace(cfg, sliding_window=128, use_sdpa_output_gate=True, seq_len=512, implementation="pallas")
    if fp8:
        cfg = apply_inference_overrides(cfg, fp8=True, fp8_attn=True)
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
        nxt = dec.step()
        torch.cuda.synchronize()
        assert torch.equal(dec.logits[:, : cfg.vocab_size], eager[:, : cfg.vocab_size])
        assert torch.equal(nxt.long(), eager.argmax(-1))
