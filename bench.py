"""Headline benchmark: decode tokens/s of a full lyra-small decode step at B=64, context 4096, FP8 KV cache and
FP8 weights on one MI355X, with the roofline of the dominant kernel (FP8 decode attention, global layer) and the
CPU restatement of the reference's decode path timed on the same machine.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--ctx 4096] [--no-cpu-baseline]

Prints ONE JSON line.  A "step" is one decode step of the whole model (16 layers + LM head) for all B sequences
with every sequence at context 4096 (the newest token is written at index 4095 and attends to all 4096 keys);
inputs (weights, KV caches) are resident in HBM before the timed region.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
os.environ.setdefault("LYRA_LOG_KERNELS", "0")

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def attention_algorithmic_bytes(batch, kv_heads, visible, head_dim, fp8=True):
    """Bytes a decode-attention launch must read: K and V rows of every visible key (+ one f32 scale per row)."""
    per_row = head_dim * (1 if fp8 else 2) + (4 if fp8 else 0)
    return 2 * batch * kv_heads * visible * per_row


def build_model(batch, ctx, device, variant="lyra-small", layout="headline", weights=None):
    """Random-init weights of the variant (or ``weights``, to run them at another batch) and caches with a synthetic history."""
    import torch

    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights
    from lyra_amd.nn.quant import QArray

    if layout == "reference-fp8":  # what the reference's serve path sets with --fp8 (generate.py:31-38), nothing more
        cfg = apply_inference_overrides(MODEL_VARIANTS[variant], fp8=True)
    else:
        cfg = apply_inference_overrides(MODEL_VARIANTS[variant], fp8=True, fp8_attn=True, per_channel=True)
    weights = init_weights(cfg, device) if weights is None else weights
    cache = init_cache(cfg, batch, ctx, device)
    g = torch.Generator(device=device)
    g.manual_seed(1002)
    for layer in cache.layers:  # synthetic history: random FP8 codes (finite) and scales ~ amax(N(0,1) row) / 448
        for arr in (layer.k, layer.v):
            assert isinstance(arr, QArray)
            codes = torch.randint(0, 0x7F, arr.qval.shape, generator=g, device=device, dtype=torch.uint8)
            signs = torch.randint(0, 2, arr.qval.shape, generator=g, device=device, dtype=torch.uint8) << 7
            arr.qval.view(torch.uint8).copy_(codes | signs)
            arr.scale.copy_(torch.rand(arr.scale.shape, generator=g, device=device) * 0.004 + 0.006)
    cache.pos.fill_(ctx - 1)
    return cfg, weights, cache


def time_decode_steps(cfg, weights, cache, batch, ctx, steps, warmup, greedy=False):
    """Wall time of `steps` replays of the captured decode step; also returns the function that runs one more step.
    ``greedy`` False: the reference's default sampler (temperature 0.8, top-k 4: lyra/model.py:107-108, generate.py:46-53)
    through lyra_sample_topk, the uniform numbers drawn inside the captured step; True: arg-max through lyra_argmax."""
    import torch

    from lyra_amd.generate import GraphedDecoder

    # every timed step runs at full context: the captured step does not move the position (ctx - 1, the last cache row);
    # each step decodes the tokens the step before it drew
    dec = GraphedDecoder(weights, cache, cfg, batch, greedy=greedy, advance=False)
    dec.tokens.copy_(torch.randint(0, cfg.vocab_size, (batch,), device=dec.tokens.device).to(torch.int32))
    one_step = dec.step

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert torch.isfinite(dec.logits[:, : cfg.vocab_size]).all(), "non-finite logits"
    return elapsed, one_step


def time_dominant_kernel(cfg, weights, cache, batch, ctx, one_step, rounds=13, front=False):
    """Average duration of the FP8 global-layer decode-attention launch through the C ABI, HIP events on the launch
    stream.  The launches come as they do in the workload: one per global layer of the model (each on that layer's
    cache, so every launch streams from HBM), timed as a group, with a replay of the whole decode step between groups.
    (A hundred launches back to back measure something else: at 6 TB/s the device reaches its power limit within
    milliseconds and the launch time climbs from 44 to 54 us.)
    ``front``: the launch the decode step itself uses, which also does the step in front of the attention (QK norm,
    rotary embedding, cache append: lyra_decode_attention_qkv) from the unsummed slices of the q/k/v projection."""
    import torch

    from lyra_amd import _lib
    from lyra_amd.model import _rope_tables

    dev = weights.emb.device
    L = _lib.lib
    N, K, H = cfg.n_attn_heads, cfg.n_kv_heads, cfg.head_dim
    q = torch.randn(batch, N, H, device=dev, dtype=torch.bfloat16)
    out = torch.empty_like(q)
    pos = torch.full((1,), ctx - 1, dtype=torch.int32, device=dev)
    layers = [c for i, c in enumerate(cache.layers) if i % 2 == 1]
    attn_w = weights.layers[1].attn
    sinks = attn_w.sinks
    need = L.lyra_decode_attention_workspace(batch, N, K, ctx, H, 0)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)
    if front:
        width = (N + 2 * K) * H
        splits = max(1, L.lyra_decode_gemm_splits(batch, cfg.n_embd, width, cfg.n_embd))
        part = torch.randn(splits, batch, width, device=dev) * 0.5
        cos_t, sin_t = _rope_tables(cfg, dev)
        qn, kn = attn_w.qnorm_scale, attn_w.knorm_scale

    def launch(c):
        if front:
            rc = L.lyra_decode_attention_qkv(
                None, part.data_ptr(), splits, qn.data_ptr() if qn is not None else None, kn.data_ptr() if kn is not None else None,
                cos_t.data_ptr(), sin_t.data_ptr(), cos_t.shape[0], cfg.norm_eps, c.k.qval.data_ptr(), c.v.qval.data_ptr(),
                c.k.scale.data_ptr(), c.v.scale.data_ptr(), sinks.data_ptr(), pos.data_ptr(), 0, None, out.data_ptr(), ws.data_ptr(),
                ws.numel(), batch, N, K, ctx, H, H**-0.5, 0, _lib.DTYPE_E4M3FN, _lib.DTYPE_BF16, stream.cuda_stream)
            _lib.check(rc, "lyra_decode_attention_qkv")
            return
        rc = L.lyra_decode_attention(
            q.data_ptr(), c.k.qval.data_ptr(), c.v.qval.data_ptr(), c.k.scale.data_ptr(), c.v.scale.data_ptr(), sinks.data_ptr(),
            pos.data_ptr(), 0, None, out.data_ptr(), ws.data_ptr(), ws.numel(), batch, N, K, ctx, H, H**-0.5, 0,
            _lib.DTYPE_E4M3FN, _lib.DTYPE_BF16, stream.cuda_stream)
        _lib.check(rc, "lyra_decode_attention")

    pairs = []
    for r in range(rounds + 2):  # the first two groups warm up
        one_step()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for c in layers:
            launch(c)
        stop.record(stream)
        if r >= 2:
            pairs.append((start, stop))
    stream.synchronize()
    return sum(a.elapsed_time(b) for a, b in pairs) * 1e-3 / (len(pairs) * len(layers))  # seconds per launch


def time_attention_sustained(cfg, weights, cache, batch, ctx, launches=104, warm=16):
    """The launch of `time_dominant_kernel(front=True)` (or the plain one when the step does not use the front step) back
    to back: `launches` launches in one HIP-event bracket, rotating over the caches of the model's global layers (8 x 277 MB
    at the headline shape: every launch streams from HBM).  Under this sustained load the device reaches its power limit
    within milliseconds, which the groups of 8 between step replays do not."""
    import torch

    from lyra_amd import _lib

    dev = weights.emb.device
    L = _lib.lib
    N, K, H = cfg.n_attn_heads, cfg.n_kv_heads, cfg.head_dim
    q = torch.randn(batch, N, H, device=dev, dtype=torch.bfloat16)
    out = torch.empty_like(q)
    pos = torch.full((1,), ctx - 1, dtype=torch.int32, device=dev)
    layers = [c for i, c in enumerate(cache.layers) if i % 2 == 1]
    sinks = weights.layers[1].attn.sinks
    ws = torch.zeros(max(L.lyra_decode_attention_workspace(batch, N, K, ctx, H, 0), 256), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)

    def launch(i):
        c = layers[i % len(layers)]
        rc = L.lyra_decode_attention(
            q.data_ptr(), c.k.qval.data_ptr(), c.v.qval.data_ptr(), c.k.scale.data_ptr(), c.v.scale.data_ptr(), sinks.data_ptr(),
            pos.data_ptr(), 0, None, out.data_ptr(), ws.data_ptr(), ws.numel(), batch, N, K, ctx, H, H**-0.5, 0,
            _lib.DTYPE_E4M3FN, _lib.DTYPE_BF16, stream.cuda_stream)
        _lib.check(rc, "lyra_decode_attention")

    return _time_launches(launch, stream, warm=warm, iters=launches), launches


def time_attention_ragged(dev, one_step, stream, rounds=10):
    """Benchmark configuration 4: gpt-oss attention shape (64 query / 8 kv heads of width 64), B=64, cache 4096, FP8, one
    length per row drawn uniformly from [256, 4096] (seeded), global layer, the rows ranked once by lyra_attention_rank as a
    decode step would do for all its layers.  Timed like the other stand-alone launches: groups (one launch per cache set,
    3 sets) between replays of the decode step."""
    import numpy as np
    import torch

    from lyra_amd import _lib

    L = _lib.lib
    B, N, K, H, S = 64, 64, 8, 64, 4096
    gen = torch.Generator(device=dev)
    gen.manual_seed(1004)
    lengths = np.random.default_rng(1004).integers(256, 4097, size=B)
    sets = []
    for _ in range(3):
        kv = [torch.randint(0, 0x78, (B, K, S, H), generator=gen, device=dev, dtype=torch.uint8) for _ in range(2)]
        sc = [torch.rand(B, K, S, generator=gen, device=dev) * 0.004 + 0.006 for _ in range(2)]
        sets.append((kv, sc))
    q = torch.randn(B, N, H, generator=gen, device=dev, dtype=torch.bfloat16)
    out = torch.empty_like(q)
    sinks = torch.randn(N, generator=gen, device=dev)
    pos = torch.from_numpy(lengths.astype(np.int32) - 1).to(dev)
    order = torch.empty(B, dtype=torch.int32, device=dev)
    _lib.check(L.lyra_attention_rank(pos.data_ptr(), B, order.data_ptr(), stream.cuda_stream), "lyra_attention_rank")
    ws = torch.zeros(max(L.lyra_decode_attention_workspace(B, N, K, S, H, 0), 256), dtype=torch.uint8, device=dev)

    def launch(kv, sc):
        rc = L.lyra_decode_attention_ranked(
            q.data_ptr(), kv[0].data_ptr(), kv[1].data_ptr(), sc[0].data_ptr(), sc[1].data_ptr(), sinks.data_ptr(), pos.data_ptr(), 1,
            order.data_ptr(), None, out.data_ptr(), ws.data_ptr(), ws.numel(), B, N, K, S, H, H**-0.5, 0, _lib.DTYPE_E4M3FN,
            _lib.DTYPE_BF16, stream.cuda_stream)
        _lib.check(rc, "lyra_decode_attention_ranked")

    pairs = []
    for r in range(rounds + 2):
        one_step()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for kv, sc in sets:
            launch(kv, sc)
        b.record(stream)
        if r >= 2:
            pairs.append((a, b))
    stream.synchronize()
    t = sum(a.elapsed_time(b) for a, b in pairs) * 1e-3 / (len(pairs) * len(sets))
    nbytes = int(2 * K * lengths.sum() * (H + 4))
    return {"kernel": "decode_attention_kernel<64, fp8, 8 wavefronts> (rows dealt out by lyra_attention_rank's order)",
            "case": "gpt-oss attention shape, B=64, 64Q/8KV, H=64, cache 4096, lengths U[256, 4096] (seed 1004), global layer",
            "bound": "hbm", "achieved": nbytes / t / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / t / 1e9 / HBM_PEAK_GBS,
            "algorithmic_bytes": nbytes, "us_per_launch": t * 1e6}


def source_fingerprint():
    """Hash of the attention kernel's sources: hardware-counter figures kept in profiles/ are only quoted for the sources
    they were collected on."""
    import hashlib

    h = hashlib.sha256()
    for rel in ("lyra_amd/csrc/decode_attention.hip", "lyra_amd/csrc/lyra_device.h"):
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _nbytes(w):
    """Bytes of a weight array as the kernels read it (codes + scales for a quantised array)."""
    from lyra_amd.nn.quant import QArray

    if isinstance(w, QArray):
        return w.qval.numel() * w.qval.element_size() + w.scale.numel() * w.scale.element_size()
    return w.numel() * w.element_size()


def step_algorithmic_bytes(cfg, weights, batch, ctx, touched_per_moe_layer):
    """Bytes one decode step has to read at the least: visible K/V rows (+ scales) of every layer, every projection and
    dense MLP weight once, the weights of the experts that have rows (counted from the step's own routing), the LM head.
    Activations, norms' small parameters and the embedding rows are left out (a few MB)."""
    from lyra_amd.model import MoEWeights

    total, moe = 0, 0
    for idx, layer in enumerate(weights.layers):
        visible = min(cfg.sliding_window, ctx) if (idx % 2 == 0 and cfg.sliding_window > 0) else ctx
        total += attention_algorithmic_bytes(batch, cfg.n_kv_heads, visible, cfg.head_dim, fp8=cfg.quantize_cache)
        total += _nbytes(layer.attn.qkv) + _nbytes(layer.attn.out)
        if isinstance(layer.mlp, MoEWeights):
            per_expert = (_nbytes(layer.mlp.mlp_up) + _nbytes(layer.mlp.mlp_down)) // cfg.n_experts
            total += per_expert * touched_per_moe_layer[moe]
            moe += 1
        else:
            total += _nbytes(layer.mlp.mlp_up) + _nbytes(layer.mlp.mlp_down)
    return total + _nbytes(weights.unemb_t)


def time_expert_matmuls(dev, one_step, stream, rounds=10):
    """The expert matmuls through the C ABI, HIP events on the launch stream, between replays of the decode step (as the
    attention launch is timed): the up projection with fused SwiGLU and the down projection at the shape of a
    lyra-medium MoE layer (benchmark configuration 3: width 4096, 31 routed + 1 shared experts of hidden 4096, 64 tokens,
    3 routed experts per token drawn from Zipf(1.1) + the shared one, seeded) and at the shape of the lyra-small layer the
    step itself runs (15 + 1 experts, width 2048, hidden 2048).  FP8 weights, one scale per output channel.  The group
    sizes are the instances `--kernels` times as "lyra-medium expert ... T=64" and "lyra-small expert ... B=64".  The launches
    are the decode step's: lyra_decode_gemm_ex with the activations in tiles of 16 rows x 32 columns, as the norm in front
    of the up projection and the up projection itself leave them (LYRA_LHS_TILED16 / LYRA_OUT_TILED16)."""
    import numpy as np
    import torch

    from lyra_amd import _lib

    L = _lib.lib
    gen = torch.Generator(device=dev)
    gen.manual_seed(1003)
    out_rows = []
    routing = benchmark_routing()
    for label, E, C, Hd, sizes in (("lyra-medium", 32, 4096, 4096, routing["medium_T64"]), ("lyra-small", 16, 2048, 2048, routing["small_B64"])):
        M, touched = int(sizes.sum()), int((sizes > 0).sum())
        gs = torch.from_numpy(sizes).to(dev)
        x = torch.randn(M, C, generator=gen, device=dev, dtype=torch.bfloat16)
        cases = []
        for name, K, N, swiglu in (("up+SwiGLU", C, 2 * Hd, True), ("down", Hd, C, False)):
            # enough weight sets that a group of launches never finds its weights in the 256 MB last-level cache
            n_sets = min(4, max(2, -(-600_000_000 // (E * K * N))))
            ws_sets = [torch.randint(0, 0x78, (E, K, N), generator=gen, device=dev, dtype=torch.uint8) for _ in range(n_sets)]
            sc = torch.rand(E, 1, N, generator=gen, device=dev) * 0.001 + 0.0005
            # (random values: the tiled layout is a permutation of the same bytes, rows rounded up to 16)
            lhs = torch.randn((M + 15) // 16 * 16, K, generator=gen, device=dev, dtype=torch.bfloat16)
            out = torch.empty((M + 15) // 16 * 16, N // 2 if swiglu else N, device=dev, dtype=torch.bfloat16)
            ws = torch.zeros(max(L.lyra_decode_gemm_workspace(M, E, K, N, int(swiglu)), 256), dtype=torch.uint8, device=dev)
            nbytes = touched * (K * N + N * 4) + M * K * 2 + M * (N // 2 if swiglu else N) * 2
            flags = _lib.LHS_TILED16 | (_lib.OUT_TILED16 if swiglu else 0)

            def launch(i, lhs=lhs, ws_sets=ws_sets, sc=sc, out=out, ws=ws, K=K, N=N, swiglu=swiglu, flags=flags):
                w = ws_sets[i % len(ws_sets)]
                rc = L.lyra_decode_gemm_ex(lhs.data_ptr(), None, w.data_ptr(), sc.data_ptr(), K, 1, gs.data_ptr(), None, None, 1.0, 0,
                                           out.data_ptr(), ws.data_ptr(), ws.numel(), M, E, K, N, _lib.DTYPE_E4M3FN | flags,
                                           _lib.DTYPE_BF16, int(swiglu), 1.702, 7.0, stream.cuda_stream)
                _lib.check(rc, "lyra_decode_gemm_ex")

            cases.append((f"{label} expert {name} ({E}x{K}x{N} fp8), 64 tokens, {touched} experts with rows", nbytes, launch, []))
        group = 4  # launches per event bracket (an event pair costs a few microseconds of its own), each on another weight set
        for r in range(rounds + 2):  # the first two rounds warm up
            one_step()
            for _, _, launch, pairs in cases:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                for i in range(group):
                    launch(r * group + i)
                b.record(stream)
                if r >= 2:
                    pairs.append((a, b))
        stream.synchronize()
        for case, nbytes, _, pairs in cases:
            t = sum(a.elapsed_time(b) for a, b in pairs) * 1e-3 / (len(pairs) * group)
            out_rows.append({"kernel": "decode_gemm_group_kernel<fp8> (tiled activations, as in the decode step)", "case": case, "bound": "hbm", "achieved": nbytes / t / 1e9,
                             "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / t / 1e9 / HBM_PEAK_GBS,
                             "algorithmic_bytes": nbytes, "us_per_launch": t * 1e6,
                             "timing": f"HIP events around groups of {group} launches on rotating weight sets, between replays of the decode step"})
        del cases
    return out_rows


def _time_launches(launch, stream, warm=5, iters=50):
    import torch

    for i in range(warm):
        launch(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream.synchronize()
    start.record(stream)
    for i in range(iters):
        launch(i)
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / iters


def benchmark_routing():
    """The routing instances of the operator table and of `roofline.gemm`, drawn in one fixed order from one seeded generator
    so that both measure the same group sizes: rows per expert for lyra-medium at 1, 16 and 64 tokens, a second 64-token draw
    (the scale-block case), lyra-max at 128 tokens, lyra-small at 8 and 64 tokens."""
    import numpy as np

    rng = np.random.default_rng(1003)
    r = {f"medium_T{T}": zipf_group_sizes(rng, T, 31, 3, 1) for T in (1, 16, 64)}
    r["medium_T64_blocks"] = zipf_group_sizes(rng, 64, 31, 3, 1)
    r["max_B128"] = zipf_group_sizes(rng, 128, 63, 3, 1)
    r["small_B8"] = zipf_group_sizes(rng, 8, 15, 3, 1)
    r["small_B64"] = zipf_group_sizes(rng, 64, 15, 3, 1)
    r["probe"] = zipf_group_sizes(rng, 64, 15, 3, 1)
    r["gptoss_B64"] = zipf_group_sizes(rng, 64, 32, 4, 0)  # gpt-oss-20b: 4 of 32 routed experts per token, no shared expert
    return r


def zipf_group_sizes(rng, tokens, n_routed, k_routed, n_shared):
    """Rows per expert when every token picks `k_routed` distinct routed experts with p_i ~ i^-1.1 and all shared ones."""
    import numpy as np

    p = 1.0 / np.arange(1, n_routed + 1) ** 1.1
    p /= p.sum()
    ids = np.stack([rng.choice(n_routed, size=k_routed, replace=False, p=p) for _ in range(tokens)])
    if n_shared:
        ids = np.concatenate([ids, np.broadcast_to(np.arange(n_routed, n_routed + n_shared), (tokens, n_shared))], 1)
    return np.bincount(ids.reshape(-1), minlength=n_routed + n_shared).astype(np.int32)


def kernel_table(dev, only="", span_major=False, tiled=False):
    """Stand-alone timings of the two operators through the C ABI at the shapes of the named model variants: HIP events
    over back-to-back launches, once rotating over enough distinct caches / weight sets that every launch streams from
    HBM ("cold") and once re-using one set ("hot", which the 256 MB last-level cache may serve in part)."""
    import numpy as np
    import torch

    from lyra_amd import _lib

    L = _lib.lib
    stream = torch.cuda.current_stream(dev)
    rows = []
    gen = torch.Generator(device=dev)
    gen.manual_seed(1000)

    def attention(label, B, N, K, H, S, sw, fp8, lengths=None, ranked=False):
        if only not in label:
            return
        es = 1 if fp8 else 2
        per = 2 * B * K * S * (H * es + (4 if fp8 else 0))
        nbuf = max(2, min(8, int(1.2e9 // per) + 1))
        caches = []
        for _ in range(nbuf):
            if fp8:
                kv = [torch.randint(0, 0x78, (B, K, S, H), generator=gen, device=dev, dtype=torch.uint8) for _ in range(2)]
                sc = [torch.rand(B, K, S, generator=gen, device=dev) * 0.004 + 0.006 for _ in range(2)]
            else:
                kv = [torch.randn(B, K, S, H, generator=gen, device=dev, dtype=torch.bfloat16) for _ in range(2)]
                sc = [None, None]
            caches.append((kv, sc))
        q = torch.randn(B, N, H, generator=gen, device=dev, dtype=torch.bfloat16)
        out = torch.empty_like(q)
        sinks = torch.randn(N, generator=gen, device=dev)
        if lengths is None:
            pos = torch.full((1,), S - 1, dtype=torch.int32, device=dev)
            stride, visible = 0, B * (min(sw, S) if sw else S)
        else:
            pos = torch.from_numpy(lengths.astype(np.int32) - 1).to(dev)
            stride, visible = 1, int(np.minimum(lengths, sw).sum() if sw else lengths.sum())
        need = L.lyra_decode_attention_workspace(B, N, K, S, H, sw)
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)

        order = None
        if ranked:  # the rows ranked by length once (lyra_attention_rank), as a decode step would do it for all its layers
            order = torch.empty(B, dtype=torch.int32, device=dev)
            _lib.check(L.lyra_attention_rank(pos.data_ptr(), B, order.data_ptr(), stream.cuda_stream), "lyra_attention_rank")

        def launch(i, hot=False):
            (k, v), (ks, vs) = caches[0 if hot else i % nbuf]
            head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), ks.data_ptr() if fp8 else None, vs.data_ptr() if fp8 else None,
                    sinks.data_ptr(), pos.data_ptr(), stride)
            tail = (None, out.data_ptr(), ws.data_ptr(), ws.numel(), B, N, K, S, H, H**-0.5, sw,
                    _lib.DTYPE_E4M3FN if fp8 else _lib.DTYPE_BF16, _lib.DTYPE_BF16, stream.cuda_stream)
            rc = L.lyra_decode_attention_ranked(*head, order.data_ptr(), *tail) if ranked else L.lyra_decode_attention(*head, *tail)
            _lib.check(rc, "lyra_decode_attention")

        nbytes = 2 * K * visible * (H * es + (4 if fp8 else 0))
        cold = _time_launches(launch, stream)
        hot = _time_launches(lambda i: launch(i, True), stream)
        rows.append({"operator": "decode_attention", "case": label, "bytes": nbytes, "cold_us": cold * 1e6, "hot_us": hot * 1e6})
        del caches

    def gemm(label, M, G, K, N, sizes, swiglu, block, fp8=True, out_f32=False):
        if only not in label:
            return
        es = 1 if fp8 else 2
        nbuf = max(2, min(6, int(600e6 // (G * K * N * es)) + 1))
        if fp8:
            weights = [torch.randint(0, 0x78, (G, K, N), generator=gen, device=dev, dtype=torch.uint8) for _ in range(nbuf)]
            bk, bn = block
            scale = torch.rand(G, K // bk, N // bn, generator=gen, device=dev) * 0.001 + 0.0005
        else:
            weights = [torch.randn(G, K, N, generator=gen, device=dev, dtype=torch.bfloat16) for _ in range(nbuf)]
            bk = bn = 0
            scale = None
        lhs = torch.randn(M, K, generator=gen, device=dev, dtype=torch.bfloat16)
        gs = torch.from_numpy(np.asarray(sizes, np.int32)).to(dev)
        NO = N // 2 if swiglu else N
        out = torch.empty(M, NO, device=dev, dtype=torch.float32 if out_f32 else torch.bfloat16)
        need = L.lyra_decode_gemm_workspace(M, G, K, N, int(swiglu))
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)
        touched = int((np.asarray(sizes) > 0).sum())
        nbytes = touched * K * N * es + (touched * (K // bk) * (N // bn) * 4 if fp8 else 0) + M * K * 2 + M * NO * out.element_size()

        dt = _lib.DTYPE_E4M3FN if fp8 else _lib.DTYPE_BF16
        flag = 0
        if tiled and N < 100000 and K % 32 == 0:  # activations in tiles of 16 rows x 32 columns, as the fused decode step hands them over
            flag |= _lib.LHS_TILED16
            lhs = torch.randn((M + 15) // 16 * 16, K, generator=gen, device=dev, dtype=torch.bfloat16)
            label += " [tiled activations]"
        if span_major and N < 100000:  # the weights in the span-major copy lyra_gemm_pack makes (not for the LM head's kernel)
            layout = 2 if (swiglu and G > 1) else 1
            flag |= _lib.RHS_SPAN_MAJOR if layout == 1 else _lib.RHS_SPAN_MAJOR_GLU
            packed = []
            for w in weights:
                buf = torch.empty(L.lyra_gemm_packed_bytes(G, K, N, dt, layout), dtype=torch.uint8, device=dev)
                _lib.check(L.lyra_gemm_pack(w.data_ptr(), buf.data_ptr(), G, K, N, dt, layout, stream.cuda_stream), "lyra_gemm_pack")
                packed.append(buf)
            stream.synchronize()
            weights = packed
            label += " [span-major]"

        def launch(i, hot=False):
            rc = L.lyra_decode_gemm_ex(
                lhs.data_ptr(), None, weights[0 if hot else i % nbuf].data_ptr(), scale.data_ptr() if fp8 else None, bk, bn,
                gs.data_ptr(), None, None, 1.0, 0, out.data_ptr(), ws.data_ptr(), ws.numel(), M, G, K, N,
                dt | flag, _lib.DTYPE_F32 if out_f32 else _lib.DTYPE_BF16, int(swiglu), 1.702, 7.0, stream.cuda_stream)
            _lib.check(rc, "lyra_decode_gemm_ex")

        cold = _time_launches(launch, stream)
        hot = _time_launches(lambda i: launch(i, True), stream)
        rows.append({"operator": "decode_gemm", "case": label, "bytes": nbytes, "rows": M, "touched_experts": touched,
                     "cold_us": cold * 1e6, "hot_us": hot * 1e6})
        del weights

    routing = benchmark_routing()
    attention("lyra-small B=1 ctx 512 bf16 global", 1, 16, 4, 128, 512, 0, False)
    attention("lyra-small B=8 ctx 4096 fp8 global", 8, 16, 4, 128, 4096, 0, True)
    attention("lyra-small B=64 ctx 4096 fp8 global (headline)", 64, 16, 4, 128, 4096, 0, True)
    attention("lyra-small B=64 ctx 4096 fp8 sliding 128", 64, 16, 4, 128, 4096, 128, True)
    attention("lyra-small B=64 ctx 4096 bf16 global", 64, 16, 4, 128, 4096, 0, False)
    attention("lyra-medium B=64 ctx 4096 fp8 global", 64, 32, 8, 128, 4096, 0, True)
    attention("lyra-max B=128 ctx 4096 fp8 global", 128, 32, 8, 128, 4096, 0, True)
    lengths = np.random.default_rng(1004).integers(256, 4097, size=64)
    attention("gpt-oss shape B=64 64Q/8KV H=64 fp8 ragged 256..4096 global", 64, 64, 8, 64, 4096, 0, True, lengths)
    attention("gpt-oss shape B=64 64Q/8KV H=64 fp8 ragged sliding 128", 64, 64, 8, 64, 4096, 128, True, lengths)
    attention("gpt-oss shape B=64 64Q/8KV H=64 ctx 4096 fp8 global", 64, 64, 8, 64, 4096, 0, True)
    attention("gpt-oss shape B=64 64Q/8KV H=64 fp8 ragged 256..4096 global, rows ranked once", 64, 64, 8, 64, 4096, 0, True, lengths, ranked=True)
    attention("lyra-medium B=64 fp8 ragged 256..4096 global", 64, 32, 8, 128, 4096, 0, True, lengths)
    attention("lyra-medium B=64 fp8 ragged 256..4096 global, rows ranked once", 64, 32, 8, 128, 4096, 0, True, lengths, ranked=True)
    attention("lyra-medium B=64 ctx 4096 fp8 global, one position per row", 64, 32, 8, 128, 4096, 0, True, np.full(64, 4096))
    attention("lyra-max B=128 ctx 4096 fp8 global, one position per row", 128, 32, 8, 128, 4096, 0, True, np.full(128, 4096))
    for T in (1, 16, 64):
        s = routing[f"medium_T{T}"]
        gemm(f"lyra-medium expert up+SwiGLU T={T} (32x4096x8192 fp8)", int(s.sum()), 32, 4096, 8192, s, True, (4096, 1))
        gemm(f"lyra-medium expert down T={T} (32x4096x4096 fp8)", int(s.sum()), 32, 4096, 4096, s, False, (4096, 1))
    even = np.array([8] * 31 + [64], np.int32)  # evenly routed tokens (what a load-balancing loss aims at) + the shared expert
    gemm("lyra-medium expert up+SwiGLU T=64, even routing (32x4096x8192 fp8)", int(even.sum()), 32, 4096, 8192, even, True, (4096, 1))
    gemm("lyra-medium expert down T=64, even routing (32x4096x4096 fp8)", int(even.sum()), 32, 4096, 4096, even, False, (4096, 1))
    s = routing["medium_T64_blocks"]
    gemm("lyra-medium expert up+SwiGLU T=64, scale blocks (256,256)", int(s.sum()), 32, 4096, 8192, s, True, (256, 256))
    s = routing["max_B128"]
    gemm("lyra-max expert up+SwiGLU B=128 (64x4096x8192 fp8)", int(s.sum()), 64, 4096, 8192, s, True, (4096, 1))
    gemm("lyra-max expert down B=128 (64x4096x4096 fp8)", int(s.sum()), 64, 4096, 4096, s, False, (4096, 1))
    for B in (8, 64):
        s = routing[f"small_B{B}"]
        gemm(f"lyra-small expert up+SwiGLU B={B} (16x2048x4096 fp8)", int(s.sum()), 16, 2048, 4096, s, True, (2048, 1))
        gemm(f"lyra-small expert down B={B} (16x2048x2048 fp8)", int(s.sum()), 16, 2048, 2048, s, False, (2048, 1))
    if only and "probe" in only:  # what the 64-row units of the shared expert cost: the same routing with a light shared expert
        s = routing["probe"]
        for shared_rows in (64, 32, 16):
            t = s.copy()
            t[15] = shared_rows
            gemm(f"probe lyra-small expert up+SwiGLU B=64, shared expert {shared_rows} rows", int(t.sum()), 16, 2048, 4096, t, True, (2048, 1))
            gemm(f"probe lyra-small expert down B=64, shared expert {shared_rows} rows", int(t.sum()), 16, 2048, 2048, t, False, (2048, 1))
        print("rows per expert:", s.tolist(), file=sys.stderr)
        # what a unit costs by its number of rows: every expert of the lyra-medium up projection with the same row count
        for rows_each in (8, 16, 32, 48, 64):
            t = np.full(32, rows_each, np.int32)
            gemm(f"probe lyra-medium expert up+SwiGLU, {rows_each} rows for each of 32 experts", int(t.sum()), 32, 4096, 8192, t, True, (4096, 1))
    for name, K, N, sw in (("q/k/v", 2048, 3072, False), ("out", 2048, 2048, False), ("dense up+SwiGLU", 2048, 6144, True),
                           ("dense down", 3072, 2048, False)):
        gemm(f"lyra-small {name} projection B=64 ({K}x{N} fp8)", 64, 1, K, N, [64], sw, (K, 1))
    gemm("lyra-medium dense up+SwiGLU B=64 (4096x12288 fp8)", 64, 1, 4096, 12288, [64], True, (4096, 1))
    # gpt-oss-20b: width 2880 = 22.5 spans of 128 columns
    s = routing["gptoss_B64"]
    gemm("gpt-oss-20b expert up+SwiGLU B=64 (32x2880x5760 fp8)", int(s.sum()), 32, 2880, 5760, s, True, (2880, 1))
    gemm("gpt-oss-20b expert down B=64 (32x2880x2880 fp8)", int(s.sum()), 32, 2880, 2880, s, False, (2880, 1))
    gemm("gpt-oss-20b q/k/v projection B=64 (2880x5120 fp8)", 64, 1, 2880, 5120, [64], False, (2880, 1))
    gemm("gpt-oss-20b out projection B=64 (4096x2880 fp8)", 64, 1, 4096, 2880, [64], False, (4096, 1))
    gemm("lyra-small LM head B=64 (2048x204800 bf16, f32 logits)", 64, 1, 2048, 204800, [64], False, None, fp8=False, out_f32=True)
    for r in rows:
        r["cold_GBs"] = r["bytes"] / r["cold_us"] / 1e3
        r["cold_frac_of_peak"] = r["cold_GBs"] / HBM_PEAK_GBS
    return rows


def traffic_probe(device, mib=256, repeats=4):
    """A plain streaming kernel of known HBM traffic (reads `mib` MiB, writes `mib` MiB per launch), launched a few
    times so that a hardware-counter run of this script can scale FETCH_SIZE / WRITE_SIZE against it."""
    import torch

    n = mib * (1 << 20) // 4
    src = torch.arange(n, dtype=torch.int32, device=device)
    dst = torch.empty_like(src)
    for _ in range(repeats):
        torch.add(src, 1, out=dst)
    torch.cuda.synchronize()
    return {"kernel": "torch add(int32, 1)", "read_bytes": n * 4, "write_bytes": n * 4, "launches": repeats}


def cpu_baseline(cfg, weights, cache, ctx, sample_batch):
    """The CPU restatement of the reference decode step (oracle/decode_step.py, threaded C contractions) on the first
    `sample_batch` sequences of the same workload: full steps, all layers, at the benchmarked context."""
    import numpy as np
    import torch

    from oracle import clib
    from oracle import decode_step as D

    wn = D.weights_to_numpy(weights, cfg)
    sub = lambda a: a[:sample_batch]
    cn = {"k": [], "v": []}
    for layer in cache.layers:
        for name in ("k", "v"):
            arr = getattr(layer, name)
            cn[name].append((sub(arr.qval.view(torch.uint8)).cpu().numpy().copy(), sub(arr.scale).float().cpu().numpy().copy()))
    tokens = np.arange(sample_batch) + 17
    # whole steps of the sampled sequences until about 10 s of CPU work are done (at most 6 steps, each at full context:
    # the appended cache row is overwritten by the next repetition)
    done, dt = 0, 0.0
    t0 = time.perf_counter()
    while done < 6 and dt < 10.0:
        logits = D.decode_step(tokens, wn, cn, ctx - 1, cfg, use_c=True)
        done += 1
        dt = time.perf_counter() - t0
    assert np.isfinite(logits[:, : cfg.vocab_size]).all()
    return {
        "value": sample_batch * done / dt,
        "unit": "tokens/s",
        "cores": clib.load().lyra_oracle_num_threads(),
        "kind": "port",
        "sample": f"{done} full decode steps ({cfg.n_layers} layers + LM head, ctx {ctx}, FP8 cache and weights) for {sample_batch} of "
                  f"the batch's sequences; {dt:.1f} s of CPU work, host cores visible: {os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=4096)
    ap.add_argument("--cpu-sample", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm-roofline", action="store_true", help="skip the stand-alone expert matmul and extra attention timings")
    ap.add_argument("--no-variants", action="store_true", help="skip the step under other settings (other sampler, B=8, reference-fp8 layout)")
    ap.add_argument("--sampler", default="default", choices=["default", "greedy"],
                    help="default: temperature 0.8 over the top 4, the reference's setting (lyra/model.py:107-108); greedy: arg-max")
    ap.add_argument("--layout", default="headline", choices=["headline", "reference-fp8"],
                    help="headline: FP8 cache, every projection and MLP weight FP8 with one scale per output channel; "
                         "reference-fp8: FP8 cache and MLP weights with (256, 256) scale blocks, attention projections bf16")
    ap.add_argument("--model", default="lyra-small", help="model variant of the decode step (the headline figure is lyra-small)")
    ap.add_argument("--kernels", action="store_true",
                    help="instead of the decode step, time both operators stand-alone at the shapes of every model variant")
    ap.add_argument("--only", default="", help="with --kernels: only the cases whose name contains this text")
    ap.add_argument("--tiled", action="store_true",
                    help="with --kernels: the matmuls read their activations in tiles of 16 rows x 32 columns (LYRA_LHS_TILED16)")
    ap.add_argument("--span-major", action="store_true",
                    help="with --kernels: the matmuls read the span-major copy of their weights (lyra_gemm_pack)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch a copy-like kernel of known size (reference point for rocprofv3 --pmc runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's decode path; run with --gpus 1 (no multi-GPU figure exists).")

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    if args.kernels:
        rows = kernel_table(dev, args.only, args.span_major, args.tiled)
        if args.traffic_probe:
            traffic_probe(dev)
        for r in rows:
            print(f"| {r['operator']} | {r['case']} | {r['bytes'] / 1e6:.1f} | {r['cold_us']:.1f} | {r['cold_GBs'] / 1e3:.2f} | "
                  f"{100 * r['cold_frac_of_peak']:.1f} | {r['hot_us']:.1f} |", file=sys.stderr)
        print(json.dumps({"metric": "operator launch time at model shapes", "unit": "us", "peak_GBs": HBM_PEAK_GBS, "kernels": rows}))
        return
    greedy = args.sampler == "greedy"
    cfg, weights, cache = build_model(args.batch, args.ctx, dev, args.model, args.layout)
    elapsed, one_step = time_decode_steps(cfg, weights, cache, args.batch, args.ctx, args.steps, args.warmup, greedy=greedy)
    tokens_per_s = args.batch * args.steps / elapsed

    from lyra_amd.model import model_apply

    def algorithmic_bytes(cfg_, weights_, cache_, batch):
        """(bytes one step must move, experts with rows per MoE layer), from the step's own routing: one eager step (the
        graph replays the same kernels on the same inputs)."""
        groups = []
        cache_.pos.fill_(args.ctx - 1)
        model_apply(torch.arange(batch, device=dev) % cfg_.vocab_size, weights_, cache_, cfg_, groups_out=groups, advance=False)
        touched_ = [int((g > 0).sum().item()) for g in groups]
        return step_algorithmic_bytes(cfg_, weights_, batch, args.ctx, touched_), touched_

    step_bytes, touched = algorithmic_bytes(cfg, weights, cache, args.batch)

    t_attn = time_dominant_kernel(cfg, weights, cache, args.batch, args.ctx, one_step)
    t_attn_front = None
    if weights.layers[1].attn.xsa_alpha is None and args.batch * cfg.n_kv_heads <= 256:  # the launch the step itself uses
        t_attn_front = time_dominant_kernel(cfg, weights, cache, args.batch, args.ctx, one_step, front=True)
    stream = torch.cuda.current_stream(dev)
    gemm_rows = time_expert_matmuls(dev, one_step, stream) if not args.no_gemm_roofline else None
    attn_bytes = attention_algorithmic_bytes(args.batch, cfg.n_kv_heads, args.ctx, cfg.head_dim, fp8=True)
    headline_shape = (args.model, args.batch, args.ctx) == ("lyra-small", 64, 4096)

    # HBM traffic per launch from hardware counters: collected in separate rocprofv3 --pmc runs and kept in profiles/; quoted
    # only while the kernel's sources are the ones the counters were collected on
    traffic, traffic_plain, traffic_note = None, None, "no counters file"
    tpath = os.path.join(ROOT, "profiles", "decode_attention_traffic.json")
    if os.path.exists(tpath) and headline_shape:
        with open(tpath) as f:
            tj = json.load(f)
        if tj.get("source_sha256_16") == source_fingerprint():
            traffic, traffic_plain = tj.get("hbm_bytes_per_launch_front_step"), tj.get("hbm_bytes_per_launch")
            traffic_note = f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, {tpath[len(ROOT) + 1:]} (sources {tj['source_sha256_16']})"
        else:
            traffic_note = "the counters in profiles/decode_attention_traffic.json were collected on other kernel sources: not quoted"

    plain = {
        "kernel": "decode_attention_kernel<128, fp8> (global layer; the operator on its own, lyra_decode_attention)",
        "us_per_launch": t_attn * 1e6,
        "achieved": attn_bytes / t_attn / 1e9,
        "frac": attn_bytes / t_attn / 1e9 / HBM_PEAK_GBS,
        "traffic": traffic_plain,
    }
    t_main = t_attn_front if t_attn_front is not None else t_attn
    result = {
        "metric": "decode tokens/s at B=64 ctx 4096 FP8 cache; achieved HBM GB/s (% peak)",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn weights and KV cache, bf16 activations, f32 accumulate",
        "data": "synthetic (random-init weights N(0,0.02), random KV history)",
        "config": {
            "workload": f"full {args.model} decode step ({cfg.n_layers} layers, {cfg.n_attn_heads}Q/{cfg.n_kv_heads}KV heads, "
                        f"H={cfg.head_dim}, {cfg.n_routed_experts}+{cfg.n_shared_experts} experts, LM head {cfg.padded_vocab_size}), "
                        f"B={args.batch}, ctx {args.ctx}, FP8 KV cache, " + ("FP8 per-output-channel weights" if args.layout == "headline" else
                        "FP8 MLP weights with (256, 256) scale blocks, bf16 attention projections") +
                        (", greedy sampling" if greedy else f", sampling at temperature {cfg.sample_temperature} over the top {cfg.sample_topk} (the reference's default)"),
            "batch": args.batch,
            "ctx": args.ctx,
            "us_per_layer": elapsed / args.steps / cfg.n_layers * 1e6,
            "step_algorithmic_bytes": step_bytes,
            "step_frac": step_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBS,  # of the 8 TB/s roofline, whole step
            "experts_with_rows_per_moe_layer": touched,
            "projections": ("q/k/v and output projections FP8 as well (quantize_attn; the reference's --fp8 leaves them bf16)"
                            if args.layout == "headline" else "q/k/v and output projections bf16, as the reference's --fp8 leaves them"),
        },
        "roofline": {
            # the launch the decode step runs: with the step in front of the attention (QK norm, rotary embedding, cache
            # append) fused in when the model allows it; timed in groups of one launch per global layer between step replays
            "kernel": ("decode_attention_kernel<128, fp8, QK norm + RoPE + cache append> (global layer; the launch of the decode step, "
                       "lyra_decode_attention_qkv)" if t_attn_front is not None else plain["kernel"]),
            "bound": "hbm",
            "achieved": attn_bytes / t_main / 1e9,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": attn_bytes / t_main / 1e9 / HBM_PEAK_GBS,
            "traffic": traffic if t_attn_front is not None else traffic_plain,
            "traffic_source": traffic_note,
            "algorithmic_bytes": attn_bytes,
            "us_per_launch": t_main * 1e6,
            "timing": "HIP events around groups of 8 launches (one per global layer's cache) between replays of the decode step",
        },
    }
    if t_attn_front is not None:
        result["roofline"]["attention_operator"] = plain
    if not args.no_gemm_roofline:
        t_sus, n_sus = time_attention_sustained(cfg, weights, cache, args.batch, args.ctx)
        result["roofline"]["attention_sustained"] = {
            "kernel": plain["kernel"], "launches_back_to_back": n_sus, "us_per_launch": t_sus * 1e6,
            "achieved": attn_bytes / t_sus / 1e9, "frac": attn_bytes / t_sus / 1e9 / HBM_PEAK_GBS,
            "note": "one HIP-event bracket around all launches, rotating over the global layers' caches (every launch from HBM)"}
        result["roofline"]["attention_ragged"] = time_attention_ragged(dev, one_step, stream)
    if gemm_rows is not None:
        result["roofline"]["gemm"] = gemm_rows
    if not args.no_variants and headline_shape and args.layout == "headline":
        # the same step under the other settings a reader may ask for; each is its own captured graph, timed like the headline
        variants = []

        def timed(name, cfg_, weights_, cache_, batch, greedy_):
            el, _ = time_decode_steps(cfg_, weights_, cache_, batch, args.ctx, args.steps, args.warmup, greedy=greedy_)
            nbytes, _ = algorithmic_bytes(cfg_, weights_, cache_, batch)
            variants.append({"variant": name, "batch": batch, "ms_per_step": el / args.steps * 1e3, "tokens_per_s": batch * args.steps / el,
                             "step_algorithmic_bytes": nbytes, "step_frac": nbytes / (el / args.steps) / 1e9 / HBM_PEAK_GBS})

        timed("greedy sampling (arg-max)" if not greedy else "sampling at temperature 0.8 over the top 4", cfg, weights, cache, args.batch, not greedy)
        cfg8, _, cache8 = build_model(8, args.ctx, dev, args.model, args.layout, weights=weights)
        timed("B=8 (benchmark configuration 2)", cfg8, weights, cache8, 8, greedy)
        del cache8
        if not args.no_cpu_baseline:  # (the CPU baseline reads the headline model: take it before the model is replaced)
            result["cpu_baseline"] = cpu_baseline(cfg, weights, cache, args.ctx, min(args.cpu_sample, args.batch))
        del weights, cache, one_step
        torch.cuda.empty_cache()
        cfg_r, weights_r, cache_r = build_model(args.batch, args.ctx, dev, args.model, "reference-fp8")
        timed("layout reference-fp8 (what the reference's --fp8 sets: FP8 MLP weights with (256, 256) scale blocks and an FP8 cache, "
              "bf16 attention projections)", cfg_r, weights_r, cache_r, args.batch, greedy)
        result["variants"] = variants
        weights = cache = None
    if args.traffic_probe:
        result["traffic_probe"] = traffic_probe(dev)
    if not args.no_cpu_baseline and "cpu_baseline" not in result:
        result["cpu_baseline"] = cpu_baseline(cfg, weights, cache, args.ctx, min(args.cpu_sample, args.batch))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
