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


def build_model(batch, ctx, device):
    import torch

    from lyra_amd.model import MODEL_VARIANTS, apply_inference_overrides, init_cache, init_weights
    from lyra_amd.nn.quant import QArray

    cfg = apply_inference_overrides(MODEL_VARIANTS["lyra-small"], fp8=True, fp8_attn=True, per_channel=True)
    weights = init_weights(cfg, device)
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


def time_decode_steps(cfg, weights, cache, batch, ctx, steps, warmup):
    import torch

    from lyra_amd.generate import GraphedDecoder

    dec = GraphedDecoder(weights, cache, cfg, batch)
    dec.tokens.copy_(torch.randint(0, cfg.vocab_size, (batch,), device=dec.tokens.device))

    def one_step():
        cache.pos.fill_(ctx - 1)  # every timed step runs at full context
        dec.step()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert torch.isfinite(dec.logits[:, : cfg.vocab_size]).all(), "non-finite logits"
    return elapsed


def time_dominant_kernel(cfg, weights, cache, batch, ctx, launches=100):
    """Average duration of the FP8 global-layer decode-attention launch, HIP events on the launch stream, rotating
    over the caches of the model's global layers so every launch streams from HBM (working set >> 256 MB MALL)."""
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
    need = L.lyra_decode_attention_workspace(batch, N, K, ctx, H, 0)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)

    def launch(i):
        c = layers[i % len(layers)]
        rc = L.lyra_decode_attention(
            q.data_ptr(), c.k.qval.data_ptr(), c.v.qval.data_ptr(), c.k.scale.data_ptr(), c.v.scale.data_ptr(), sinks.data_ptr(),
            pos.data_ptr(), 0, None, out.data_ptr(), ws.data_ptr(), ws.numel(), batch, N, K, ctx, H, H**-0.5, 0,
            _lib.DTYPE_E4M3FN, _lib.DTYPE_BF16, stream.cuda_stream)
        _lib.check(rc, "lyra_decode_attention")

    for i in range(10):
        launch(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream.synchronize()
    start.record(stream)
    for i in range(launches):
        launch(i)
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / launches  # seconds per launch


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
    `sample_batch` sequences of the same workload: one full step, all layers, context 4096."""
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
    t0 = time.perf_counter()
    logits = D.decode_step(tokens, wn, cn, ctx - 1, cfg, use_c=True)
    dt = time.perf_counter() - t0
    assert np.isfinite(logits[:, : cfg.vocab_size]).all()
    return {
        "value": sample_batch / dt,
        "unit": "tokens/s",
        "cores": clib.load().lyra_oracle_num_threads(),
        "kind": "port",
        "sample": f"one full decode step (16 layers + LM head, ctx {ctx}, FP8 cache and weights) for {sample_batch} of the "
                  f"batch's sequences; {dt:.1f} s of CPU work, host cores visible: {os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=4096)
    ap.add_argument("--cpu-sample", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch a copy-like kernel of known size (reference point for rocprofv3 --pmc runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's decode path; run with --gpus 1 (no multi-GPU figure exists).")

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    cfg, weights, cache = build_model(args.batch, args.ctx, dev)
    elapsed = time_decode_steps(cfg, weights, cache, args.batch, args.ctx, args.steps, args.warmup)
    tokens_per_s = args.batch * args.steps / elapsed

    t_attn = time_dominant_kernel(cfg, weights, cache, args.batch, args.ctx)
    attn_bytes = attention_algorithmic_bytes(args.batch, cfg.n_kv_heads, args.ctx, cfg.head_dim, fp8=True)
    achieved = attn_bytes / t_attn / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "decode_attention_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")

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
            "workload": f"full lyra-small decode step (16 layers, 16Q/4KV heads, H=128, 15+1 experts, LM head 204800), "
                        f"B={args.batch}, ctx {args.ctx}, FP8 KV cache, FP8 per-output-channel weights, greedy sampling",
            "batch": args.batch,
            "ctx": args.ctx,
            "us_per_layer": elapsed / args.steps / cfg.n_layers * 1e6,
        },
        "roofline": {
            "kernel": "decode_attention_kernel<128, fp8> (global layer)",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "algorithmic_bytes": attn_bytes,
            "us_per_launch": t_attn * 1e6,
        },
    }
    if args.traffic_probe:
        result["traffic_probe"] = traffic_probe(dev)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, weights, cache, args.ctx, min(args.cpu_sample, args.batch))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
