"""Writes the golden fixtures under tests/golden/ with the NumPy oracle (oracle/lyra_oracle.py).

    python tests/golden/make_fixtures.py

The reference cannot be imported in this environment (it needs Python >= 3.14 and JAX), so the vectors are the
oracle's float32 outputs on seeded inputs; the oracle itself is pinned by tests/test_oracle_*.py against torch,
closed forms and the vectors the reference's own tests hold.  Each .npz stores inputs and expected outputs; the GPU
tests feed the same inputs to the HIP kernels, the CPU tests feed them to the C restatement.  Files stay small
(reduced sizes of the benchmark configurations).
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import lyra_oracle as O  # noqa: E402


def attention_fixture(name, seed, B, N, K, S, H, sw, fp8, positions, gate):
    rng = np.random.default_rng(seed)
    q = O.bf16_round(rng.standard_normal((B, N, 1, H), dtype=np.float32))
    k = O.bf16_round(rng.standard_normal((B, K, S, H), dtype=np.float32))
    v = O.bf16_round(rng.standard_normal((B, K, S, H), dtype=np.float32))
    sinks = rng.standard_normal(N).astype(np.float32)
    g = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((B, N))))).astype(np.float32)) if gate else None
    data = dict(q=O.bf16_bits(q), sinks=sinks, position=np.asarray(positions, np.int32), sliding_window=np.int32(sw))
    if fp8:
        kq, ks = O.quantize(k, (1, H))
        vq, vs = O.quantize(v, (1, H))
        data.update(k_codes=kq, k_scale=ks, v_codes=vq, v_scale=vs)
        kk, vv = (kq, ks), (vq, vs)
    else:
        data.update(k=O.bf16_bits(k), v=O.bf16_bits(v))
        kk, vv = k, v
    out = np.stack([
        O.decode_attention_reference(q[b : b + 1], _row(kk, b), _row(vv, b), sinks, H**-0.5, sw, int(positions[b]),
                                     mode="fp32", gate=None if g is None else g[b : b + 1])[0]
        for b in range(B)
    ])
    if g is not None:
        data["gate"] = O.bf16_bits(g)
    data["out_fp32"] = out.astype(np.float32)
    np.savez_compressed(os.path.join(HERE, name), **data)


def _row(arr, b):
    return (arr[0][b : b + 1], arr[1][b : b + 1]) if isinstance(arr, tuple) else arr[b : b + 1]


def gemm_fixture(name, seed, sizes, K, N, fp8, block, swiglu, bias):
    rng = np.random.default_rng(seed)
    sizes = np.asarray(sizes, np.int32)
    G, M = sizes.shape[0], int(sizes.sum()) + 2  # two rows past the last group (ragged_dot zero rows)
    lhs = O.bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    w = O.bf16_round((rng.standard_normal((G, K, N)) * 0.05).astype(np.float32))
    b = rng.standard_normal((G, N)).astype(np.float32) if bias else None
    data = dict(lhs=O.bf16_bits(lhs), group_sizes=sizes, swiglu=np.int32(swiglu))
    if fp8:
        wq, ws = O.quantize(w, block)
        data.update(rhs_codes=wq, rhs_scale=ws, block=np.asarray(block, np.int32))
        out = O.decode_gemm_reference(lhs, (wq, ws), sizes, block=block, bias=b, fused_swiglu=swiglu, mode="fp32")
    else:
        data.update(rhs=O.bf16_bits(w))
        out = O.decode_gemm_reference(lhs, w, sizes, bias=b, fused_swiglu=swiglu, mode="fp32")
    if b is not None:
        data["bias"] = b
    data["out_fp32"] = out.astype(np.float32)
    np.savez_compressed(os.path.join(HERE, name), **data)


def tables_fixture():
    S = 512
    rows = []
    for sw in (0, 1, 127, 128, 129, 256):
        for pos in range(S):
            lo, hi = O.visible_range(pos, sw, S)
            rows.append((sw, pos, lo, hi, O.sliding_start(pos, sw, S) if O.is_sw(sw, S) else 0, int(O.is_sw(sw, S))))
    np.savez_compressed(os.path.join(HERE, "tables.npz"), fp8_e4m3fn=O.fp8_e4m3fn_decode_table().astype(np.float32),
                        window_rows=np.asarray(rows, np.int32),
                        window_columns=np.asarray(["sliding_window", "position", "first_visible", "last_visible", "slab_start", "is_sw"]))


def routing_fixture():
    # assignments of lyra's tests/test_combine.py:13-17 and their stable counting sort
    assignments = np.asarray([0, 2, 4, 7, 1, 3, 4, 7], np.int32)
    groups = np.bincount(assignments, minlength=8).astype(np.int32)
    perm, dest = O.bpermute(assignments, groups, 8)
    rng = np.random.default_rng(1006)
    logits = rng.standard_normal((16, 15)).astype(np.float32)
    logits[3, :] = 0.5
    scores, active, g2 = O.route_tokens(logits, 3, 15, 1)
    p2, d2 = O.bpermute(active, g2, 16)
    np.savez_compressed(os.path.join(HERE, "routing.npz"), assignments=assignments, groups=groups, permute=perm, unpermute=dest,
                        logits=logits, scores=scores, active_map=active, route_groups=g2, route_permute=p2, route_unpermute=d2)


def main():
    # config 1 of the benchmark list at full size; the others reduced
    attention_fixture("attn_cfg1_bf16_b1_s512.npz", 1001, 1, 16, 4, 512, 128, 0, False, [511], True)
    attention_fixture("attn_small_fp8_b3_s512.npz", 1002, 3, 16, 4, 512, 128, 0, True, [511, 300, 0], True)
    attention_fixture("attn_small_fp8_window_b3_s512.npz", 1012, 3, 16, 4, 512, 128, 128, True, [511, 130, 5], False)
    attention_fixture("attn_cfg4_fp8_ragged_b2_s384.npz", 1004, 2, 64, 8, 384, 64, 0, True, [383, 256], False)
    attention_fixture("attn_cfg4_fp8_window_b2_s384.npz", 1014, 2, 64, 8, 384, 64, 128, True, [383, 256], False)
    gemm_fixture("gemm_fp8_blk256_g4_k256_n512_swiglu.npz", 1003, [3, 0, 5, 1], 256, 512, True, (256, 256), True, False)
    gemm_fixture("gemm_fp8_perchannel_g4_k256_n512_bias.npz", 1013, [1, 2, 0, 4], 256, 512, True, (256, 1), False, True)
    gemm_fixture("gemm_bf16_g3_k128_n256_swiglu_bias.npz", 1023, [2, 0, 3], 128, 256, False, None, True, True)
    gemm_fixture("gemm_fp8_dense_g1_k512_n256.npz", 1033, [20], 512, 256, True, (256, 256), False, False)
    tables_fixture()
    routing_fixture()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
