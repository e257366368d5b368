"""CPU restatement of one decode step of the reference model (lyra/model.py:734-793 in Mode.DECODE).

TEST INFRASTRUCTURE ONLY (parity checker for lyra_amd.model and the timed CPU baseline of bench.py).
It chains the oracle pieces exactly in the order the reference calls them:
embedding -> per layer [attention_apply (model.py:284-374), mlp_apply (:498-567 / :608-636)] -> final norm ->
LM head.  bf16 arrays are float32 arrays holding bf16-representable values; every point where the JAX code
holds a bf16 array is rounded with ``bf16_round``.  The heavy contractions (attention, grouped matmul) run in
the threaded C restatement when ``use_c`` is set (bench baseline, large parity cases), else in NumPy.
"""
from __future__ import annotations

import functools
import math

import numpy as np

from oracle import clib
from oracle import lyra_oracle as O

R = O.bf16_round


def _gemm(lhs, w, sizes, *, swiglu=False, beta=1.702, limit=7.0, use_c=False, out_bf16=True, bias=None, inner="ref", fmt=1):
    """decode_gemm / quant.dot: w is float32 [G,K,N] (bf16 weights) or (qval, scale, block); bias [G,N] float32 or None.
    inner="ref": dequantised weights are rounded to bf16 before the product, as the JAX code holds them (quant.py:85);
    inner="fp32": the product is taken on the exact dequantised values; either way the result is one bf16 array.
    fmt: the 1-byte format of quantised weights (1 e4m3fn, 2 e5m2)."""
    ref = inner == "ref"
    if isinstance(w, tuple):
        q, s, block = w
        if use_c:
            y = clib.decode_gemm(O.bf16_bits(lhs), q, s, block, sizes, bias, fused_swiglu=swiglu, beta=beta, limit=limit, ref_rounding=ref,
                                 fp8_format=fmt)
        else:
            y = O.decode_gemm_reference(lhs, (q, s), sizes, block=block, bias=bias, fused_swiglu=swiglu, swiglu_beta=beta, swiglu_limit=limit,
                                        mode="ref" if ref else "fp32", fp8_format=fmt)
        return R(y) if out_bf16 else y
    if use_c:
        y = clib.decode_gemm(O.bf16_bits(lhs), O.bf16_bits(w), None, None, sizes, bias, fused_swiglu=swiglu, beta=beta, limit=limit, ref_rounding=out_bf16)
    else:
        y = O.decode_gemm_reference(lhs, w, sizes, bias=bias, fused_swiglu=swiglu, swiglu_beta=beta, swiglu_limit=limit, mode="ref" if out_bf16 else "fp32")
    return y


def _bias(b):
    """acast(bias, compute_dtype) (lyra/nn/params.py:47-48): a float32 parameter used as a bf16 array."""
    return None if b is None else R(np.asarray(b, dtype=np.float32))


def decode_step(tokens, weights, cache, pos, cfg, *, use_c=False, router_margins=None, hidden_out=None, inner="ref", layer_offset=0):
    """tokens [B] int; weights/cache: dicts of NumPy arrays mirroring lyra_amd.model; pos: int.
    router_margins: optional list; receives one float32 [B] array per MoE layer, the gap between the last router logit
    that is selected and the first that is not (top-k is discontinuous: a row with a tiny gap is not a parity case).

    cache["k"][l], cache["v"][l]: float32 [B,K,S,H] (bf16 cache) or (qval uint8, scale f32 [B,K,S,1]); updated in
    place.  Returns float32 logits [B, padded_vocab] with -inf beyond vocab_size.
    inner: "ref" rounds inside the two operators wherever the reference's plain-JAX path holds a bf16 array (dequantised
    cache and weights, the logits q.k); "fp32" computes each operator exactly in float32 from its (bf16 / FP8) inputs and
    rounds only its output - the form the acceptance tolerances of the kernels are stated against.
    hidden_out: optional list; receives the residual stream [B, C] as it enters every layer, then as it leaves the last
    one (before the final norm): n_layers + 1 arrays.
    layer_offset: index, in the whole model, of the first layer of ``weights["layers"]`` (even layers have the sliding
    window, model.py:337): lets a caller run a few layers of a deep model on their own, fed that layer's input as "emb".
    """
    fmt = 2 if str(getattr(cfg, "gemm_dtype", "")).endswith("e5m2") else 1  # the format of every FP8 array of the model (one config field)
    gemm = functools.partial(_gemm, fmt=fmt)
    B = tokens.shape[0]
    C, H, N, K = cfg.n_embd, cfg.head_dim, cfg.n_attn_heads, cfg.n_kv_heads
    cos_t, sin_t = O.rope_tables(cfg.seq_len, H, cfg.rope_base, cfg.rope_scale, cfg.ntk_alpha, cfg.ntk_beta)
    cos, sin = cos_t[pos], sin_t[pos]
    one = np.array([B], np.int32)
    h = R(weights["emb"][tokens])
    for idx, lw in enumerate(weights["layers"], layer_offset):
        if hidden_out is not None:
            hidden_out.append(h.copy())
        # ---- attention_apply ----
        a = lw["attn"]
        hn = R(O.rms_norm(h, a["norm_scale"], cfg.norm_eps))
        qkv = gemm(hn, a["qkv"], one, use_c=use_c, inner=inner)
        if a.get("qkv_bias") is not None:  # model.py:310-313
            qkv = R(qkv + _bias(a["qkv_bias"]))
        q, k, v = np.split(qkv, [N * H, (N + K) * H], axis=-1)
        q, k, v = q.reshape(B, N, H), k.reshape(B, K, H), v.reshape(B, K, H)
        if a["qnorm_scale"] is not None:
            q = R(O.rms_norm(q, a["qnorm_scale"], cfg.norm_eps))
            k = R(O.rms_norm(k, a["knorm_scale"], cfg.norm_eps))
        q, k = R(O.rotate(q, cos, sin)), R(O.rotate(k, cos, sin))
        ck, cv = cache["k"][idx - layer_offset], cache["v"][idx - layer_offset]
        if isinstance(ck, tuple):  # qupdate: quantise the new token with block (1, H) and write it at pos
            for (cq, cs), new in ((ck, k), (cv, v)):
                nq, ns = O.quantize(new[:, :, None, :], (1, H), fmt)
                cq[:, :, pos : pos + 1] = nq
                cs[:, :, pos : pos + 1] = ns
        else:
            ck[:, :, pos] = k
            cv[:, :, pos] = v
        sw = cfg.sliding_window if idx % 2 == 0 else 0
        gate = None
        if a["sdpa_gate"] is not None:
            gate = R((2.0 / (1.0 + np.exp(-(hn.astype(np.float32) @ a["sdpa_gate"])))).astype(np.float32))
        ref = inner == "ref"
        g_in = gate if ref else None  # inner="fp32": the operator's exact output is rounded once, then gated (model.py:347)
        if use_c:
            if isinstance(ck, tuple):
                t = clib.decode_attention(O.bf16_bits(q[:, :, None, :]), ck[0], cv[0], ck[1][..., 0], cv[1][..., 0], a["sinks"],
                                          pos, g_in, H**-0.5, sw, ref_rounding=ref, fp8_format=fmt)
            else:
                t = clib.decode_attention(O.bf16_bits(q[:, :, None, :]), O.bf16_bits(ck), O.bf16_bits(cv), None, None, a["sinks"],
                                          pos, g_in, H**-0.5, sw, ref_rounding=ref)
        else:
            t = O.decode_attention_reference(q[:, :, None, :], ck, cv, a["sinks"], H**-0.5, sw, pos, mode="ref" if ref else "fp32", gate=g_in,
                                             fp8_format=fmt)
        if not ref and gate is not None:
            t = R(R(t) * gate[:, :, None, None])
        t = R(t.reshape(B, N, H))
        if a.get("xsa_alpha") is not None:  # model.py:351-363, on the new token's value rows as projected (not as cached)
            t = O.xsa(t, v, a["xsa_alpha"], mode="ref")
        t = gemm(t.reshape(B, N * H), a["out"], one, use_c=use_c, inner=inner)
        if a.get("out_bias") is not None:  # model.py:367-368
            t = R(t + _bias(a["out_bias"]))
        t = R(t * np.float32(cfg.residual_scale))
        h = R(h + t)
        # ---- mlp_apply ----
        m = lw["mlp"]
        xn = R(O.rms_norm(h, m["norm_scale"], cfg.norm_eps))
        if "router" in m:
            logits = xn.astype(np.float32) @ m["router"]
            if m["router_bias"] is not None:
                logits = logits + m["router_bias"]
            if router_margins is not None:
                srt = np.sort(logits, axis=-1)[:, ::-1]
                kr = cfg.n_active_routed_experts
                router_margins.append((srt[:, kr - 1] - srt[:, kr]).astype(np.float32) if kr < srt.shape[1] else np.full(B, np.inf, np.float32))
            scores, active_map, groups = O.route_tokens(logits, cfg.n_active_routed_experts, cfg.n_routed_experts, cfg.n_shared_experts)
            topk = cfg.n_active_experts
            perm, dest = O.bpermute(active_map, groups, cfg.n_experts)
            t = xn[perm // topk]
            t = gemm(t, m["mlp_up"], groups, swiglu=True, beta=cfg.swiglu_beta, limit=cfg.swiglu_limit, use_c=use_c,
                      bias=_bias(m.get("mlp_up_bias")), inner=inner)
            t = gemm(R(t), m["mlp_down"], groups, use_c=use_c, bias=_bias(m.get("mlp_down_bias")), inner=inner)
            t = R(O.combine(R(t), scores, dest))
            t = R(t * np.float32(cfg.residual_scale))
            h = R(h + t)
        else:
            if ref and m.get("mlp_up_bias") is not None:
                # model.py:613-616: the product is a bf16 array, the bias is added to it in bf16, SwiGLU follows
                # (inner="fp32", like the kernels, adds the bias to the float32 product inside the fused epilogue)
                t = gemm(xn, m["mlp_up"], one, use_c=use_c, inner=inner)
                t = R(t + _bias(m["mlp_up_bias"])[0])
                t = R(O.swiglu(t, cfg.swiglu_beta, cfg.swiglu_limit))
            else:
                t = gemm(xn, m["mlp_up"], one, swiglu=True, beta=cfg.swiglu_beta, limit=cfg.swiglu_limit, use_c=use_c,
                          bias=_bias(m.get("mlp_up_bias")), inner=inner)
            t = gemm(R(t), m["mlp_down"], one, use_c=use_c, inner=inner)
            if m.get("mlp_down_bias") is not None:  # model.py:629-630
                t = R(t + _bias(m["mlp_down_bias"])[0])
            t = R(t * np.float32(cfg.dense_residual_scale))
            h = R(h + t)
    if hidden_out is not None:
        hidden_out.append(h.copy())
    h = R(O.rms_norm(h, weights["norm_scale"], cfg.norm_eps))
    logits = gemm(h, weights["unemb_t"], one, use_c=use_c, out_bf16=False)
    logits[:, cfg.vocab_size :] = -np.inf
    return logits


def weights_to_numpy(model, cfg):
    """lyra_amd.model.ModelWeights (torch) -> the dict layout decode_step takes."""
    import torch

    from lyra_amd.nn.quant import QArray

    def conv(w):
        if isinstance(w, QArray):
            return (w.qval.view(torch.uint8).cpu().numpy(), w.scale.float().cpu().numpy(), tuple(w.block))
        return w.float().cpu().numpy()

    f = lambda t: None if t is None else t.float().cpu().numpy()
    layers = []
    for lw in model.layers:
        a = lw.attn
        attn = dict(qkv=conv(a.qkv), out=conv(a.out), sinks=f(a.sinks), norm_scale=f(a.norm_scale), qnorm_scale=f(a.qnorm_scale),
                    knorm_scale=f(a.knorm_scale), sdpa_gate=f(a.sdpa_gate), xsa_alpha=f(a.xsa_alpha), qkv_bias=f(a.qkv_bias),
                    out_bias=f(a.out_bias))
        m = lw.mlp
        mlp = dict(mlp_up=conv(m.mlp_up), mlp_down=conv(m.mlp_down), norm_scale=f(m.norm_scale),
                   mlp_up_bias=f(m.mlp_up_bias), mlp_down_bias=f(m.mlp_down_bias))
        if hasattr(m, "router"):
            mlp.update(router=f(m.router), router_bias=f(m.router_bias))
        layers.append(dict(attn=attn, mlp=mlp))
    return dict(emb=f(model.emb), unemb_t=f(model.unemb_t), norm_scale=f(model.norm_scale), layers=layers)


def cache_to_numpy(cache):
    import torch

    from lyra_amd.nn.quant import QArray

    def conv(c):
        if isinstance(c, QArray):
            return (c.qval.view(torch.uint8).cpu().numpy().copy(), c.scale.float().cpu().numpy().copy())
        return c.float().cpu().numpy().copy()

    return dict(k=[conv(l.k) for l in cache.layers], v=[conv(l.v) for l in cache.layers])
