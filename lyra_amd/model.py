"""Decode-mode model driver: the callers of the two decode kernels (lyra/model.py of the reference).

Only ``Mode.DECODE`` with one new token per sequence is implemented: ``attention_apply`` (model.py:284-374),
``route_tokens`` / ``bpermute`` / ``moe_apply`` (model.py:451-567), ``dense_mlp_apply`` (model.py:608-636) and
``model_apply`` (model.py:734-793).  Everything runs on torch device tensors; the attention and every
matmul (projections, experts, LM head) go through the HIP kernels of this package.  The KV cache is updated
in place (the reference returns a new cache object; a functional copy of a multi-GB cache per token is the
one thing a decode loop cannot afford), everything else is a pure function of its inputs.
"""
from __future__ import annotations

import os

import math
from dataclasses import dataclass, field, replace
from functools import lru_cache

import numpy as np
import torch

from lyra_amd.kernels.common import Implementation
from lyra_amd.kernels.op import Mode, attn_op, gmm_op
from lyra_amd.nn.quant import QArray, dot, quantize

PADDED_VOCAB_SIZE = 204800  # lyra/tokenizer.py:3


def interleaved_moe(layers: int, *, every: int, first: int) -> tuple[str, ...]:
    """lyra/nn/params.py:128-129 (layers are numbered from 1)."""
    return tuple("moe" if layer >= first and (layer - first) % every == 0 else "dense" for layer in range(1, layers + 1))


def moe_outer_dense(layers: int, start_dense: int = 0, end_dense: int = 0) -> tuple[str, ...]:
    """lyra/nn/params.py:132-133."""
    return ("dense",) * start_dense + ("moe",) * (layers - start_dense - end_dense) + ("dense",) * end_dense


@dataclass(frozen=True)
class ModelConfig:
    """The decode-relevant fields of lyra/model.py:39-129, same names and defaults."""

    name: str
    seq_len: int = 4096
    n_embd: int = 2048
    n_layers: int = 16
    vocab_size: int = 201088
    tie_embeddings: bool = True
    padded_vocab_size: int = PADDED_VOCAB_SIZE
    seed: int = 42
    head_dim: int = 128
    n_attn_heads: int = 16
    n_kv_heads: int = 4
    sliding_window: int = 128
    use_qk_norm: bool = True
    use_sdpa_output_gate: bool = False
    use_learned_xsa: bool = False
    use_qkv_bias: bool = False
    use_attn_out_bias: bool = False
    use_mlp_bias: bool = False
    mlp_map: tuple[str, ...] = ()
    n_routed_experts: int = 15
    n_shared_experts: int = 1
    n_active_experts: int = 4
    expert_mlp_widening: float = 2.0
    dense_mlp_widening: float = 3.0
    swiglu_beta: float = 1.702
    swiglu_limit: float = 7.0
    use_router_bias: bool = True
    rope_base: float = 150000.0
    rope_scale: float = 1.0
    ntk_alpha: float = 1.0
    ntk_beta: float = 32.0
    gemm_dtype: torch.dtype = torch.bfloat16
    quantize_attn: bool = False
    quantize_mlp: bool = False
    quantize_cache: bool = False
    quant_block: tuple[int, int] = (256, 256)
    per_channel_scales: bool = False  # FP8 weights with one scale per output channel (block (K, 1)) instead of quant_block
    mode: Mode = Mode.DECODE
    implementation: Implementation = "auto"
    fused_glue: bool = True  # run norms, RoPE, cache append, routing and residual adds as fused HIP launches
    sample_topk: int = 4
    sample_temperature: float = 0.8
    norm_eps: float = 1e-5
    w_std: float = 0.02  # synthetic weights ~ N(0, w_std)

    @property
    def n_experts(self) -> int:
        return self.n_routed_experts + self.n_shared_experts

    @property
    def n_active_routed_experts(self) -> int:
        return self.n_active_experts - self.n_shared_experts

    @property
    def residual_scale(self) -> float:
        return 1.0 / math.sqrt(2.0 * self.n_layers)

    @property
    def dense_residual_scale(self) -> float:
        return self.residual_scale * (self.n_active_experts**-0.5 if "moe" in self.mlp_map else 1.0)

    @property
    def expert_hidden(self) -> int:
        return int(self.n_embd * self.expert_mlp_widening) // 2

    @property
    def dense_hidden(self) -> int:
        return int(self.n_embd * self.dense_mlp_widening) // 2


# lyra/variants.py:7-61 (decode-relevant fields)
lyra_dev = ModelConfig(name="Lyra Dev", seq_len=256, n_embd=256, n_layers=4, n_attn_heads=2, n_kv_heads=1, head_dim=64,
                       sliding_window=0, n_routed_experts=7, n_active_experts=2, vocab_size=1000, padded_vocab_size=1024,
                       mlp_map=interleaved_moe(layers=4, first=2, every=2))
lyra_small = ModelConfig(name="Lyra Small", use_sdpa_output_gate=True, mlp_map=interleaved_moe(layers=16, every=4, first=4))
lyra_medium = ModelConfig(name="Lyra Medium", n_embd=4096, n_layers=32, tie_embeddings=False, n_attn_heads=32, n_kv_heads=8,
                          use_sdpa_output_gate=True, use_learned_xsa=True, mlp_map=interleaved_moe(32, first=4, every=4),
                          n_routed_experts=31)
lyra_max = replace(lyra_medium, name="Lyra Max", mlp_map=moe_outer_dense(32, start_dense=2), n_routed_experts=63,
                   dense_mlp_widening=4.0)
# lyra/variants.py:62-80: every layer an expert layer, no shared expert, no QK norm, biases on every projection, YaRN
gpt_oss_20b = ModelConfig(name="GPT-OSS 20B", rope_scale=32.0, n_embd=2880, n_layers=24, head_dim=64, n_attn_heads=64,
                          n_kv_heads=8, mlp_map=("moe",) * 24, n_routed_experts=32, n_shared_experts=0, n_active_experts=4,
                          tie_embeddings=False, use_qk_norm=False, use_qkv_bias=True, use_attn_out_bias=True, use_mlp_bias=True)
MODEL_VARIANTS = {"dev": lyra_dev, "lyra-small": lyra_small, "lyra-medium": lyra_medium, "lyra-max": lyra_max,
                  "gpt-oss-20b": gpt_oss_20b}


def apply_inference_overrides(cfg: ModelConfig, *, fp8: bool = False, fp8_attn: bool = False, per_channel: bool = False) -> ModelConfig:
    """lyra/generate.py:31-38: --fp8 turns on FP8 MLP weights and an FP8 KV cache.

    ``fp8_attn`` additionally quantises the attention projections (``quantize_attn``, model.py:276-281) and
    ``per_channel`` selects per-output-channel weight scales; both are off in the reference's serve path.
    """
    if fp8:
        cfg = replace(cfg, gemm_dtype=torch.float8_e4m3fn, quantize_mlp=True, quantize_cache=True)
    if fp8_attn:
        cfg = replace(cfg, gemm_dtype=torch.float8_e4m3fn, quantize_attn=True)
    if per_channel:
        cfg = replace(cfg, per_channel_scales=True)
    return cfg


# ---- RoPE and norm -----------------------------------------------------------------------------------
@lru_cache(maxsize=8)
def precompute_freq_cis(cfg: ModelConfig) -> tuple[np.ndarray, np.ndarray]:
    """lyra/model.py:160-180 (float64 angles, float32 tables; YaRN branch for rope_scale > 1)."""
    positions = np.arange(int(cfg.seq_len * cfg.rope_scale), dtype=np.float64)
    inv_freq = 1.0 / (cfg.rope_base ** (np.arange(0, cfg.head_dim, 2, dtype=np.float64) / cfg.head_dim))
    concentration = 1.0
    if cfg.rope_scale > 1.0:
        concentration = 0.1 * math.log(cfg.rope_scale) + 1.0
        dim_half = cfg.head_dim / 2.0
        log_base = math.log(cfg.rope_base) ** -1.0
        low = dim_half * math.log(cfg.seq_len / (cfg.ntk_beta * 2.0 * math.pi)) * log_base
        high = dim_half * math.log(cfg.seq_len / (cfg.ntk_alpha * 2.0 * math.pi)) * log_base
        ramp = 1.0 - np.clip((np.arange(int(dim_half), dtype=np.float64) - low) / (high - low), 0.0, 1.0)
        inv_freq = (1.0 - ramp) * (inv_freq / cfg.rope_scale) + ramp * inv_freq
    angles = np.einsum("i,j->ij", positions, inv_freq)
    return (np.cos(angles) * concentration).astype(np.float32), (np.sin(angles) * concentration).astype(np.float32)


def rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """lyra/model.py:183-186: x bf16 times float32 tables promotes to float32, result cast back."""
    x1, x2 = x.to(torch.float32).chunk(2, dim=-1)
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)


def rms_norm(x: torch.Tensor, scale: torch.Tensor, eps: float) -> torch.Tensor:
    """lyra/model.py:189-191."""
    t = x.to(torch.float32)
    return (t * torch.rsqrt(t.pow(2).mean(dim=-1, keepdim=True) + eps) * scale).to(x.dtype)


# ---- weights -----------------------------------------------------------------------------------------
@dataclass
class AttentionWeights:
    qkv: torch.Tensor | QArray  # [C, (N + 2K) H]: q, k, v projections side by side (one launch instead of three)
    out: torch.Tensor | QArray  # [N H, C]
    sinks: torch.Tensor         # [N] f32
    norm_scale: torch.Tensor    # [C] f32
    qnorm_scale: torch.Tensor | None
    knorm_scale: torch.Tensor | None
    sdpa_gate: torch.Tensor | None  # [C, N] f32
    xsa_alpha: torch.Tensor | None = None  # [N] f32 (use_learned_xsa, model.py:269)
    qkv_bias: torch.Tensor | None = None   # [(N + 2K) H] f32: q, k and v biases side by side (use_qkv_bias, model.py:258-262)
    out_bias: torch.Tensor | None = None   # [C] f32 (use_attn_out_bias)


@dataclass
class MoEWeights:
    router: torch.Tensor            # [C, n_routed] f32
    router_bias: torch.Tensor | None
    mlp_up: torch.Tensor | QArray   # [E, C, 2*hidden]   (gate half first: lyra/model.py:494-495)
    mlp_down: torch.Tensor | QArray  # [E, hidden, C]
    norm_scale: torch.Tensor
    mlp_up_bias: torch.Tensor | None = None    # [E, 2*hidden] f32 (use_mlp_bias, model.py:399-402)
    mlp_down_bias: torch.Tensor | None = None  # [E, C] f32


@dataclass
class DenseMLPWeights:
    mlp_up: torch.Tensor | QArray    # [1, C, 2*hidden]
    mlp_down: torch.Tensor | QArray  # [1, hidden, C]
    norm_scale: torch.Tensor
    mlp_up_bias: torch.Tensor | None = None    # [1, 2*hidden] f32
    mlp_down_bias: torch.Tensor | None = None  # [1, C] f32


@dataclass
class LayerWeights:
    attn: AttentionWeights
    mlp: MoEWeights | DenseMLPWeights


@dataclass
class ModelWeights:
    emb: torch.Tensor         # [V_padded, C] bf16
    unemb_t: torch.Tensor     # [1, C, V_padded] bf16: LM head weight laid out for the decode matmul
    norm_scale: torch.Tensor  # [C] f32
    layers: list[LayerWeights] = field(default_factory=list)
    # [1, V_padded] f32: 0 for real tokens, -inf for the padding of the vocabulary.  Passed to the LM-head matmul as its
    # bias, it makes `logits[:, vocab_size:] = -inf` (lyra/model.py:789) part of that launch.
    vocab_mask: torch.Tensor | None = None


def _maybe_quantize(w: torch.Tensor, cfg: ModelConfig, enabled: bool):
    """model.py:154-156: block (gcd(K, bk), gcd(N, bn)) of quant_block, or per-output-channel (K, 1)."""
    if not enabled:
        return w
    K, N = w.shape[-2], w.shape[-1]
    block = (K, 1) if cfg.per_channel_scales else (math.gcd(K, cfg.quant_block[0]), math.gcd(N, cfg.quant_block[1]))
    return quantize(w, cfg.gemm_dtype, block)


def init_weights(cfg: ModelConfig, device, seed: int | None = None) -> ModelWeights:
    """Random weights ~ N(0, w_std) in the reference's shapes (model.py:252-274,389-404,582-592,673-683); norm
    scales 1, sinks and router bias ~ N(0, 1) / 0 so that every code path is exercised by synthetic runs."""
    g = torch.Generator(device=device)
    g.manual_seed(cfg.seed if seed is None else seed)
    C, H, N, K = cfg.n_embd, cfg.head_dim, cfg.n_attn_heads, cfg.n_kv_heads

    def rnd(*shape, std=cfg.w_std, dtype=torch.bfloat16):
        return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * std).to(dtype)

    ones = lambda n: torch.ones(n, device=device, dtype=torch.float32)
    layers = []
    for idx in range(cfg.n_layers):
        attn = AttentionWeights(
            qkv=_maybe_quantize(rnd(1, C, (N + 2 * K) * H), cfg, cfg.quantize_attn),
            out=_maybe_quantize(rnd(1, N * H, C), cfg, cfg.quantize_attn),
            sinks=rnd(N, std=1.0, dtype=torch.float32),
            norm_scale=ones(C),
            qnorm_scale=ones(H) if cfg.use_qk_norm else None,
            knorm_scale=ones(H) if cfg.use_qk_norm else None,
            sdpa_gate=rnd(C, N, dtype=torch.float32) if cfg.use_sdpa_output_gate else None,
            xsa_alpha=rnd(N, std=1.0, dtype=torch.float32) if cfg.use_learned_xsa else None,
            qkv_bias=rnd((N + 2 * K) * H, std=0.5, dtype=torch.float32) if cfg.use_qkv_bias else None,
            out_bias=rnd(C, std=0.5, dtype=torch.float32) if cfg.use_attn_out_bias else None,
        )
        if cfg.mlp_map[idx] == "moe":
            E, Hd = cfg.n_experts, cfg.expert_hidden
            mlp = MoEWeights(
                router=rnd(C, cfg.n_routed_experts, std=0.5 / math.sqrt(C), dtype=torch.float32),
                router_bias=torch.zeros(cfg.n_routed_experts, device=device) if cfg.use_router_bias else None,
                mlp_up=_maybe_quantize(rnd(E, C, 2 * Hd), cfg, cfg.quantize_mlp),
                mlp_down=_maybe_quantize(rnd(E, Hd, C), cfg, cfg.quantize_mlp),
                norm_scale=ones(C),
                mlp_up_bias=rnd(E, 2 * Hd, std=0.5, dtype=torch.float32) if cfg.use_mlp_bias else None,
                mlp_down_bias=rnd(E, C, std=0.5, dtype=torch.float32) if cfg.use_mlp_bias else None,
            )
        else:
            Hd = cfg.dense_hidden
            mlp = DenseMLPWeights(
                mlp_up=_maybe_quantize(rnd(1, C, 2 * Hd), cfg, cfg.quantize_mlp),
                mlp_down=_maybe_quantize(rnd(1, Hd, C), cfg, cfg.quantize_mlp),
                norm_scale=ones(C),
                mlp_up_bias=rnd(1, 2 * Hd, std=0.5, dtype=torch.float32) if cfg.use_mlp_bias else None,
                mlp_down_bias=rnd(1, C, std=0.5, dtype=torch.float32) if cfg.use_mlp_bias else None,
            )
        layers.append(LayerWeights(attn=attn, mlp=mlp))
    emb = rnd(cfg.padded_vocab_size, C)
    unemb = emb if cfg.tie_embeddings else rnd(cfg.padded_vocab_size, C)
    vocab_mask = torch.zeros(1, cfg.padded_vocab_size, dtype=torch.float32, device=device)
    vocab_mask[:, cfg.vocab_size :] = float("-inf")
    return ModelWeights(emb=emb, unemb_t=unemb.t().contiguous()[None], norm_scale=ones(C), layers=layers, vocab_mask=vocab_mask)


# ---- KV cache ----------------------------------------------------------------------------------------
@dataclass
class LayerCache:
    k: torch.Tensor | QArray
    v: torch.Tensor | QArray


@dataclass
class ModelCache:
    layers: list[LayerCache]
    pos: torch.Tensor  # int32 scalar on the device: index the next token is written at


def init_cache(cfg: ModelConfig, batch: int, length: int, device) -> ModelCache:
    """lyra/generate.py:93-96 + ModelCache.quantize (model.py:221-226): zeros, FP8 block (1, H) when quantised."""
    shape = (batch, cfg.n_kv_heads, length, cfg.head_dim)

    def buf():
        if cfg.quantize_cache:
            return QArray(torch.zeros(shape, dtype=torch.uint8, device=device).view(cfg.gemm_dtype),
                          torch.ones((*shape[:-1], 1), dtype=torch.float32, device=device), (1, cfg.head_dim))
        return torch.zeros(shape, dtype=torch.bfloat16, device=device)

    return ModelCache(layers=[LayerCache(buf(), buf()) for _ in range(cfg.n_layers)],
                      pos=torch.zeros((), dtype=torch.int32, device=device))


def cache_update(cache: LayerCache, k: torch.Tensor, v: torch.Tensor, pos: torch.Tensor) -> LayerCache:
    """lyra/model.py:204-212 / quant.py:89-98 for one new token, written in place at ``pos`` (device scalar).

    A position outside the cache writes nothing, as in the HIP kernels that append (the index lives on the device and
    ``index_copy_`` does not check it: the row at the clamped index is read and written back unchanged instead)."""
    S = (cache.k.qval if isinstance(cache.k, QArray) else cache.k).shape[2]
    p64 = pos.to(torch.int64).reshape(1)
    inside = (p64 >= 0) & (p64 < S)
    idx = p64.clamp(0, S - 1)

    def put(dst: torch.Tensor, new: torch.Tensor):
        dst.index_copy_(2, idx, torch.where(inside, new, dst.index_select(2, idx)))

    for dst, new in ((cache.k, k), (cache.v, v)):
        if isinstance(dst, QArray):
            q = quantize(new, dst.dtype, dst.block, dst.stype)
            put(dst.qval.view(torch.uint8), q.qval.view(torch.uint8))
            put(dst.scale, q.scale)
        else:
            put(dst, new.to(dst.dtype))
    return cache


# ---- layers ------------------------------------------------------------------------------------------
def _dense(x: torch.Tensor, w, cfg: ModelConfig, *, fused_swiglu=False, out_f32=False, bias=None) -> torch.Tensor:
    """quant.dot for a [B, C] activation (lyra/nn/quant.py:106-108) = the one-group decode matmul.  With a SwiGLU or a
    float32 bias behind it the operator's fused epilogue does both (the decode_gemm operator itself)."""
    if not fused_swiglu and bias is None:
        w2 = QArray(w.qval[0], w.scale[0], w.block) if isinstance(w, QArray) else w[0]
        return dot(x, w2, preferred_element_type=torch.float32 if out_f32 else None, implementation=cfg.implementation)
    gmm = gmm_op(cfg.mode, cfg.implementation)
    sizes = torch.full((1,), x.shape[0], dtype=torch.int32, device=x.device)
    lhs = x.to(torch.float32) if out_f32 else x
    return gmm(lhs, w, sizes, bias=bias, fused_swiglu=fused_swiglu, swiglu_beta=cfg.swiglu_beta, swiglu_limit=cfg.swiglu_limit,
               quant_dtype=cfg.gemm_dtype if isinstance(w, QArray) else None)


def attention_apply(x, w: AttentionWeights, idx: int, pos, cos, sin, cache: LayerCache, cfg: ModelConfig):
    """lyra/model.py:284-374 for T == 1; x [B, C] bf16, cos/sin [H/2] f32 of this position."""
    B, C = x.shape
    H, N, K = cfg.head_dim, cfg.n_attn_heads, cfg.n_kv_heads
    h = rms_norm(x, w.norm_scale, cfg.norm_eps)
    qkv = _dense(h, w.qkv, cfg)
    if w.qkv_bias is not None:  # :310-313, bf16 array + bf16 bias
        qkv = qkv + w.qkv_bias.to(qkv.dtype)
    q, k, v = qkv.split([N * H, K * H, K * H], dim=-1)
    q, k, v = q.reshape(B, N, H), k.reshape(B, K, H), v.reshape(B, K, H)
    if w.qnorm_scale is not None and w.knorm_scale is not None:
        q = rms_norm(q, w.qnorm_scale, cfg.norm_eps)
        k = rms_norm(k, w.knorm_scale, cfg.norm_eps)
    q, k = rotate(q, cos, sin), rotate(k, cos, sin)
    cache = cache_update(cache, k[:, :, None, :], v[:, :, None, :], pos)
    sliding_window = cfg.sliding_window if idx % 2 == 0 else 0  # even layers local, odd global (:337)
    gate = None
    if w.sdpa_gate is not None:  # :343-347, fused into the attention epilogue
        gate = (2.0 * torch.sigmoid(h.to(torch.float32) @ w.sdpa_gate)).to(x.dtype)
    attn = attn_op(cfg.mode, cfg.implementation)
    xsa_v = None
    if w.xsa_alpha is not None:  # :353-354: the new token's value rows (not their cached, quantised copy) at unit length
        v32 = v.to(torch.float32)
        xsa_v = (v32 * torch.rsqrt(v32.pow(2).sum(dim=-1, keepdim=True) + 1e-10)).to(x.dtype)
    t = attn(q[:, :, None, :], cache.k, cache.v, w.sinks, H**-0.5, sliding_window, pos, gate=gate, xsa_v=xsa_v, xsa_alpha=w.xsa_alpha)
    t = _dense(t.reshape(B, N * H), w.out, cfg)
    if w.out_bias is not None:  # :367-368
        t = t + w.out_bias.to(t.dtype)
    t = t * cfg.residual_scale
    return (x + t).to(x.dtype), cache


def route_tokens(t: torch.Tensor, w: MoEWeights, cfg: ModelConfig):
    """lyra/model.py:451-480 (inference part): f32 logits, stable top-k, softmax over the selected, shared experts
    appended with score 1, tokens per expert."""
    tokens = t.shape[0]
    routed, shared = cfg.n_routed_experts, cfg.n_shared_experts
    logits = t.to(torch.float32) @ w.router
    if w.router_bias is not None:
        logits = logits + w.router_bias
    top, indices = torch.sort(logits, dim=-1, descending=True, stable=True)  # lax.top_k: ties to the lower index
    top, indices = top[:, : cfg.n_active_routed_experts], indices[:, : cfg.n_active_routed_experts]
    scores = torch.softmax(top, dim=-1)
    if shared:
        shared_idx = torch.arange(routed, cfg.n_experts, device=t.device).expand(tokens, shared)
        indices = torch.cat([indices, shared_idx], dim=-1)
        scores = torch.cat([scores, torch.ones(tokens, shared, device=t.device)], dim=-1)
    active_map = indices.reshape(-1)
    groups = torch.zeros(cfg.n_experts, dtype=torch.int32, device=t.device)
    groups.scatter_add_(0, active_map, torch.ones_like(active_map, dtype=torch.int32))
    return scores, active_map, groups


def bpermute(expert_ids: torch.Tensor):
    """lyra/model.py:483-491: stable counting sort of the assignments by expert -> (permutation, destinations)."""
    permutation = torch.sort(expert_ids, stable=True).indices
    destinations = torch.empty_like(permutation)
    destinations[permutation] = torch.arange(permutation.numel(), device=permutation.device)
    return permutation, destinations


def moe_apply(x, w: MoEWeights, cfg: ModelConfig, groups_out: list | None = None):
    """lyra/model.py:498-567 without expert parallelism."""
    B, C = x.shape
    gmm = gmm_op(cfg.mode, cfg.implementation)
    xn = rms_norm(x, w.norm_scale, cfg.norm_eps)
    scores, active_map, groups = route_tokens(xn, w, cfg)
    if groups_out is not None:
        groups_out.append(groups)
    topk = cfg.n_active_experts
    permute_map, unpermute_map = bpermute(active_map)
    t = xn[permute_map // topk]
    qd = cfg.gemm_dtype if isinstance(w.mlp_up, QArray) else None
    bf = lambda bias: None if bias is None else bias.to(x.dtype).to(torch.float32)  # acast(bias, compute_dtype), :527-528
    t = gmm(t, w.mlp_up, groups, bias=bf(w.mlp_up_bias), fused_swiglu=True, swiglu_beta=cfg.swiglu_beta,
            swiglu_limit=cfg.swiglu_limit, quant_dtype=qd)
    t = gmm(t, w.mlp_down, groups, bias=bf(w.mlp_down_bias), quant_dtype=qd)
    t = torch.einsum("fkc,fk->fc", t[unpermute_map].reshape(B, topk, C).to(torch.float32), scores).to(x.dtype)  # :557
    t = t * cfg.residual_scale
    return x + t


def dense_mlp_apply(x, w: DenseMLPWeights, cfg: ModelConfig):
    """lyra/model.py:608-636 (SwiGLU fused into the up projection's epilogue)."""
    t = rms_norm(x, w.norm_scale, cfg.norm_eps)
    bf = lambda bias: None if bias is None else bias.to(x.dtype).to(torch.float32)
    t = _dense(t, w.mlp_up, cfg, fused_swiglu=True, bias=bf(w.mlp_up_bias))
    t = _dense(t, w.mlp_down, cfg)
    if w.mlp_down_bias is not None:  # :629-630
        t = t + w.mlp_down_bias[0].to(t.dtype)
    t = t * cfg.dense_residual_scale
    return (x + t).to(x.dtype)


# ---- the same layers with every step between the two hot kernels as one fused HIP launch --------------------
def _one_group(rows: int, device) -> torch.Tensor:
    key = (rows, str(device))
    if key not in _ONE_GROUP:
        _ONE_GROUP[key] = torch.full((1,), rows, dtype=torch.int32, device=device)
    return _ONE_GROUP[key]


_ONE_GROUP: dict = {}
_SEPARATE_COMBINE = os.environ.get("LYRA_MOE_COMBINE_KERNEL") is not None  # tuning override: combine in a launch of its own
_SEPARATE_QKV_POST = os.environ.get("LYRA_QKV_POST_KERNEL") is not None  # tuning override: QK norm + RoPE + cache append in a launch of its own
_TILED_ACTIVATIONS = os.environ.get("LYRA_ROW_MAJOR_ACTIVATIONS") is None  # tuning override: expert matmuls read row-major activations
_LOGIT_TILE_MAX = os.environ.get("LYRA_NO_LOGIT_TILE_MAX") is None  # tuning override: samplers read the whole vocabulary
# Dense projections (q/k/v, output, MLP up and down) are handed to the kernels in the span-major copy whatever their width:
# a K-split workgroup then reads one contiguous run per wavefront instead of pieces a weight row apart (0.2-0.3 us of each
# 5-10 us launch).  Expert weights keep the reference's array unless their rows straddle cache lines (the copy costs the
# expert kernel more than it gains there).  LYRA_SPAN_MAJOR_DENSE=0: the alignment rule for every array.
_DENSE_SPAN_MAJOR = os.environ.get("LYRA_SPAN_MAJOR_DENSE", "1") != "0"


@dataclass
class TokenRows:
    """The residual stream before the first layer, not gathered yet: rows ``table[tokens]``."""

    table: torch.Tensor   # [V, C] bf16
    tokens: torch.Tensor  # [B] int32


def _bf16_bias(bias, groups: int = 1):
    """A bias as the matmul epilogue takes it: [groups, N] float32 holding the values rounded to bf16 (None stays None;
    lyra/model.py:527-528 casts the biases to the compute dtype).  Converted once and kept on the bias tensor itself, so
    that a decode step does not spend launches on its own weights (an in-place change of the bias converts it again)."""
    if bias is None:
        return None
    kept = getattr(bias, "_lyra_bf16_as_f32", None)
    if kept is None or kept[0] != (bias._version, groups):
        kept = ((bias._version, groups), bias.to(torch.bfloat16).to(torch.float32).reshape(groups, -1).contiguous())
        bias._lyra_bf16_as_f32 = kept
    return kept[1]


def attention_apply_fused(x, w: AttentionWeights, idx: int, pos, cos_t, sin_t, cache: LayerCache, cfg: ModelConfig):
    """attention_apply as 4 launches: norm(+gate) | qkv matmul | QK norm + RoPE + cache append + attention | output matmul.
    ``x`` is the residual stream or an ``Unsummed`` projection that still has to be added to it; the return value likewise
    (dense projections run split over K and leave the sum of their slices to the kernel that consumes them)."""
    from lyra_amd.kernels import decode_fused as F

    H, N, K = cfg.head_dim, cfg.n_attn_heads, cfg.n_kv_heads
    tiled = _TILED_ACTIVATIONS and cfg.n_embd % 32 == 0  # (the normalised rows only feed the q/k/v projection: 16 x 32 tiles)
    if isinstance(x, TokenRows):  # first layer of a step: the embedding rows are gathered by the norm kernel
        h, gate, x = F.embed_rmsnorm_proj(x.table, x.tokens, w.norm_scale, cfg.norm_eps, w.sdpa_gate, None, gate=True, tiled=tiled)
    elif isinstance(x, (F.Unsummed, F.Uncombined)):
        h, gate, x = F.rmsnorm_proj(x, w.norm_scale, cfg.norm_eps, w.sdpa_gate, None, gate=True, tiled=tiled)
    else:
        h, gate = F.rmsnorm_proj(x, w.norm_scale, cfg.norm_eps, w.sdpa_gate, None, gate=True, tiled=tiled)
    B = x.shape[0]
    one = _one_group(B, x.device)
    w_qkv, w_out = F.span_major(w.qkv, always=_DENSE_SPAN_MAJOR), F.span_major(w.out, always=_DENSE_SPAN_MAJOR)
    # (:310-313: a bias is added to the projection's bf16 result, in bf16: by the attention launch that sums the slices when
    # that launch is certain to take them - one position for the batch, no learned exclusive self attention - else inside
    # the matmul's epilogue, which costs the launch that sums the slices)
    front_step = w.xsa_alpha is None and not _SEPARATE_QKV_POST
    qkv = F.gemm_unsummed(h, w_qkv, one) if (w.qkv_bias is None or (front_step and pos.numel() == 1)) else None
    if qkv is not None and w.qkv_bias is not None:
        qkv.bias = _bf16_bias(w.qkv_bias).reshape(-1)
    if qkv is None:
        qkv = F.gemm(h, w_qkv, one, bias=_bf16_bias(w.qkv_bias), bias_after_cast=w.qkv_bias is not None)
    sliding_window = cfg.sliding_window if idx % 2 == 0 else 0
    t = None
    if front_step:  # QK norm + RoPE + cache append inside the attention launch
        t = F.attention_qkv(qkv, w.qnorm_scale, w.knorm_scale, cos_t, sin_t, pos, cache.k, cache.v, w.sinks, H**-0.5,
                            sliding_window, N, K, H, cfg.norm_eps, gate=gate)
    if t is None:  # (learned exclusive self attention, or a ragged batch the whole-row attention kernel takes)
        if isinstance(qkv, F.Unsummed) and qkv.bias is not None:  # (refused after all: the summed form carries the bias)
            qkv = F.gemm(h, w_qkv, one, bias=_bf16_bias(w.qkv_bias), bias_after_cast=True)
        q = F.qkv_post(qkv, w.qnorm_scale, w.knorm_scale, cos_t, sin_t, pos, cache.k, cache.v, N, K, H, cfg.norm_eps,
                       unit_v=w.xsa_alpha is not None)
        xsa_v = None
        if w.xsa_alpha is not None:  # the attention launch finishes with the exclusive-self-attention step (:351-363)
            q, xsa_v = q
        attn = attn_op(cfg.mode, cfg.implementation)
        t = attn(q[:, :, None, :], cache.k, cache.v, w.sinks, H**-0.5, sliding_window, pos, gate=gate, xsa_v=xsa_v,
                 xsa_alpha=w.xsa_alpha).reshape(B, N * H)
    # :366-373: projection, + bias, * residual scale, + residual, each a bf16 result - left to the norm that sums the slices
    out = F.gemm_unsummed(t, w_out, one)
    if out is None:
        return F.gemm(t, w_out, one, bias=_bf16_bias(w.out_bias), bias_after_cast=w.out_bias is not None, residual=x,
                      out_scale=cfg.residual_scale), cache
    out.residual, out.scale = x, cfg.residual_scale
    out.bias = None if w.out_bias is None else _bf16_bias(w.out_bias).reshape(-1)
    return out, cache


def moe_apply_fused(x, w: MoEWeights, cfg: ModelConfig, groups_out: list | None = None):
    """moe_apply as norm+router | routing | up matmul (token gather fused) | down matmul; the combine + residual step is
    handed to the next norm as an ``Uncombined`` value."""
    from lyra_amd.kernels import decode_fused as F

    topk = cfg.n_active_experts
    # (the normalised rows and the up projection's output feed expert matmuls only: both travel in 16 x 32 tiles, which is
    # how units of many rows - the shared expert's - read them fastest)
    tiled = _TILED_ACTIVATIONS and cfg.n_embd % 32 == 0 and cfg.expert_hidden % 32 == 0 and cfg.n_experts > 1
    if isinstance(x, (F.Unsummed, F.Uncombined)):
        xn, logits, x = F.rmsnorm_proj(x, w.norm_scale, cfg.norm_eps, w.router, w.router_bias, tiled=tiled)
    else:
        xn, logits = F.rmsnorm_proj(x, w.norm_scale, cfg.norm_eps, w.router, w.router_bias, tiled=tiled)
    B = x.shape[0]
    scores, groups, row_map, dest = F.moe_route(logits, cfg.n_routed_experts, cfg.n_shared_experts, cfg.n_active_routed_experts)
    if groups_out is not None:
        groups_out.append(groups)
    G = cfg.n_experts
    t = F.gemm(xn, F.span_major(w.mlp_up, glu=True), groups, rows=B * topk, row_map=row_map, fused_swiglu=True,
               swiglu_beta=cfg.swiglu_beta, swiglu_limit=cfg.swiglu_limit, bias=_bf16_bias(w.mlp_up_bias, G), out_tiled=tiled)
    t = F.gemm(t, F.span_major(w.mlp_down), groups, bias=_bf16_bias(w.mlp_down_bias, G))
    if topk <= 16 and not _SEPARATE_COMBINE:  # the combine step is left to the norm that follows (the next layer's, or the final one)
        return F.Uncombined(t, scores, dest, x, cfg.residual_scale)
    return F.moe_combine(t, scores, dest, x, cfg.residual_scale)


def dense_mlp_apply_fused(x, w: DenseMLPWeights, cfg: ModelConfig):
    from lyra_amd.kernels import decode_fused as F

    tiled = _TILED_ACTIVATIONS and cfg.n_embd % 32 == 0 and cfg.dense_hidden % 32 == 0
    if isinstance(x, (F.Unsummed, F.Uncombined)):
        t, _, x = F.rmsnorm_proj(x, w.norm_scale, cfg.norm_eps, tiled=tiled)
    else:
        t, _ = F.rmsnorm_proj(x, w.norm_scale, cfg.norm_eps, tiled=tiled)
    one = _one_group(x.shape[0], x.device)
    w_up, w_down = F.span_major(w.mlp_up, always=_DENSE_SPAN_MAJOR), F.span_major(w.mlp_down, always=_DENSE_SPAN_MAJOR)
    t = F.gemm(t, w_up, one, fused_swiglu=True, swiglu_beta=cfg.swiglu_beta, swiglu_limit=cfg.swiglu_limit,
               bias=_bf16_bias(w.mlp_up_bias), out_tiled=tiled)
    # :628-636: projection, + bias, * residual scale, + residual, each a bf16 result - left to the norm that sums the slices
    down = F.gemm_unsummed(t, w_down, one)
    if down is None:
        return F.gemm(t, w_down, one, bias=_bf16_bias(w.mlp_down_bias), bias_after_cast=w.mlp_down_bias is not None, residual=x,
                      out_scale=cfg.dense_residual_scale)
    down.residual, down.scale = x, cfg.dense_residual_scale
    down.bias = None if w.mlp_down_bias is None else _bf16_bias(w.mlp_down_bias).reshape(-1)
    return down


def _fused_supported(model: ModelWeights, cfg: ModelConfig) -> bool:
    """Shapes the fused launches cover (the matmul kernel's: K % 32, N % 8; the norm kernels': width % 4; the
    attention's: head width 64 or 128).  Projections whose widths are whole 128-column spans also run split over K with
    the sum left to their consumer; the others, and those followed by a bias, are summed by the matmul itself."""
    if not (cfg.fused_glue and cfg.implementation != "xla" and model.emb.is_cuda):
        return False
    C, H = cfg.n_embd, cfg.head_dim
    widths_ok = C % 32 == 0 and (cfg.n_attn_heads * H) % 32 == 0
    hidden = [cfg.dense_hidden] + ([cfg.expert_hidden] if "moe" in cfg.mlp_map else [])
    return (widths_ok and H in (64, 128) and all(h % 32 == 0 for h in hidden) and cfg.n_routed_experts <= 128
            and cfg.n_active_routed_experts <= 8 and cfg.padded_vocab_size % 8 == 0)


def model_apply_fused(tokens: torch.Tensor, model: ModelWeights, cache: ModelCache, cfg: ModelConfig, hidden_out: list | None = None,
                      groups_out: list | None = None, advance: bool = True):
    from lyra_amd.kernels import decode_fused as F

    # int32 token ids are gathered by the first norm kernel (one launch fewer, and a sampler can write them in place)
    h = TokenRows(model.emb, tokens) if tokens.dtype == torch.int32 and tokens.is_contiguous() else model.emb[tokens]
    cos_t, sin_t = _rope_tables(cfg, model.emb.device)
    pos = cache.pos
    for idx, layer in enumerate(model.layers):
        h, _ = attention_apply_fused(h, layer.attn, idx, pos, cos_t, sin_t, cache.layers[idx], cfg)
        h = moe_apply_fused(h, layer.mlp, cfg, groups_out) if isinstance(layer.mlp, MoEWeights) else dense_mlp_apply_fused(h, layer.mlp, cfg)
    normed = F.rmsnorm_proj(h, model.norm_scale, cfg.norm_eps)
    if hidden_out is not None:  # the residual stream after the last layer (the norm kernel completes it on its way)
        hidden_out.append(normed[2] if len(normed) > 2 else h)
    h = normed[0]
    # The LM head also leaves the maximum of every 128-column tile of the logits; they travel with the tensor (with the
    # version it had when they were taken) and `sample_token` hands them to a sampler that reads a few tiles per row instead
    # of the whole vocabulary - unless the logits have been written to since.
    w_head = F.span_major(model.unemb_t, always=True)  # (the span-major copy, made on the first step and kept)
    with_max = F.gemm_tile_max(h, w_head, _one_group(h.shape[0], h.device), bias=model.vocab_mask) if _LOGIT_TILE_MAX else None
    if with_max is not None:
        logits = with_max[0]
    else:
        logits = F.gemm(h, w_head, _one_group(h.shape[0], h.device), out_f32=True, bias=model.vocab_mask)
    if model.vocab_mask is None:
        logits[:, cfg.vocab_size :] = float("-inf")
    elif with_max is not None:
        logits.tile_max = (with_max[1], logits._version)
    if advance:
        cache.pos += 1
    return logits, cache


def model_apply(tokens: torch.Tensor, model: ModelWeights, cache: ModelCache, cfg: ModelConfig, hidden_out: list | None = None,
                groups_out: list | None = None, advance: bool = True):
    """lyra/model.py:734-793 in decode mode: tokens [B] int -> (logits [B, V_padded] f32, cache advanced by one).
    ``hidden_out``: optional list that receives the residual stream after the last layer [B, C] (for parity checks);
    ``groups_out``: optional list that receives the rows-per-expert tensor of every MoE layer;
    ``advance=False`` leaves ``cache.pos`` where it is (the caller's sampler advances it, or nobody does)."""
    if _fused_supported(model, cfg):
        return model_apply_fused(tokens, model, cache, cfg, hidden_out, groups_out, advance)
    h = model.emb[tokens.long()].to(torch.bfloat16)
    cos_t, sin_t = _rope_tables(cfg, h.device)
    pos = cache.pos
    cos, sin = cos_t.index_select(0, pos.to(torch.int64).reshape(1))[0], sin_t.index_select(0, pos.to(torch.int64).reshape(1))[0]
    for idx, layer in enumerate(model.layers):
        h, _ = attention_apply(h, layer.attn, idx, pos, cos, sin, cache.layers[idx], cfg)
        h = moe_apply(h, layer.mlp, cfg, groups_out) if isinstance(layer.mlp, MoEWeights) else dense_mlp_apply(h, layer.mlp, cfg)
    if hidden_out is not None:
        hidden_out.append(h)
    h = rms_norm(h, model.norm_scale, cfg.norm_eps)
    logits = _dense(h, model.unemb_t, cfg, out_f32=True)  # f32 logits (model.py:784-790)
    logits[:, cfg.vocab_size :] = float("-inf")
    if advance:
        cache.pos += 1
    return logits, cache


_ROPE_CACHE: dict = {}


def _rope_tables(cfg: ModelConfig, device):
    key = (cfg.seq_len, cfg.head_dim, cfg.rope_base, cfg.rope_scale, cfg.ntk_alpha, cfg.ntk_beta, str(device))
    if key not in _ROPE_CACHE:
        cos, sin = precompute_freq_cis(cfg)
        _ROPE_CACHE[key] = (torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device))
    return _ROPE_CACHE[key]
