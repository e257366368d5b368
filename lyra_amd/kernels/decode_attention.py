"""Decode attention behind the call signature of lyra/kernels/decode_attention.py:364-375.

``decode_attention(q, k, v, sinks, sm_scale, sliding_window, position, *, dtype, implementation)``
runs the gfx950 HIP kernel through ``lyra_decode_attention`` (include/lyra_hip.h).  Extensions that
default to the reference behaviour: ``position`` may be a ``[B]`` vector (ragged batch), and
``gate`` (``[B,N]``) fuses the output gate of lyra/model.py:343-347 into the kernel's epilogue.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from lyra_amd import _lib
from lyra_amd.kernels.common import Implementation, dispatch_kernel
from lyra_amd.nn.quant import QArray, dequantize, is_scaled

_DECODE_BLOCK = 128  # lyra/kernels/decode_attention.py:29 (slab granularity of the plain path)
_KERNEL_TILE = 32    # tokens per matrix-core tile in the HIP kernel
_MAX_HEAD_GROUPS = 16
_MAX_GRID_YZ = 65535


@dataclass(frozen=True)
class DecodeAttentionConfig:
    """What the HIP kernel was specialised on (mirrors decode_attention.py:32-38)."""

    tile_kv: int = _KERNEL_TILE
    kv_buffer_count: int = 2
    out_dtype: torch.dtype = torch.bfloat16
    cache_dtype: torch.dtype | None = None


def select_decode_attention_config(
    head_dim: int,
    head_groups: int,
    kv_len: int,
    sliding_window: int,
    out_dtype: torch.dtype,
    cache_dtype: torch.dtype | None = None,
    batch: int = 1,
    kv_heads: int = 1,
) -> DecodeAttentionConfig | None:
    """Support predicate of the HIP kernel (cf. decode_attention.py:41-60).

    Unlike the TPU kernel there is no ``kv_len % 128`` or ``head_dim % 128`` restriction.
    """
    cache_dtype = cache_dtype if cache_dtype is not None and is_scaled(cache_dtype) else None
    if head_dim not in (64, 128):
        return None
    if head_groups <= 0 or head_groups > _MAX_HEAD_GROUPS:
        return None
    if kv_len <= 0 or sliding_window < 0:
        return None
    if batch > _MAX_GRID_YZ or kv_heads > _MAX_GRID_YZ:  # batch rows and kv heads are grid dimensions of the launch
        return None
    if cache_dtype is not None and cache_dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
        return None
    if out_dtype not in (torch.bfloat16, torch.float32):
        return None
    return DecodeAttentionConfig(out_dtype=out_dtype, cache_dtype=cache_dtype)


def decode_window(sliding_window: int, block: int = _DECODE_BLOCK) -> int:
    """lyra/kernels/decode_attention.py:63-65."""
    n_blocks = -(-(sliding_window + block - 1) // block)
    return n_blocks * block


def is_sw(sliding_window: int, kv_len: int, block: int = _DECODE_BLOCK) -> bool:
    """lyra/kernels/decode_attention.py:68-69."""
    return sliding_window > 0 and decode_window(sliding_window, block) < kv_len


def _position_vector(position, batch: int, device) -> tuple[torch.Tensor, int]:
    """int32 device tensor and its stride (0: one scalar for the batch, 1: one entry per row)."""
    pos = torch.as_tensor(position, device=device)
    if pos.dtype != torch.int32:
        pos = pos.to(torch.int32)
    if pos.ndim == 0 or pos.numel() == 1:
        return pos.reshape(1).contiguous(), 0
    if pos.numel() != batch:
        raise ValueError(f"position must be a scalar or have one entry per batch row ({batch}), got {tuple(pos.shape)}")
    return pos.reshape(batch).contiguous(), 1


def rank_rows(position: torch.Tensor) -> torch.Tensor:
    """lyra_attention_rank: the batch rows from the longest to the shortest (int32 [B], ties to the lower row) for a [B]
    int32 device tensor of positions.  The order only changes when the batch does (every row grows by one token per step):
    compute it once per step or per batch and hand it to every layer's ``decode_attention(..., row_order=...)``."""
    pos = position.to(torch.int32).reshape(-1).contiguous()
    order = torch.empty_like(pos)
    rc = _lib.lib.lyra_attention_rank(pos.data_ptr(), pos.numel(), order.data_ptr(), torch.cuda.current_stream(pos.device).cuda_stream)
    _lib.check(rc, "lyra_attention_rank")
    return order


def _decode_attention(q, k, v, sinks, sm_scale, sliding_window, position, config: DecodeAttentionConfig, dtype, gate=None,
                      xsa_v=None, xsa_alpha=None, row_order=None):
    """Launch the HIP kernel (the counterpart of decode_attention.py:150-260)."""
    B, N, T, H = q.shape
    if T != 1:
        raise ValueError(f"decode attention takes one query token per sequence, got T={T}")
    _, K, S, _ = k.shape
    quantized = config.cache_dtype is not None
    if quantized:
        if not isinstance(k, QArray) or not isinstance(v, QArray):
            raise ValueError("quantized decode attention config requires QArray k/v")
        if k.block != (1, H) or v.block != (1, H):
            raise ValueError(f"FP8 KV cache block must be (1, {H}), got {k.block}/{v.block}")
        k_val, v_val = k.qval, v.qval
        k_scale = k.scale.to(torch.float32).reshape(B, K, S).contiguous()
        v_scale = v.scale.to(torch.float32).reshape(B, K, S).contiguous()
        kv_dtype = _lib.fp8_code(k_val.dtype)
    else:
        if isinstance(k, QArray) or isinstance(v, QArray):
            raise ValueError("dense decode attention config received QArray k/v")
        k_val, v_val = k.to(torch.bfloat16), v.to(torch.bfloat16)
        k_scale = v_scale = None
        kv_dtype = _lib.DTYPE_BF16
    if not q.is_cuda:
        raise ValueError("the HIP decode attention kernel needs device tensors")
    dev = q.device
    q_c = q.to(torch.bfloat16).reshape(B, N, H).contiguous()
    k_c, v_c = k_val.contiguous(), v_val.contiguous()
    sinks_c = sinks.to(device=dev, dtype=torch.float32).reshape(N).contiguous()
    pos, stride = _position_vector(position, B, dev)
    gate_c = None
    if gate is not None:
        gate_c = gate.to(device=dev, dtype=torch.bfloat16).reshape(B, N).contiguous()
    out_dtype = torch.float32 if dtype == torch.float32 else torch.bfloat16
    out = torch.empty((B, N, 1, H), dtype=out_dtype, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    need = _lib.lib.lyra_decode_attention_workspace(B, N, K, S, H, int(sliding_window))
    ws = _lib.workspace("attention", dev, stream, need)
    head = (q_c.data_ptr(), k_c.data_ptr(), v_c.data_ptr(),
            k_scale.data_ptr() if quantized else None, v_scale.data_ptr() if quantized else None,
            sinks_c.data_ptr(), pos.data_ptr(), stride, gate_c.data_ptr() if gate_c is not None else None)
    tail = (out.data_ptr(), ws.data_ptr(), ws.numel(), B, N, K, S, H, float(sm_scale), int(sliding_window), kv_dtype,
            _lib.DTYPE_F32 if out_dtype == torch.float32 else _lib.DTYPE_BF16, stream)
    with torch.cuda.device(dev):
        if xsa_v is not None:
            vn = xsa_v.to(device=dev, dtype=torch.bfloat16).reshape(B, K, H).contiguous()
            alpha = xsa_alpha.to(device=dev, dtype=torch.float32).reshape(N).contiguous()
            rc = _lib.lib.lyra_decode_attention_xsa(*head, vn.data_ptr(), alpha.data_ptr(), *tail)
        elif row_order is not None:
            order = row_order.to(device=dev, dtype=torch.int32).reshape(B).contiguous()
            rc = _lib.lib.lyra_decode_attention_ranked(*head[:8], order.data_ptr(), head[8], *tail)
        else:
            rc = _lib.lib.lyra_decode_attention(*head, *tail)
    _lib.check(rc, "lyra_decode_attention")
    return out if out.dtype == dtype else out.to(dtype)


def _reference_rows(q, k, v, sinks, sm_scale, sliding_window, pos: int, dtype):
    """decode_attention.py:311-361 for rows sharing one scalar position; q [b,N,1,H], k/v [b,K,S,H]."""
    B, N, T, H = q.shape
    _, K, S, _ = k.shape
    G = N // K
    if is_sw(sliding_window, S):
        # sliding_decode, :263-308: read a block-aligned slab that contains the window
        wlen = decode_window(sliding_window)
        vis0 = pos - sliding_window + 1
        start = min(max((vis0 // _DECODE_BLOCK) * _DECODE_BLOCK, 0), S - wlen)
        k, v = k[:, :, start : start + wlen], v[:, :, start : start + wlen]
        key_pos = start + torch.arange(wlen, device=q.device)
        visible = (key_pos <= pos) & (key_pos > pos - sliding_window)
    else:
        key_pos = torch.arange(S, device=q.device)
        visible = key_pos <= pos
        if sliding_window > 0:
            visible &= key_pos > pos - sliding_window
    mask = torch.where(visible, 0.0, float("-inf")).to(dtype)[None, :]
    qg = q.to(dtype).reshape(B, K, G, T, H)
    qk = torch.einsum("bkgth,bksh->bkgts", qg, k.to(dtype)) * sm_scale
    qk = qk + mask
    sk = sinks.to(torch.float32).reshape(K, G)[None, :, :, None, None].expand(B, K, G, T, 1)
    qk32 = qk.to(torch.float32)
    virtual_max = torch.maximum(qk32.amax(dim=-1, keepdim=True), sk)
    sink_strength = torch.exp(sk - virtual_max)
    unnormalized = torch.exp(qk32 - virtual_max)
    normalizer = torch.reciprocal(unnormalized.sum(dim=-1, keepdim=True) + sink_strength)
    a = unnormalized * normalizer
    out = torch.einsum("bkgts,bksh->bkgth", a, v.to(torch.float32))
    return out.to(dtype).reshape(B, N, T, H)


def xsa_reference(t, unit_v, xsa_alpha, dtype):
    """lyra/model.py:355-360 on t [B,N,1,H] (after the gate), unit_v [B,K,H] (the new value rows at unit length)."""
    B, N, T, H = t.shape
    K = unit_v.shape[1]
    t_g = t.to(dtype).reshape(B, K, N // K, T, H)
    vn_g = unit_v.to(dtype)[:, :, None, None, :]
    coef = (t_g * vn_g).to(torch.float32).sum(dim=-1, keepdim=True)
    alpha = torch.tanh(xsa_alpha.to(torch.float32)).reshape(1, K, N // K, 1, 1).to(dtype)
    return (t_g - alpha * coef.to(dtype) * vn_g).reshape(B, N, T, H)


def decode_attention_reference(q, k, v, sinks, sm_scale, sliding_window, position, dtype=None, gate=None):
    """Plain torch restatement of lyra/kernels/decode_attention.py:311-361 on the inputs' device.

    This is the ``implementation="xla"`` path: the whole cache is dequantised to bf16 first
    (:327-330), logits are held in ``dtype``, the sink softmax runs in float32.
    """
    B = q.shape[0]
    dtype = dtype if dtype is not None else q.dtype
    if isinstance(k, QArray) or isinstance(v, QArray):
        assert isinstance(k, QArray) and isinstance(v, QArray)
        k, v = dequantize(k, torch.bfloat16), dequantize(v, torch.bfloat16)
    pos = torch.as_tensor(position).reshape(-1).tolist()
    if len(pos) == 1:
        out = _reference_rows(q, k, v, sinks, sm_scale, sliding_window, int(pos[0]), dtype)
    else:
        if len(pos) != B:
            raise ValueError(f"position must be a scalar or have one entry per batch row ({B})")
        out = torch.cat(
            [_reference_rows(q[b : b + 1], k[b : b + 1], v[b : b + 1], sinks, sm_scale, sliding_window, int(pos[b]), dtype) for b in range(B)]
        )
    if gate is not None:
        out = out * gate.to(out.device).reshape(B, -1)[:, :, None, None].to(dtype)
    return out


def decode_attention(
    q: torch.Tensor,
    k,
    v,
    sinks: torch.Tensor,
    sm_scale: float,
    sliding_window: int,
    position,
    *,
    dtype: torch.dtype | None = None,
    implementation: Implementation = "auto",
    gate: torch.Tensor | None = None,
    xsa_v: torch.Tensor | None = None,
    xsa_alpha: torch.Tensor | None = None,
    row_order: torch.Tensor | None = None,
) -> torch.Tensor:
    """q [B,N,1,H]; k, v [B,K,S,H] tensors or QArray (e4m3fn or e5m2 codes, block (1,H)); sinks [N]; returns [B,N,1,H].

    ``row_order`` (``rank_rows(position)``; ragged batches only): lets the kernel deal the rows out by length instead of
    ranking them in every launch.  It changes which workgroup computes which row, never a result.

    ``xsa_v`` [B,K,H] (the new token's value rows at unit length) with ``xsa_alpha`` [N] fuses the learned exclusive
    self attention of lyra/model.py:351-363 behind the gate; both default to None (the reference operator).

    Deliberate divergence from the reference: ``"auto"`` selects the kernel when the shape is
    supported (the reference's auto always takes XLA for this op, decode_attention.py:408).
    """
    B, N, _, H = q.shape
    _, K, S, _ = k.shape
    HEAD_GROUPS = N // K
    dtype = dtype if dtype is not None else q.dtype
    cache_dtype = k.dtype if isinstance(k, QArray) else None
    supported_layout = N % K == 0 and q.is_cuda
    config = (
        select_decode_attention_config(
            head_dim=H, head_groups=HEAD_GROUPS, kv_len=S, sliding_window=sliding_window, out_dtype=dtype, cache_dtype=cache_dtype,
            batch=B, kv_heads=K,
        )
        if supported_layout
        else None
    )

    if (xsa_v is None) != (xsa_alpha is None):
        raise ValueError("xsa_v and xsa_alpha go together")

    def reference():
        t = decode_attention_reference(q, k, v, sinks, sm_scale, sliding_window, position, dtype, gate=gate)
        return t if xsa_v is None else xsa_reference(t, xsa_v, xsa_alpha, dtype)

    def kernel():
        assert config is not None
        return _decode_attention(q, k, v, sinks, sm_scale, sliding_window, position, config, dtype, gate=gate,
                                 xsa_v=xsa_v, xsa_alpha=xsa_alpha, row_order=row_order)

    tiling = None if config is None else f"kv{config.tile_kv} buf{config.kv_buffer_count} {'fp8' if config.cache_dtype else 'bf16'}"
    op_shape = f"b{B} n{N} k{K} s{S} h{H} sw{sliding_window}"
    return dispatch_kernel(
        "decode_attention",
        implementation=implementation,
        shape=op_shape,
        config=config,
        tiling=tiling,
        kernel=kernel,
        reference=reference,
    )
