"""Host wrappers of the fused decode-step kernels (include/lyra_hip.h: lyra_rmsnorm_proj, lyra_qkv_post,
lyra_decode_gemm_ex, lyra_moe_route, lyra_moe_combine).

The reference leaves these steps to XLA fusion inside its jitted decode step (lyra/model.py:284-374, 451-567,
608-636); here each is one HIP launch.  Every function takes and returns torch device tensors and launches on the
current stream, so a whole decode step can be captured in a HIP graph.
"""
from __future__ import annotations

import torch

from lyra_amd import _lib
from lyra_amd.nn.quant import QArray

_L = _lib.lib


def _stream(dev) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _f32(t):
    assert t.dtype == torch.float32 and t.is_contiguous()
    return t


_TRANSPOSED: dict = {}


def _transposed(w: torch.Tensor) -> torch.Tensor:
    """[C,n] parameter -> contiguous [n,C] copy, made once per weight tensor (weights do not change while decoding)."""
    key = (w.data_ptr(), tuple(w.shape), w.device)
    hit = _TRANSPOSED.get(key)
    if hit is None or hit[0] is not w:
        hit = (w, w.t().contiguous())
        _TRANSPOSED[key] = hit
    return hit[1]


class Unsummed:
    """A projection whose K slices are still separate: ``partials`` [splits, M, N] float32, plus the residual update that
    follows it (``residual`` [M, N] bf16 and ``scale``), to be applied by the kernel that consumes it.  ``bias``: the
    projection's own bias [N] (float32 holding bf16 values), which the consumer adds to the bf16-rounded sum in bf16
    (lyra/model.py:310-313, 367-368, 629-630); the attention launch with the front step and the norm kernel take it,
    ``qkv_post`` does not."""

    __slots__ = ("partials", "residual", "scale", "bias")

    def __init__(self, partials: torch.Tensor, residual: torch.Tensor | None = None, scale: float = 1.0,
                 bias: torch.Tensor | None = None):
        self.partials, self.residual, self.scale, self.bias = partials, residual, scale, bias


class Uncombined:
    """The end of a MoE layer before its combine step: expert outputs ``rows`` [T * topk, C] bf16 in sorted order,
    ``scores`` [T, topk] float32, ``dest`` [T * topk] int32, the residual stream ``residual`` [T, C] bf16 and the residual
    ``scale``; the kernel that consumes it forms bf16(residual + bf16(bf16(sum_k scores * rows[dest]) * scale))."""

    __slots__ = ("rows", "scores", "dest", "residual", "scale")

    def __init__(self, rows: torch.Tensor, scores: torch.Tensor, dest: torch.Tensor, residual: torch.Tensor, scale: float):
        self.rows, self.scores, self.dest, self.residual, self.scale = rows, scores, dest, residual, scale


class Tiled16:
    """bf16 activations [rows, cols] in tiles of 16 rows x 32 columns (element (r, c) at
    (((r >> 4) * (cols >> 5) + (c >> 5)) * 16 + (r & 15)) * 32 + (c & 31)): what ``rmsnorm_proj(..., tiled=True)`` and
    ``gemm(..., out_tiled=True)`` write and ``gemm`` reads as lhs when the rows feed an expert matmul."""

    __slots__ = ("data", "rows", "cols")

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @staticmethod
    def empty(rows: int, cols: int, device) -> "Tiled16":
        assert cols % 32 == 0
        return Tiled16(torch.empty(((rows + 15) // 16 * 16) * cols, dtype=torch.bfloat16, device=device), rows, cols)

    def untiled(self) -> torch.Tensor:
        """The row-major [rows, cols] array (tests)."""
        rb = self.data.numel() // (16 * self.cols)
        return self.data.reshape(rb, self.cols // 32, 16, 32).permute(0, 2, 1, 3).reshape(rb * 16, self.cols)[: self.rows]


def tile16(x: torch.Tensor) -> Tiled16:
    """Row-major [rows, cols] bf16 -> Tiled16, with torch ops (tests, fallbacks)."""
    rows, cols = x.shape
    rb = (rows + 15) // 16
    pad = torch.zeros(rb * 16, cols, dtype=x.dtype, device=x.device)
    pad[:rows] = x
    return Tiled16(pad.reshape(rb, 16, cols // 32, 32).permute(0, 2, 1, 3).contiguous().reshape(-1), rows, cols)


class SpanMajor:
    """Weights [G, K, N] (bf16, or FP8 with their QArray scales) in the span-major copy ``lyra_gemm_pack`` makes once when a
    model is loaded: every 128-column span of every matrix is one contiguous run of K rows.  ``layout`` 1: spans of 128
    consecutive columns; 2: spans of 64 gate columns followed by their 64 linear columns (expert up projections, whose
    SwiGLU is fused).  ``scale`` / ``block`` keep the reference's [G, K/bk, N/bn] layout.  Accepted by ``gemm`` and
    ``gemm_unsummed`` wherever the reference array is; the array itself is no longer needed then."""

    __slots__ = ("data", "shape", "dtype", "scale", "block", "layout", "fallback")

    def __init__(self, data, shape, dtype, scale, block, layout, fallback=None):
        self.data, self.shape, self.dtype, self.scale, self.block, self.layout = data, tuple(shape), dtype, scale, block, layout
        self.fallback = fallback  # the reference array, when the caller kept it: used where no kernel reads this layout


def pack_weights(rhs, glu: bool = False) -> SpanMajor:
    """rhs: bf16 [G, K, N] tensor or FP8 QArray -> SpanMajor (layout 2 when ``glu``: gate and linear columns paired)."""
    fp8 = isinstance(rhs, QArray)
    rv = rhs.qval if fp8 else rhs
    assert rv.is_contiguous() and rv.ndim == 3 and (fp8 or rv.dtype == torch.bfloat16)
    G, K, N = rv.shape
    layout = 2 if glu else 1
    dt = _lib.fp8_code(rv.dtype) if fp8 else _lib.DTYPE_BF16
    nbytes = _L.lyra_gemm_packed_bytes(G, K, N, dt, layout)
    if nbytes == 0:
        raise ValueError(f"no span-major layout {layout} for weights {tuple(rv.shape)} {rv.dtype}")
    data = torch.empty(nbytes, dtype=torch.uint8, device=rv.device)
    _lib.check(_L.lyra_gemm_pack(rv.data_ptr(), data.data_ptr(), G, K, N, dt, layout, _stream(rv.device)), "lyra_gemm_pack")
    return SpanMajor(data, (G, K, N), rv.dtype, _f32(rhs.scale) if fp8 else None, tuple(rhs.block) if fp8 else None, layout)


_SPAN_MAJOR: dict = {}
_SPAN_MAJOR_MODE = __import__("os").environ.get("LYRA_SPAN_MAJOR", "auto")  # tuning override: "0" never, "1" every weight


def span_major(rhs, glu: bool = False, always: bool = False):
    """The weight operand a fused decode step should hand to ``gemm``: the span-major copy (made once per weight array and
    kept) when the rows of the reference's array do not start on 128-byte lines - FP8 weights whose width, or whose linear
    half under a fused SwiGLU, is not a multiple of 128 columns, as with gpt-oss-20b's 2880: every 128-byte piece a
    workgroup reads from such an array straddles two lines and the launch fetches half as much again - else ``rhs``.
    ``always``: the copy whatever the width (the LM head: a wavefront then walks one contiguous 512 KB run instead of 2048
    pieces 400 KB apart, 2-3 % of that launch)."""
    if isinstance(rhs, SpanMajor) or _SPAN_MAJOR_MODE == "0":
        return rhs
    fp8 = isinstance(rhs, QArray)
    rv = rhs.qval if fp8 else rhs
    N = rv.shape[-1]
    row = N * rv.element_size()
    if _SPAN_MAJOR_MODE != "1" and not always and row % 128 == 0 and not (glu and (row // 2) % 128):
        return rhs
    if N % (16 if glu else 8) or not rv.is_cuda:
        return rhs
    key = (rv.data_ptr(), tuple(rv.shape), glu)
    hit = _SPAN_MAJOR.get(key)
    if hit is None or hit[0] is not rv:
        packed = pack_weights(rhs, glu)
        packed.fallback = rhs
        hit = (rv, packed)
        _SPAN_MAJOR[key] = hit
    return hit[1]


def _rhs_args(rhs):
    """(data tensor, scale tensor | None, bk, bn, rhs_dtype word of the C ABI, shape) of a weight operand."""
    if isinstance(rhs, SpanMajor):
        fp8 = rhs.scale is not None
        flag = _lib.RHS_SPAN_MAJOR if rhs.layout == 1 else _lib.RHS_SPAN_MAJOR_GLU
        bk, bn = rhs.block if fp8 else (0, 0)
        return rhs.data, rhs.scale, bk, bn, (_lib.fp8_code(rhs.dtype) if fp8 else _lib.DTYPE_BF16) | flag, rhs.shape
    if isinstance(rhs, QArray):
        bk, bn = rhs.block
        assert rhs.qval.is_contiguous()
        return rhs.qval, _f32(rhs.scale), bk, bn, _lib.fp8_code(rhs.qval.dtype), tuple(rhs.shape)
    assert rhs.dtype == torch.bfloat16 and rhs.is_contiguous()
    return rhs, None, 0, 0, _lib.DTYPE_BF16, tuple(rhs.shape)


def gemm_unsummed(lhs: torch.Tensor, rhs, group_sizes: torch.Tensor) -> Unsummed | None:
    """lyra_decode_gemm_partials for a one-group projection; None when the shape does not run split over K."""
    tiled = isinstance(lhs, Tiled16)
    M, K = (lhs.rows, lhs.cols) if tiled else lhs.shape
    lhs_t = lhs.data if tiled else lhs
    rv, rs, bk, bn, rd, (G, _, N) = _rhs_args(rhs)
    if G != 1 or K % 32 or N % 8 or (isinstance(rhs, SpanMajor) and rhs.layout != 1):
        return None
    splits = _L.lyra_decode_gemm_splits(M, K, N, bk)
    if splits <= 0:
        return None
    assert lhs_t.dtype == torch.bfloat16 and lhs_t.is_contiguous()
    part = torch.empty((splits, M, N), dtype=torch.float32, device=lhs_t.device)
    rc = _L.lyra_decode_gemm_partials(lhs_t.data_ptr(), rv.data_ptr(), _ptr(rs), bk, bn,
                                      group_sizes.data_ptr(), part.data_ptr(), part.numel() * 4, M, K, N,
                                      rd | (_lib.LHS_TILED16 if tiled else 0), _stream(lhs_t.device))
    _lib.check(rc, "lyra_decode_gemm_partials")
    return Unsummed(part)


def rmsnorm_proj(x, scale: torch.Tensor, eps: float, proj: torch.Tensor | None = None,
                 bias: torch.Tensor | None = None, gate: bool = False, tiled: bool = False):
    """rms_norm (lyra/model.py:189-191) of x [B,C] bf16; with ``proj`` [C,n] f32 also f32(h) @ proj (+ bias) as
    float32 logits, or bf16 ``2*sigmoid`` gates when ``gate`` is set (model.py:343-347).  Returns (h, y | None).
    ``tiled``: h comes back as a ``Tiled16`` (the layout an expert matmul reads its rows fastest in; C % 32 == 0).

    ``x`` may be an ``Unsummed`` projection with its residual: the row is then first formed as
    ``bf16(residual + bf16(bf16(sum of slices) * scale))`` and returned as a third value.  Likewise for an ``Uncombined``
    MoE layer end (the combine step of lyra/model.py:557-567 happens while the row is read)."""
    if isinstance(x, Uncombined):
        u = x
        B, C = u.residual.shape
        topk = u.scores.shape[1]
        assert u.residual.dtype == torch.bfloat16 and u.residual.is_contiguous()
        assert u.rows.dtype == torch.bfloat16 and u.rows.is_contiguous() and tuple(u.rows.shape) == (B * topk, C)
        x_out = torch.empty_like(u.residual)
        h_obj, h, mode = _norm_out(u.residual, tiled, gate)
        y, n = None, 0
        if proj is not None:
            n = proj.shape[1]
            y = torch.empty((B, n), dtype=torch.bfloat16 if gate else torch.float32, device=h.device)
            proj = _f32(_transposed(proj))
        rc = _L.lyra_rmsnorm_proj_combine(u.rows.data_ptr(), _f32(u.scores).data_ptr(), u.dest.data_ptr(), topk, u.residual.data_ptr(),
                                          float(u.scale), x_out.data_ptr(), _f32(scale).data_ptr(), h.data_ptr(), _ptr(proj),
                                          _ptr(bias), _ptr(y), B, C, n, mode, float(eps), _stream(h.device))
        _lib.check(rc, "lyra_rmsnorm_proj_combine")
        return h_obj, y, x_out
    if isinstance(x, Unsummed):
        u = x
        splits, B, C = u.partials.shape
        assert u.residual is not None and u.residual.dtype == torch.bfloat16 and u.residual.is_contiguous()
        x_out = torch.empty_like(u.residual)
        h_obj, h, mode = _norm_out(u.residual, tiled, gate)
        y, n = None, 0
        if proj is not None:
            n = proj.shape[1]
            y = torch.empty((B, n), dtype=torch.bfloat16 if gate else torch.float32, device=h.device)
            proj = _f32(_transposed(proj))
        if u.bias is not None:
            assert u.bias.dtype == torch.float32 and u.bias.is_contiguous() and u.bias.numel() == C
        rc = _L.lyra_rmsnorm_proj_sum_bias(None, u.partials.data_ptr(), splits, _ptr(u.bias), u.residual.data_ptr(), float(u.scale),
                                           x_out.data_ptr(), _f32(scale).data_ptr(), h.data_ptr(), _ptr(proj), _ptr(bias), _ptr(y),
                                           B, C, n, mode, float(eps), _stream(h.device))
        _lib.check(rc, "lyra_rmsnorm_proj_sum_bias")
        return h_obj, y, x_out
    B, C = x.shape
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    h_obj, h, mode = _norm_out(x, tiled, gate)
    y, n = None, 0
    if proj is not None:
        n = proj.shape[1]
        y = torch.empty((B, n), dtype=torch.bfloat16 if gate else torch.float32, device=x.device)
        proj = _f32(_transposed(proj))
    rc = _L.lyra_rmsnorm_proj(x.data_ptr(), _f32(scale).data_ptr(), h.data_ptr(), _ptr(proj), _ptr(bias), _ptr(y), B, C, n,
                              mode, float(eps), _stream(x.device))
    _lib.check(rc, "lyra_rmsnorm_proj")
    return h_obj, y


def _norm_out(like: torch.Tensor, tiled: bool, gate: bool):
    """(what the caller gets, the tensor the kernel writes, the kernel's mode word) for the normalised rows of a norm launch."""
    mode = 1 if gate else 2
    if not tiled:
        h = torch.empty_like(like)
        return h, h, mode
    obj = Tiled16.empty(like.shape[0], like.shape[1], like.device)
    return obj, obj.data, mode | 4


def embed_rmsnorm_proj(table: torch.Tensor, tokens: torch.Tensor, scale: torch.Tensor, eps: float,
                       proj: torch.Tensor | None = None, bias: torch.Tensor | None = None, gate: bool = False, tiled: bool = False):
    """The first norm of a decode step with the token gather folded in (lyra/model.py:752 + :303): rows
    ``table[tokens]`` (table [V,C] bf16, tokens [B] int32) are normalised as in ``rmsnorm_proj``; returns (h, y | None, x)
    with x [B,C] the gathered rows, i.e. the residual stream."""
    V, C = table.shape
    B = tokens.shape[0]
    assert table.dtype == torch.bfloat16 and table.is_contiguous() and tokens.dtype == torch.int32 and tokens.is_contiguous()
    x = torch.empty((B, C), dtype=torch.bfloat16, device=table.device)
    h_obj, h, mode = _norm_out(x, tiled, gate)
    y, n = None, 0
    if proj is not None:
        n = proj.shape[1]
        y = torch.empty((B, n), dtype=torch.bfloat16 if gate else torch.float32, device=x.device)
        proj = _f32(_transposed(proj))
    rc = _L.lyra_rmsnorm_proj_embed(table.data_ptr(), tokens.data_ptr(), V, x.data_ptr(), _f32(scale).data_ptr(), h.data_ptr(),
                                    _ptr(proj), _ptr(bias), _ptr(y), B, C, n, mode, float(eps), _stream(x.device))
    _lib.check(rc, "lyra_rmsnorm_proj_embed")
    return h_obj, y, x


def qkv_post(qkv, qnorm, knorm, cos_t: torch.Tensor, sin_t: torch.Tensor, pos: torch.Tensor, cache_k, cache_v,
             n_heads: int, n_kv_heads: int, head_dim: int, eps: float, unit_v: bool = False):
    """QK norm + rotary embedding + KV-cache append (quantising for an FP8 cache) for one new token per sequence
    (lyra/model.py:309-336); ``pos`` is an int32 device scalar or a [B] tensor.  Returns q [B,N,H] bf16; the caches
    are updated in place.  ``unit_v``: also return the new value rows scaled to unit length [B,K,H] bf16
    (model.py:353-354), as (q, v_unit)."""
    N, K, H = n_heads, n_kv_heads, head_dim
    unsummed = isinstance(qkv, Unsummed)
    if unsummed:  # the projection arrives as K slices; they are summed while reading
        assert qkv.bias is None, "a projection with a bias comes summed (gemm with bias_after_cast) to qkv_post"
        part = qkv.partials
        splits, B, width = part.shape
        assert width == (N + 2 * K) * H and qkv.residual is None
        dev = part.device
    else:
        B = qkv.shape[0]
        assert qkv.dtype == torch.bfloat16 and qkv.is_contiguous() and qkv.shape[1] == (N + 2 * K) * H
        dev = qkv.device
    assert pos.dtype == torch.int32
    q = torch.empty((B, N, H), dtype=torch.bfloat16, device=dev)
    fp8 = isinstance(cache_k, QArray)
    if fp8:
        assert tuple(cache_k.block) == (1, H) and cache_k.scale.dtype == torch.float32
        kq, vq, ks, vs = cache_k.qval, cache_v.qval, cache_k.scale, cache_v.scale
        S = kq.shape[2]
    else:
        kq, vq, ks, vs = cache_k, cache_v, None, None
        S = kq.shape[2]
        assert kq.dtype == torch.bfloat16
    assert kq.is_contiguous() and vq.is_contiguous() and tuple(kq.shape) == (B, K, S, H)
    vn = torch.empty((B, K, H), dtype=torch.bfloat16, device=dev) if unit_v else None
    rc = _L.lyra_qkv_post_sum(None if unsummed else qkv.data_ptr(), part.data_ptr() if unsummed else None, splits if unsummed else 0,
                              _ptr(qnorm), _ptr(knorm), _f32(cos_t).data_ptr(), _f32(sin_t).data_ptr(), pos.data_ptr(),
                              0 if pos.numel() == 1 else 1, q.data_ptr(), kq.data_ptr(), vq.data_ptr(), _ptr(ks), _ptr(vs),
                              _ptr(vn), B, N, K, S, H, cos_t.shape[0], _lib.fp8_code(kq.dtype) if fp8 else _lib.DTYPE_BF16, float(eps),
                              _stream(dev))
    _lib.check(rc, "lyra_qkv_post_sum")
    return (q, vn) if unit_v else q


def attention_qkv(qkv, qnorm, knorm, cos_t: torch.Tensor, sin_t: torch.Tensor, pos: torch.Tensor, cache_k, cache_v, sinks,
                  sm_scale: float, sliding_window: int, n_heads: int, n_kv_heads: int, head_dim: int, eps: float, gate=None,
                  out_dtype: torch.dtype = torch.bfloat16):
    """``qkv_post`` and the decode attention in one launch (lyra/model.py:309-347): the attention kernel's workgroups sum
    the projection's slices, apply QK norm and the rotary embedding, append the new key and value rows to the caches (in
    place) and attend.  Results and cache contents are bit-identical to the two launches.  Returns [B, N*H] bf16, or None
    when the launch does not exist for this shape (a ragged batch of more than 256 (row, kv head) pairs, which the
    whole-row kernel takes): the caller then runs the two launches.  ``out_dtype``: bfloat16 (what the decode step
    uses) or float32 (the attention's ``dtype`` argument, lyra/kernels/decode_attention.py:373)."""
    N, K, H = n_heads, n_kv_heads, head_dim
    assert out_dtype in (torch.bfloat16, torch.float32)
    unsummed = isinstance(qkv, Unsummed)
    if unsummed:
        part = qkv.partials
        splits, B, width = part.shape
        assert width == (N + 2 * K) * H and qkv.residual is None
        dev = part.device
    else:
        B = qkv.shape[0]
        assert qkv.dtype == torch.bfloat16 and qkv.is_contiguous() and qkv.shape[1] == (N + 2 * K) * H
        dev = qkv.device
    assert pos.dtype == torch.int32
    fp8 = isinstance(cache_k, QArray)
    if fp8:
        assert tuple(cache_k.block) == (1, H) and cache_k.scale.dtype == torch.float32
        kq, vq, ks, vs = cache_k.qval, cache_v.qval, cache_k.scale, cache_v.scale
    else:
        kq, vq, ks, vs = cache_k, cache_v, None, None
        assert kq.dtype == torch.bfloat16
    S = kq.shape[2]
    assert kq.is_contiguous() and vq.is_contiguous() and tuple(kq.shape) == (B, K, S, H)
    assert sinks.dtype == torch.float32 and sinks.numel() == N and sinks.is_contiguous()
    if gate is not None:
        assert gate.dtype == torch.bfloat16 and gate.is_contiguous() and gate.numel() == B * N
    out = torch.empty((B, N * H), dtype=out_dtype, device=dev)
    stream = _stream(dev)
    need = _L.lyra_decode_attention_workspace(B, N, K, S, H, int(sliding_window))
    ws = _lib.workspace("attention", dev, stream, need)
    qkv_bias = qkv.bias if unsummed else None
    if qkv_bias is not None:
        assert qkv_bias.dtype == torch.float32 and qkv_bias.is_contiguous() and qkv_bias.numel() == (N + 2 * K) * H
    rc = _L.lyra_decode_attention_qkv_bias(None if unsummed else qkv.data_ptr(), part.data_ptr() if unsummed else None,
                                      splits if unsummed else 0, _ptr(qkv_bias), _ptr(qnorm), _ptr(knorm), _f32(cos_t).data_ptr(),
                                      _f32(sin_t).data_ptr(), cos_t.shape[0], float(eps), kq.data_ptr(), vq.data_ptr(), _ptr(ks),
                                      _ptr(vs), sinks.data_ptr(), pos.data_ptr(), 0 if pos.numel() == 1 else 1, _ptr(gate),
                                      out.data_ptr(), ws.data_ptr(), ws.numel(), B, N, K, S, H, float(sm_scale),
                                      int(sliding_window), _lib.fp8_code(kq.dtype) if fp8 else _lib.DTYPE_BF16,
                                      _lib.DTYPE_F32 if out_dtype == torch.float32 else _lib.DTYPE_BF16, stream)
    if rc == _lib.E_UNSUPPORTED:
        return None
    _lib.check(rc, "lyra_decode_attention_qkv")
    return out


def gemm(lhs: torch.Tensor, rhs, group_sizes: torch.Tensor, *, rows: int | None = None, row_map: torch.Tensor | None = None,
         residual: torch.Tensor | None = None, out_scale: float | None = None, fused_swiglu: bool = False,
         swiglu_beta: float = 1.702, swiglu_limit: float = 7.0, out_f32: bool = False,
         bias: torch.Tensor | None = None, bias_after_cast: bool = False, out_tiled: bool = False):
    """lyra_decode_gemm_ex: the decode grouped matmul with an optional row gather on the input and an optional
    ``bf16(residual + bf16(bf16(t) * out_scale))`` epilogue.  rhs: bf16 [G,K,N] tensor or FP8 QArray.
    A ``SpanMajor`` rhs (``pack_weights``) is read in that layout.
    ``bias`` [G, N] float32 is added to the float32 product (lyra/kernels/gemm.py:1600-1605), or with ``bias_after_cast``
    (one group, no SwiGLU) to the product rounded to bf16, in bf16, as a caller does that adds a bias to the operator's
    result (lyra/model.py:310-313, 367-368)."""
    rv, rs, bk, bn, rd, (G, K, N) = _rhs_args(rhs)
    lhs_tiled = isinstance(lhs, Tiled16)
    if lhs_tiled:  # (rows in tiles of 16 x 32, what the norm or the matmul before wrote)
        assert lhs.cols == K
        M = rows if rows is not None else lhs.rows
        lhs_t = lhs.data
    else:
        M = rows if rows is not None else lhs.shape[0]
        assert lhs.dtype == torch.bfloat16 and lhs.is_contiguous() and lhs.shape[1] == K
        lhs_t = lhs
    dev = lhs_t.device
    assert group_sizes.dtype == torch.int32 and group_sizes.numel() == G
    NO = N // 2 if fused_swiglu else N
    if out_tiled:
        assert not out_f32 and residual is None and NO % 32 == 0
        out_obj = Tiled16.empty(M, NO, dev)
        out = out_obj.data
    else:
        out = torch.empty((M, NO), dtype=torch.float32 if out_f32 else torch.bfloat16, device=dev)
    if residual is not None:
        assert residual.dtype == torch.bfloat16 and residual.is_contiguous() and tuple(residual.shape) == (M, NO)
    if row_map is not None:
        assert row_map.dtype == torch.int32 and row_map.numel() >= M
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == G * N
    stream = _stream(dev)
    need = _L.lyra_decode_gemm_workspace(M, G, K, N, int(fused_swiglu))
    ws = _lib.workspace("gemm", dev, stream, need)
    rc = _L.lyra_decode_gemm_ex(lhs_t.data_ptr(), _ptr(row_map), rv.data_ptr(), _ptr(rs), bk, bn, group_sizes.data_ptr(), _ptr(bias),
                                _ptr(residual), 1.0 if out_scale is None else float(out_scale),
                                int(out_scale is not None) | (2 if bias_after_cast else 0),
                                out.data_ptr(), ws.data_ptr(), ws.numel(), M, G, K, N,
                                rd | (_lib.LHS_TILED16 if lhs_tiled else 0) | (_lib.OUT_TILED16 if out_tiled else 0),
                                _lib.DTYPE_F32 if out_f32 else _lib.DTYPE_BF16, int(fused_swiglu), float(swiglu_beta),
                                float(swiglu_limit), stream)
    if rc == _lib.E_UNSUPPORTED and (lhs_tiled or out_tiled):
        # (a plan without tiled activations, e.g. one group with more rows than the K-split kernel takes: through row-major copies)
        res = gemm(lhs.untiled().contiguous() if lhs_tiled else lhs, rhs, group_sizes, rows=rows, row_map=row_map, residual=residual,
                   out_scale=out_scale, fused_swiglu=fused_swiglu, swiglu_beta=swiglu_beta, swiglu_limit=swiglu_limit, out_f32=out_f32,
                   bias=bias, bias_after_cast=bias_after_cast)
        return tile16(res) if out_tiled else res
    if rc == _lib.E_UNSUPPORTED and isinstance(rhs, SpanMajor) and rhs.fallback is not None:
        # (a shape whose plan has no span-major kernel, e.g. one group with too many rows for the K-split kernel)
        return gemm(lhs, rhs.fallback, group_sizes, rows=rows, row_map=row_map, residual=residual, out_scale=out_scale,
                    fused_swiglu=fused_swiglu, swiglu_beta=swiglu_beta, swiglu_limit=swiglu_limit, out_f32=out_f32, bias=bias,
                    bias_after_cast=bias_after_cast, out_tiled=out_tiled)
    _lib.check(rc, "lyra_decode_gemm_ex")
    return out_obj if out_tiled else out


def gemm_tile_max(lhs: torch.Tensor, rhs, group_sizes: torch.Tensor, bias: torch.Tensor | None = None):
    """lyra_decode_gemm_tile_max: float32 ``lhs @ rhs (+ bias)`` for one group (the LM head, lyra/model.py:784-790) together
    with the maximum of every 128-column tile of every result row, which ``argmax`` / ``sample_topk`` take as
    ``tile_max``.  Returns (out [M, N], tile_max [M, ceil(N / 128)]) or None for a shape the launch does not take."""
    rv, rs, bk, bn, rd, (G, K, N) = _rhs_args(rhs)
    if G != 1 or not isinstance(lhs, torch.Tensor):
        return None
    M = lhs.shape[0]
    assert lhs.dtype == torch.bfloat16 and lhs.is_contiguous() and lhs.shape[1] == K
    assert group_sizes.dtype == torch.int32 and group_sizes.numel() == 1
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == N
    dev = lhs.device
    out = torch.empty((M, N), dtype=torch.float32, device=dev)
    tmax = torch.empty((M, (N + 127) // 128), dtype=torch.float32, device=dev)
    stream = _stream(dev)
    ws = _lib.workspace("gemm", dev, stream, _L.lyra_decode_gemm_workspace(M, 1, K, N, 0))
    rc = _L.lyra_decode_gemm_tile_max(lhs.data_ptr(), None, rv.data_ptr(), _ptr(rs), bk, bn, group_sizes.data_ptr(), _ptr(bias),
                                      out.data_ptr(), tmax.data_ptr(), ws.data_ptr(), ws.numel(), M, 1, K, N, rd, _lib.DTYPE_F32,
                                      stream)
    if rc == _lib.E_UNSUPPORTED:
        if isinstance(rhs, SpanMajor) and rhs.fallback is not None:  # (a shape whose kernel does not read this layout)
            return gemm_tile_max(lhs, rhs.fallback, group_sizes, bias=bias)
        return None
    _lib.check(rc, "lyra_decode_gemm_tile_max")
    return out, tmax


def moe_route(logits: torch.Tensor, n_routed: int, n_shared: int, k_routed: int):
    """Router top-k + softmax + shared experts + stable sort by expert (lyra/model.py:459-491).
    Returns (scores [T,topk] f32, groups [E] i32, row_map [T*topk] i32, dest [T*topk] i32)."""
    T = logits.shape[0]
    assert logits.dtype == torch.float32 and logits.is_contiguous() and logits.shape[1] == n_routed
    topk, E = k_routed + n_shared, n_routed + n_shared
    dev = logits.device
    scores = torch.empty((T, topk), dtype=torch.float32, device=dev)
    groups = torch.empty(E, dtype=torch.int32, device=dev)
    row_map = torch.empty(T * topk, dtype=torch.int32, device=dev)
    dest = torch.empty(T * topk, dtype=torch.int32, device=dev)
    rc = _L.lyra_moe_route(logits.data_ptr(), scores.data_ptr(), groups.data_ptr(), row_map.data_ptr(), dest.data_ptr(), T,
                           n_routed, n_shared, k_routed, _stream(dev))
    _lib.check(rc, "lyra_moe_route")
    return scores, groups, row_map, dest


def moe_combine(rows: torch.Tensor, scores: torch.Tensor, dest: torch.Tensor, x: torch.Tensor, residual_scale: float) -> torch.Tensor:
    """x + bf16(bf16(sum_k scores[f,k] * rows[dest[f,k]]) * residual_scale)  (lyra/model.py:557-567)."""
    T, C = x.shape
    topk = scores.shape[1]
    assert rows.dtype == torch.bfloat16 and rows.is_contiguous() and tuple(rows.shape) == (T * topk, C)
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    out = torch.empty_like(x)
    rc = _L.lyra_moe_combine(rows.data_ptr(), _f32(scores).data_ptr(), dest.data_ptr(), x.data_ptr(), out.data_ptr(), T, topk, C,
                             float(residual_scale), _stream(x.device))
    _lib.check(rc, "lyra_moe_combine")
    return out


def _check_tile_max(tile_max: torch.Tensor, rows: int, cols: int, device) -> None:
    assert tile_max.dtype == torch.float32 and tile_max.is_contiguous() and tile_max.device == device
    assert tile_max.dim() == 2 and tile_max.shape[0] == rows and tile_max.shape[1] >= (cols + 127) // 128


def argmax(logits: torch.Tensor, cols: int | None = None, out: torch.Tensor | None = None,
           advance: torch.Tensor | None = None, tile_max: torch.Tensor | None = None) -> torch.Tensor:
    """Greedy token choice (lyra/generate.py:46-53 at temperature 0): first index of each row's maximum over the first
    ``cols`` columns of float32 ``logits`` [rows, ld]; returns int32 [rows].  ``advance``: an int32 device scalar (the
    cache position) the launch increments by one.  ``tile_max``: what ``gemm_tile_max`` returned with these logits -
    the launch then reads those and one tile per row (lyra_argmax_tiles)."""
    rows, ld = logits.shape
    cols = ld if cols is None else cols
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    assert out.dtype == torch.int32 and out.is_contiguous() and out.numel() == rows
    stream = _stream(logits.device)
    if tile_max is not None:
        _check_tile_max(tile_max, rows, cols, logits.device)
        assert advance is None or (advance.dtype == torch.int32 and advance.numel() == 1)
        rc = _L.lyra_argmax_tiles(logits.data_ptr(), tile_max.data_ptr(), out.data_ptr(), rows, cols, ld, tile_max.shape[1],
                                  _ptr(advance), stream)
        _lib.check(rc, "lyra_argmax_tiles")
        return out
    ws = _lib.workspace("argmax", logits.device, stream, _L.lyra_argmax_workspace(rows, cols))
    assert advance is None or (advance.dtype == torch.int32 and advance.numel() == 1)
    rc = _L.lyra_argmax(logits.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, ld, _ptr(advance), stream)
    _lib.check(rc, "lyra_argmax")
    return out


def sample_topk(logits: torch.Tensor, uniforms: torch.Tensor, k: int, temperature: float, cols: int | None = None,
                out: torch.Tensor | None = None, advance: torch.Tensor | None = None,
                tile_max: torch.Tensor | None = None) -> torch.Tensor:
    """Temperature / top-k token choice (lyra/generate.py:46-53 at temperature > 0) for every row of float32 ``logits``
    [rows, ld] over its first ``cols`` columns: softmax of the k largest ``logits / temperature`` (ties to the lower
    index), inverse CDF at ``uniforms`` [rows] in [0, 1); returns int32 [rows].  ``uniforms`` may instead be the
    generator state ``rng_state(seed)`` makes (int64 [2] on the device: seed, draws so far): the launch then makes its own
    uniform numbers and moves the state on (lyra_sample_topk_rng).  ``tile_max``: what ``gemm_tile_max`` returned with
    these logits - same result from the tile maxima and a few tiles per row (lyra_sample_topk_tiles)."""
    rows, ld = logits.shape
    cols = ld if cols is None else cols
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    own_rng = uniforms.dtype == torch.int64
    if own_rng:
        assert uniforms.shape == (2,) and uniforms.is_contiguous() and uniforms.device == logits.device
    else:
        assert uniforms.dtype == torch.float32 and uniforms.shape == (rows,) and uniforms.is_contiguous()
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    assert out.dtype == torch.int32 and out.is_contiguous() and out.numel() == rows
    stream = _stream(logits.device)
    ws = _lib.workspace("argmax", logits.device, stream, _L.lyra_sample_topk_workspace(rows, cols, k))
    if tile_max is not None and k <= 8:
        _check_tile_max(tile_max, rows, cols, logits.device)
        rc = _L.lyra_sample_topk_tiles(logits.data_ptr(), tile_max.data_ptr(), None if own_rng else uniforms.data_ptr(),
                                       uniforms.data_ptr() if own_rng else None, out.data_ptr(), ws.data_ptr(), ws.numel(), rows,
                                       cols, ld, tile_max.shape[1], k, float(temperature), _ptr(advance), stream)
        if rc != _lib.E_UNSUPPORTED:  # (rows that are not 16-byte aligned: the whole-row sampler below)
            _lib.check(rc, "lyra_sample_topk_tiles")
            return out
    fn = _L.lyra_sample_topk_rng if own_rng else _L.lyra_sample_topk
    rc = fn(logits.data_ptr(), uniforms.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, ld, k,
            float(temperature), _ptr(advance), stream)
    _lib.check(rc, "lyra_sample_topk")
    return out


_RNG_STATES: dict = {}


def rng_state(device, seed: int | None = None) -> torch.Tensor:
    """The state of the sampler's own generator on ``device`` (int64 [2]: seed, draws so far).  With ``seed`` a fresh state;
    without, one state per device, seeded from torch's initial seed the first time it is asked for."""
    if seed is not None:
        return torch.tensor([seed & 0x7FFFFFFFFFFFFFFF, 0], dtype=torch.int64, device=device)
    key = str(device)
    if key not in _RNG_STATES:
        _RNG_STATES[key] = torch.tensor([torch.initial_seed() & 0x7FFFFFFFFFFFFFFF, 0], dtype=torch.int64, device=device)
    return _RNG_STATES[key]
