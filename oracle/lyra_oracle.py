"""CPU oracle for Lyra's decode hot path (NumPy, fp32).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` use it, and only as the checker.

Every function restates one piece of the reference's plain-JAX ("XLA") decode
path and cites the reference file:line it follows.  Two arithmetic modes:

* ``mode="fp32"``  - all arithmetic in float32, no intermediate rounding.  This
  is the "fp32 reference" the acceptance tolerances are stated against.
* ``mode="ref"``   - additionally rounds to bfloat16 at the points where the
  JAX code holds a bf16 array (dequantised cache, ``qk`` logits, output), so
  the size of those roundings can be measured rather than assumed.

Pinning status (what fixes each function independently of this file's own
formulas; the checks live in tests/test_oracle_*.py):

* fp8 e4m3fn / e5m2 decode/encode .. all 256 codes and all rounding midpoints
                                     against ``torch.float8_e4m3fn`` / ``torch.float8_e5m2``
* bf16 rounding .................... against ``torch.bfloat16`` casts
* quantize / dequantize ............ closed forms of lyra/nn/quant.py:68-72
* sink softmax attention ........... ``torch`` SDPA / softmax with one extra
                                     key of logit ``sink`` and value 0; limits
* window / slab index arithmetic ... brute force over every position
* grouped GEMM ..................... per-group ``torch.matmul``; brute force
* SwiGLU ........................... scalar closed forms
* routing / bpermute ............... stable argsort + bincount; the input
                                     vector of reference tests/test_combine.py:13
* xsa / unit_rows .................. closed forms: alpha = 0 is the identity; t parallel to v^ with tanh(alpha) -> 1
                                     gives 0; the component of t orthogonal to v^ is unchanged and the parallel one is
                                     scaled by 1 - tanh(alpha); head n uses kv head n // G (one-hot rows); scalar
                                     loops on H = 8
* rope_tables / rotate ............. rotation of the complex pair (x_i, x_{i+H/2}) by pos * base^(-2i/H); YaRN branch:
                                     magnitude (0.1 ln s + 1), untouched / interpolated pairs and the linear ramp between
                                     the hand-computed landmarks 8.09 and 17.39 at the gpt-oss setting
* sample_topk ....................... closed forms: k = 1 is the argmax, u -> 0 / u -> 1 pick the first / k-th
                                     candidate, ties to the lower index, frequencies over a grid of u against
                                     ``torch.softmax`` of the k largest logits / temperature
* ``jax.random.categorical``'s key stream (lyra/generate.py:53): PARITY UNPINNED - the draw is restated as the
  inverse CDF at a caller-supplied uniform number (same distribution, different randomness)
* exact XLA bf16 rounding points and summation order inside einsum:
  PARITY UNPINNED (needs the reference runtime, which cannot be imported
  here); irrelevant to acceptance because tolerances are against fp32.
"""
from __future__ import annotations

import math

import numpy as np

FP8_E4M3FN_MAX = 448.0  # jnp.finfo(float8_e4m3fn).max, lyra/nn/quant.py:68
DECODE_BLOCK = 128  # lyra/kernels/decode_attention.py:29


# ---------------------------------------------------------------------------
# Number formats
# ---------------------------------------------------------------------------
def fp8_e4m3fn_decode_table() -> np.ndarray:
    """float32 value of each of the 256 OCP FP8 E4M3 ("fn": finite, no inf) codes.

    Layout s.eeee.mmm, bias 7; exponent field 0 is subnormal (m/8 * 2^-6);
    S.1111.111 is NaN; every other code is finite (max 448 = 1.75 * 2^8).
    """
    table = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            val = float("nan")
        elif e == 0:
            val = sign * (m / 8.0) * 2.0**-6
        else:
            val = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        table[code] = val
    return table


_FP8_TABLE = fp8_e4m3fn_decode_table()

FP8_E5M2_MAX = 57344.0  # jnp.finfo(float8_e5m2).max: the other format of FP8_DTYPES, lyra/nn/quant.py:10


def fp8_e5m2_decode_table() -> np.ndarray:
    """float32 value of each of the 256 OCP FP8 E5M2 codes.

    Layout s.eeeee.mm, bias 15, IEEE-like: exponent field 0 is subnormal (m/4 * 2^-14), exponent field 31 is
    infinity (m = 0) or NaN; max finite 57344 = 1.75 * 2^15.  The code is the upper byte of the float16 with the same value.
    """
    table = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 2) & 0x1F
        m = code & 0x3
        if e == 0x1F:
            val = float("nan") if m else sign * float("inf")
        elif e == 0:
            val = sign * (m / 4.0) * 2.0**-14
        else:
            val = sign * (1.0 + m / 4.0) * 2.0 ** (e - 15)
        table[code] = val
    return table


_FP8_E5M2_TABLE = fp8_e5m2_decode_table()
FP8_FORMATS = {1: "e4m3fn", 2: "e5m2"}  # the format numbers the C oracle and the device library use for 1-byte arrays


def fp8_max(fmt: int = 1) -> float:
    return {1: FP8_E4M3FN_MAX, 2: FP8_E5M2_MAX}[fmt]


def fp8_decode(codes: np.ndarray, fmt: int = 1) -> np.ndarray:
    return {1: _FP8_TABLE, 2: _FP8_E5M2_TABLE}[fmt][np.asarray(codes, dtype=np.uint8)]


def fp8_e5m2_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> e5m2 code, round-to-nearest-even, as ``astype(float8_e5m2)``: magnitudes that round above 57344 become
    infinity (0x7c), NaN becomes 0x7f.  The reference clips to +-57344 first (lyra/nn/quant.py:72)."""
    x = np.asarray(x, dtype=np.float32)
    sign = np.signbit(x).astype(np.uint8) << 7
    a = np.abs(x).astype(np.float64)
    nan = np.isnan(a)
    inf = np.isinf(a)
    a = np.where(nan | inf, 1.0, a)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.clip(e, -14, 15)
    ulp = 2.0 ** (e - 2)  # 2 mantissa bits
    val = np.rint(a / ulp) * ulp  # numpy rint = round half to even; exact in float64
    with np.errstate(divide="ignore", invalid="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    e2 = np.clip(e2, -14, 16)
    sub = val < 2.0**-14
    mant = np.where(sub, val / 2.0**-16, (val / 2.0**e2 - 1.0) * 4.0)
    expf = np.where(sub, 0, e2 + 15)
    code = (expf.astype(np.int64) << 2) | np.rint(mant).astype(np.int64)
    code = np.where((val > FP8_E5M2_MAX) | inf, 0x7C, code)
    code = np.where(nan, 0x7F, code)
    return ((code.astype(np.uint8) & 0x7F) | sign).astype(np.uint8)


def fp8_encode(x: np.ndarray, fmt: int = 1) -> np.ndarray:
    return fp8_e5m2_encode(x) if fmt == 2 else fp8_e4m3fn_encode(x)


def fp8_e4m3fn_decode(codes: np.ndarray) -> np.ndarray:
    return _FP8_TABLE[np.asarray(codes, dtype=np.uint8)]


def fp8_e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn code, round-to-nearest-even, as ``astype(float8_e4m3fn)``.

    Finite inputs beyond the largest finite value saturate to NaN in the "fn"
    format when cast directly; the reference clips to +-448 first
    (lyra/nn/quant.py:72) so that branch is unreachable there; here magnitudes
    that round above 448 map to NaN (0x7f) like the direct cast.
    """
    x = np.asarray(x, dtype=np.float32)
    sign = np.signbit(x).astype(np.uint8) << 7
    a = np.abs(x).astype(np.float64)
    out = np.zeros(x.shape, dtype=np.uint8)
    nan = np.isnan(a)
    # exponent of the value's binade, clamped to the subnormal binade (-6)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.clip(e, -6, 8)
    ulp = 2.0 ** (e - 3)  # 3 mantissa bits
    q = a / ulp  # in units of ulp; exact in float64
    r = np.rint(q)  # numpy rint = round half to even
    val = r * ulp
    # re-derive fields from the rounded value (rounding may carry into the next binade)
    with np.errstate(divide="ignore", invalid="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    e2 = np.clip(e2, -6, 9)
    sub = val < 2.0**-6
    mant = np.where(sub, val / 2.0**-9, (val / 2.0**e2 - 1.0) * 8.0)
    expf = np.where(sub, 0, e2 + 7)
    code = (expf.astype(np.int64) << 3) | np.rint(mant).astype(np.int64)
    over = val > FP8_E4M3FN_MAX
    code = np.where(over | nan, 0x7F, code)
    out = (code.astype(np.uint8) & 0x7F) | sign
    return out.astype(np.uint8)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bfloat16 (ties to even); result kept as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    r = bits >> np.uint32(16)
    r &= np.uint32(1)
    r += np.uint32(0x7FFF)
    r += bits
    r &= np.uint32(0xFFFF0000)
    out = r.view(np.float32)
    nan = np.isnan(x)
    if nan.any():
        out[nan] = x[nan]
    return out


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of bf16_round(x) (for handing bf16 buffers to device code)."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------------------
# Block-scaled FP8 arrays  (lyra/nn/quant.py)
# ---------------------------------------------------------------------------
def _tile(x: np.ndarray, block: tuple[int, ...]) -> np.ndarray:
    """lyra/nn/quant.py:34-40 - split each trailing dim d into (d // b, b)."""
    n = len(block)
    lead, tail = x.shape[: x.ndim - n], x.shape[x.ndim - n :]
    bad = [(d, b) for d, b in zip(tail, block) if d % b]
    if bad:
        raise ValueError(f"block {block} does not divide trailing dims {tail}")
    return x.reshape(*lead, *(v for d, b in zip(tail, block) for v in (d // b, b)))


def _block_axes(ldim: int, sdim: int) -> tuple[int, ...]:
    """lyra/nn/quant.py:43-45."""
    return tuple(ldim + 2 * i + 1 for i in range(sdim))


def quantize(x: np.ndarray, block: tuple[int, ...], fmt: int = 1) -> tuple[np.ndarray, np.ndarray]:
    """lyra/nn/quant.py:48-75 for dtype=float8_e4m3fn (``fmt`` 1) or float8_e5m2 (``fmt`` 2), scale_dtype=float32.

    Returns (qval uint8 codes with x.shape, scale float32 of shape lead x (dim/block)).
    """
    x = np.asarray(x, dtype=np.float32)
    sdim = len(block)
    ldim = x.ndim - sdim
    axes = _block_axes(ldim, sdim)
    tiled = _tile(x, block)
    fmax = np.float32(fp8_max(fmt))
    amax = np.max(np.abs(tiled), axis=axes).astype(np.float32)
    scale = np.where(amax > 0, amax / fmax, np.float32(1.0)).astype(np.float32)  # :70
    qinv = np.expand_dims((np.float32(1.0) / scale).astype(np.float32), axes)  # :71
    scaled = np.clip((tiled * qinv).astype(np.float32), -fmax, fmax)  # :72
    qval = fp8_encode(scaled, fmt).reshape(x.shape)
    return qval, scale


def dequantize(qval: np.ndarray, scale: np.ndarray, block: tuple[int, ...], *, to_bf16: bool = True, fmt: int = 1) -> np.ndarray:
    """lyra/nn/quant.py:78-86: f32(qval) * scale, then cast (bf16 by default)."""
    sdim = len(block)
    ldim = qval.ndim - sdim
    axes = _block_axes(ldim, sdim)
    tiled = _tile(fp8_decode(qval, fmt), block)
    s = np.expand_dims(np.asarray(scale, dtype=np.float32), axes)
    x = (tiled * s).astype(np.float32).reshape(qval.shape)
    return bf16_round(x) if to_bf16 else x


def qupdate(qval: np.ndarray, scale: np.ndarray, block: tuple[int, ...], x: np.ndarray, start: tuple[int, ...]):
    """lyra/nn/quant.py:89-98 - quantise ``x`` with the array's block and write it at ``start``."""
    ldim = qval.ndim - len(block)
    eff = [1 if a < ldim else block[a - ldim] for a in range(qval.ndim)]
    for axis, s in enumerate(start):
        if s % eff[axis]:
            raise ValueError(f"start {s} on axis {axis} is not aligned to block {eff[axis]}")
    qn, sn = quantize(x, block)
    qval, scale = qval.copy(), scale.copy()
    sl = tuple(slice(s, s + d) for s, d in zip(start, qn.shape))
    qval[sl] = qn
    sstart = tuple(s // eff[a] for a, s in enumerate(start))
    ssl = tuple(slice(s, s + d) for s, d in zip(sstart, sn.shape))
    scale[ssl] = sn
    return qval, scale


# ---------------------------------------------------------------------------
# Decode attention  (lyra/kernels/decode_attention.py)
# ---------------------------------------------------------------------------
def decode_window(sliding_window: int, block: int = DECODE_BLOCK) -> int:
    """lyra/kernels/decode_attention.py:63-65."""
    n_blocks = -(-(sliding_window + block - 1) // block)
    return n_blocks * block


def is_sw(sliding_window: int, kv_len: int, block: int = DECODE_BLOCK) -> bool:
    """lyra/kernels/decode_attention.py:68-69."""
    return sliding_window > 0 and decode_window(sliding_window, block) < kv_len


def sliding_start(position: int, sliding_window: int, kv_len: int) -> int:
    """First key of the slab read by ``sliding_decode`` (decode_attention.py:277-280).

    ``//`` is floor division (XLA/NumPy semantics on negative operands).
    """
    wlen = decode_window(sliding_window)
    vis = int(position) - sliding_window + 1
    return int(min(max((vis // DECODE_BLOCK) * DECODE_BLOCK, 0), kv_len - wlen))


def visible_mask(position: int, sliding_window: int, kv_len: int) -> np.ndarray:
    """bool[S]: key j is attended iff j <= pos and (sw == 0 or j > pos - sw).

    decode_attention.py:338-340 (full path) and :285-286 (slab path) give the same set.
    """
    j = np.arange(kv_len)
    vis = j <= position
    if sliding_window > 0:
        vis &= j > position - sliding_window
    return vis


def visible_range(position: int, sliding_window: int, kv_len: int) -> tuple[int, int]:
    """Closed interval [lo, hi] of attended keys; (0, -1) when empty."""
    hi = min(int(position), kv_len - 1)
    lo = max(0, int(position) - sliding_window + 1) if sliding_window > 0 else 0
    return (lo, hi) if hi >= lo else (0, -1)


def _softmax_with_sink(qk: np.ndarray, sinks: np.ndarray) -> np.ndarray:
    """decode_attention.py:348-355; qk [..., S] float32 (masked = -inf), sinks broadcastable [..., 1]."""
    vmax = np.maximum(np.max(qk, axis=-1, keepdims=True), sinks)
    sink_strength = np.exp(sinks - vmax)
    un = np.exp(qk - vmax)
    normalizer = np.float32(1.0) / (np.sum(un, axis=-1, keepdims=True, dtype=np.float32) + sink_strength)
    return (un * normalizer).astype(np.float32)


def _attend(q, k, v, sinks, sm_scale, mask, mode):
    """Shared body of decode_attention_reference / sliding_decode for one batch row.

    q [K,G,H] f32, k/v [K,S',H] f32, sinks [K,G] f32, mask bool[S'].
    """
    qk = np.einsum("kgh,ksh->kgs", q, k, dtype=np.float32)
    if mode == "ref":
        # einsum of two bf16 arrays yields bf16; "* sm_scale" stays bf16 (weak python float)
        qk = bf16_round(bf16_round(qk) * np.float32(sm_scale))
    else:
        qk = (qk * np.float32(sm_scale)).astype(np.float32)
    qk = np.where(mask[None, None, :], qk, np.float32(-np.inf)).astype(np.float32)
    a = _softmax_with_sink(qk, sinks[:, :, None].astype(np.float32))
    out = np.einsum("kgs,ksh->kgh", a, v, dtype=np.float32)
    return bf16_round(out) if mode == "ref" else out


def decode_attention_reference(
    q: np.ndarray,
    k,
    v,
    sinks: np.ndarray,
    sm_scale: float,
    sliding_window: int,
    position,
    *,
    mode: str = "fp32",
    gate: np.ndarray | None = None,
    fp8_format: int = 1,
) -> np.ndarray:
    """decode_attention.py:311-361 (+ :263-308 slab path, :392-395 dequantise-first).

    q        [B,N,1,H] float32 holding bf16-representable values
    k, v     [B,K,S,H] float32 (bf16 cache)  or  (qval uint8, scale f32 [B,K,S,1]) for an
             FP8 cache quantised with block (1,H); ``fp8_format`` names the codes (1 e4m3fn, 2 e5m2)
    sinks    [N] float32; head n belongs to KV head n // G, slot n % G   (:349-350)
    position scalar or [B] int - index of the newest token; the reference takes one
             scalar, a vector is the ragged-batch extension (each row on its own scalar)
    gate     optional [B,N] float32 multiplied onto the output (model.py:343-347; the
             caller passes bf16(2*sigmoid(.)))
    Returns  [B,N,1,H] float32 (bf16-representable when mode="ref").
    """
    assert mode in ("fp32", "ref")
    q = np.asarray(q, dtype=np.float32)
    B, N, T, H = q.shape
    assert T == 1
    if isinstance(k, tuple):
        kq, ks = k
        vq, vs = v
        # decode_attention.py:393-394 - the whole cache is dequantised to bf16 first
        k = dequantize(kq, ks, (1, H), to_bf16=(mode == "ref"), fmt=fp8_format)
        v = dequantize(vq, vs, (1, H), to_bf16=(mode == "ref"), fmt=fp8_format)
    k = np.asarray(k, dtype=np.float32)
    v = np.asarray(v, dtype=np.float32)
    _, K, S, _ = k.shape
    G = N // K
    pos = np.broadcast_to(np.asarray(position, dtype=np.int64).reshape(-1), (B,)) if np.ndim(position) else np.full((B,), int(position))
    sinks_kg = np.asarray(sinks, dtype=np.float32).reshape(K, G)
    out = np.empty((B, N, 1, H), dtype=np.float32)
    for b in range(B):
        p = int(pos[b])
        qb = q[b, :, 0, :].reshape(K, G, H)
        if is_sw(sliding_window, S):
            # sliding_decode: only a slab of wlen keys is read (:277-288)
            wlen = decode_window(sliding_window)
            start = sliding_start(p, sliding_window, S)
            key_pos = start + np.arange(wlen)
            mask = (key_pos <= p) & (key_pos > p - sliding_window)
            ob = _attend(qb, k[b, :, start : start + wlen], v[b, :, start : start + wlen], sinks_kg, sm_scale, mask, mode)
        else:
            mask = visible_mask(p, sliding_window, S)
            ob = _attend(qb, k[b], v[b], sinks_kg, sm_scale, mask, mode)
        out[b, :, 0, :] = ob.reshape(N, H)
    if gate is not None:
        out = out * np.asarray(gate, dtype=np.float32)[:, :, None, None]
        if mode == "ref":
            out = bf16_round(out)
    return out


# ---------------------------------------------------------------------------
# Decode GEMM  (lyra/kernels/decode_gemm.py, gemm.py, common.py)
# ---------------------------------------------------------------------------
def expert_ids(group_sizes: np.ndarray, total: int) -> np.ndarray:
    """gemm.py:450-456 - repeat(arange(G), group_sizes, total_repeat_length=total).

    jnp.repeat with total_repeat_length gathers a[cumsum(onehot(group starts)) - 1]; every
    group start is <= sum(group_sizes), so rows at or beyond the sum get id G-1.
    """
    gs = np.asarray(group_sizes, dtype=np.int64)
    ids = np.repeat(np.arange(gs.shape[0], dtype=np.int32), gs)
    if ids.shape[0] < total:
        ids = np.concatenate([ids, np.full(total - ids.shape[0], gs.shape[0] - 1, dtype=np.int32)])
    return ids[:total]


def normalize_bias(bias: np.ndarray | None, groups: int, features: int) -> np.ndarray:
    """gemm.py:393-400 -> float32 [G,1,N]."""
    if bias is None:
        return np.zeros((groups, 1, features), dtype=np.float32)
    bias = np.asarray(bias, dtype=np.float32)
    if bias.ndim == 2:
        bias = bias[:, None, :]
    if bias.shape != (groups, 1, features):
        raise ValueError(f"Unsupported bias shape: {bias.shape}")
    return bias


def swiglu(x: np.ndarray, beta: float = 1.702, limit: float = 7.0, shift: float = 1.0) -> np.ndarray:
    """common.py:98-114 with interleaved=False: first half gates, second half is linear."""
    x = np.asarray(x, dtype=np.float32)
    glu, lin = np.split(x, 2, axis=-1)
    glu = np.minimum(glu, np.float32(limit))
    lin = np.clip(lin, np.float32(-limit), np.float32(limit))
    with np.errstate(over="ignore"):
        sig = np.float32(1.0) / (np.float32(1.0) + np.exp(-np.float32(beta) * glu))
    return ((lin + np.float32(shift)) * (glu * sig)).astype(np.float32)


def grouped_gemm_reference(
    lhs: np.ndarray,
    rhs: np.ndarray,
    group_sizes: np.ndarray,
    *,
    bias: np.ndarray | None = None,
    fused_swiglu: bool = False,
    swiglu_beta: float = 1.702,
    swiglu_limit: float = 7.0,
    mode: str = "fp32",
) -> np.ndarray:
    """gemm.py:1575-1617 with quant_dtype=None (how decode calls it, decode_gemm.py:390-399).

    lhs [M,K] f32 (bf16-representable), rhs [G,K,N] f32 already dequantised,
    group_sizes [G]; rows are sorted by group; rows >= sum(group_sizes) are zero
    (lax.ragged_dot) before the bias of the padded expert id is added.
    """
    lhs = np.asarray(lhs, dtype=np.float32)
    rhs = np.asarray(rhs, dtype=np.float32)
    M, K = lhs.shape
    G, _, N = rhs.shape
    gs = np.asarray(group_sizes, dtype=np.int64)
    t = np.zeros((M, N), dtype=np.float32)
    off = 0
    for g in range(G):
        n = int(gs[g])
        if n:
            t[off : off + n] = lhs[off : off + n] @ rhs[g]
        off += n
    if bias is not None:
        ids = expert_ids(gs, M)
        t = t + normalize_bias(bias, G, N)[ids, 0, :]
    if fused_swiglu:
        t = swiglu(t, swiglu_beta, swiglu_limit)
    return bf16_round(t) if mode == "ref" else t.astype(np.float32)


def decode_gemm_reference(
    lhs: np.ndarray,
    rhs,
    group_sizes: np.ndarray,
    *,
    block: tuple[int, int] | None = None,
    bias: np.ndarray | None = None,
    fused_swiglu: bool = False,
    swiglu_beta: float = 1.702,
    swiglu_limit: float = 7.0,
    mode: str = "fp32",
    dequant_bf16: bool | None = None,
    fp8_format: int = 1,
) -> np.ndarray:
    """decode_gemm.py:368-401 / :419-449.

    rhs is either float32 [G,K,N] (dense weights; the reference casts them to
    lhs.dtype = bf16, :437) or (qval uint8 [G,K,N], scale f32 [G,K/bk,N/bn]) with
    ``block=(bk,bn)`` (codes of ``fp8_format``: 1 e4m3fn, 2 e5m2), dequantised to lhs.dtype before the grouped product (:431).
    The lhs is never quantised on this path (quant_dtype=None at :398).
    ``dequant_bf16`` overrides what ``mode`` says about the dequantised weights alone: True rounds them to bf16 as the
    reference does (quant.py:85) while the product, bias and SwiGLU stay in float32 when mode="fp32".
    """
    if isinstance(rhs, tuple):
        qval, scale = rhs
        assert block is not None
        w = dequantize(qval, scale, block, to_bf16=(mode == "ref") if dequant_bf16 is None else dequant_bf16, fmt=fp8_format)
    else:
        w = np.asarray(rhs, dtype=np.float32)
        if mode == "ref":
            w = bf16_round(w)
    return grouped_gemm_reference(
        lhs, w, group_sizes, bias=bias, fused_swiglu=fused_swiglu, swiglu_beta=swiglu_beta, swiglu_limit=swiglu_limit, mode=mode
    )


def default_weight_block(k: int, n: int, quant_block: tuple[int, int] = (256, 256)) -> tuple[int, int]:
    """model.py:154-156 / decode_gemm.py:385."""
    return (math.gcd(k, quant_block[0]), math.gcd(n, quant_block[1]))


# ---------------------------------------------------------------------------
# Callers of the two kernels  (lyra/model.py) - integer parts are bit-exact contracts
# ---------------------------------------------------------------------------
def rms_norm(x: np.ndarray, scale: np.ndarray, eps: float) -> np.ndarray:
    """model.py:189-191 (float32 maths; the caller casts)."""
    t = np.asarray(x, dtype=np.float32)
    return (t / np.sqrt(np.mean(t * t, axis=-1, keepdims=True, dtype=np.float32) + np.float32(eps)) * scale).astype(np.float32)


def rotate(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """model.py:183-186 - half-split rotary embedding."""
    x1, x2 = np.split(np.asarray(x, dtype=np.float32), 2, axis=-1)
    return np.concatenate([x1 * cos - x2 * sin, x2 * cos + x1 * sin], axis=-1).astype(np.float32)


def rope_tables(seq_len: int, head_dim: int, rope_base: float = 150000.0, rope_scale: float = 1.0,
                ntk_alpha: float = 1.0, ntk_beta: float = 32.0) -> tuple[np.ndarray, np.ndarray]:
    """model.py:160-180 (float64 angles -> float32 cos/sin), including the YaRN branch."""
    positions = np.arange(int(seq_len * rope_scale), dtype=np.float64)
    inv_freq = 1.0 / (rope_base ** (np.arange(0, head_dim, 2, dtype=np.float64) / head_dim))
    concentration = 1.0
    if rope_scale > 1.0:
        concentration = 0.1 * math.log(rope_scale) + 1.0
        dim_half = head_dim / 2.0
        log_base = math.log(rope_base) ** -1.0
        low = dim_half * math.log(seq_len / (ntk_beta * 2.0 * math.pi)) * log_base
        high = dim_half * math.log(seq_len / (ntk_alpha * 2.0 * math.pi)) * log_base
        ramp = 1.0 - np.clip((np.arange(int(dim_half), dtype=np.float64) - low) / (high - low), 0.0, 1.0)
        inv_freq = (1.0 - ramp) * (inv_freq / rope_scale) + ramp * inv_freq
    angles = np.einsum("i,j->ij", positions, inv_freq)
    return (np.cos(angles) * concentration).astype(np.float32), (np.sin(angles) * concentration).astype(np.float32)


def unit_rows(v: np.ndarray, mode: str = "fp32") -> np.ndarray:
    """model.py:353-354 - the new token's value rows scaled to unit length: v * rsqrt(sum(v^2) + 1e-10) in float32,
    held as a bf16 array by the JAX code (``mode="ref"`` rounds there)."""
    v32 = np.asarray(v, dtype=np.float32)
    vn = v32 * (np.float32(1.0) / np.sqrt(np.sum(v32 * v32, axis=-1, keepdims=True, dtype=np.float32) + np.float32(1e-10)))
    return bf16_round(vn) if mode == "ref" else vn.astype(np.float32)


def xsa(t: np.ndarray, current_v: np.ndarray, xsa_alpha: np.ndarray, mode: str = "fp32") -> np.ndarray:
    """model.py:351-363 (learned exclusive self attention) for one new token per sequence.

    t [B, N, H]: attention output after the output gate; current_v [B, K, H]: the new token's value rows as the
    projection produced them (not the cached, possibly quantised copy); xsa_alpha [N].  Query head n belongs to kv head
    n // (N // K).  With v^ the unit row of its kv head:  t - tanh(alpha_n) * <t, v^> * v^ .
    ``mode="ref"`` rounds to bf16 wherever the JAX code holds a bf16 array: v^, the elementwise product inside the
    inner product, the inner product, tanh(alpha), each of the two products and the difference.
    """
    t = np.asarray(t, dtype=np.float32)
    B, N, H = t.shape
    K = current_v.shape[1]
    G = N // K
    ref = mode == "ref"
    rnd = bf16_round if ref else (lambda a: np.asarray(a, dtype=np.float32))
    vn_g = unit_rows(current_v, mode)[:, :, None, :]                         # [B, K, 1, H]
    t_g = t.reshape(B, K, G, H)
    coef = np.sum(rnd(t_g * vn_g), axis=-1, keepdims=True, dtype=np.float32)  # float32 sum of (bf16) products
    alpha = rnd(np.tanh(np.asarray(xsa_alpha, dtype=np.float32))).reshape(1, K, G, 1)
    out = rnd(t_g - rnd(rnd(alpha * rnd(coef)) * vn_g))
    return out.reshape(B, N, H).astype(np.float32)


def route_tokens(logits: np.ndarray, n_active_routed: int, n_routed: int, n_shared: int):
    """model.py:459-478 on float32 router logits [F, n_routed] (bias already added).

    top-k is stable: among equal logits the lower index wins (lax.top_k).
    Returns scores [F, k+shared] f32, active_map [F*(k+shared)] int32, groups [E] int32.
    """
    logits = np.asarray(logits, dtype=np.float32)
    F = logits.shape[0]
    order = np.argsort(-logits, axis=-1, kind="stable")[:, :n_active_routed]
    top = np.take_along_axis(logits, order, axis=-1)
    e = np.exp(top - top.max(axis=-1, keepdims=True))
    scores = (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)
    indices = order.astype(np.int32)
    if n_shared:
        shared = np.broadcast_to(np.arange(n_routed, n_routed + n_shared, dtype=np.int32)[None, :], (F, n_shared))
        indices = np.concatenate([indices, shared], axis=-1)
        scores = np.concatenate([scores, np.ones((F, n_shared), dtype=np.float32)], axis=-1)
    active_map = indices.reshape(-1)
    groups = np.bincount(active_map, minlength=n_routed + n_shared).astype(np.int32)
    return scores, active_map, groups


def bpermute(expert_ids_: np.ndarray, group_sizes: np.ndarray, n_experts: int):
    """model.py:483-491 - stable counting sort of assignments by expert.

    destinations[i] = (start of expert e_i's rows) + (rank of i among earlier assignments to e_i)
    permutation     = inverse of destinations (row r of the sorted lhs takes assignment permutation[r]).
    """
    e = np.asarray(expert_ids_, dtype=np.int64)
    gs = np.asarray(group_sizes, dtype=np.int64)
    membership = np.zeros((e.shape[0], n_experts), dtype=np.int64)
    membership[np.arange(e.shape[0]), e] = 1
    local_rank = (np.cumsum(membership, axis=0) - 1)[np.arange(e.shape[0]), e]
    destinations = (np.cumsum(gs) - gs)[e] + local_rank
    permutation = np.empty_like(destinations)
    permutation[destinations] = np.arange(e.shape[0])
    return permutation.astype(np.int32), destinations.astype(np.int32)


def combine(rows: np.ndarray, scores: np.ndarray, unpermute_map: np.ndarray) -> np.ndarray:
    """model.py:557 - einsum("fkc,fk->fc", rows[unpermute].reshape(F,k,C), scores)."""
    F, k = scores.shape
    t = np.asarray(rows, dtype=np.float32)[unpermute_map].reshape(F, k, -1)
    return np.einsum("fkc,fk->fc", t, np.asarray(scores, dtype=np.float32), dtype=np.float32)


def sample_topk(logits: np.ndarray, uniforms: np.ndarray, k: int, temperature: float) -> np.ndarray:
    """lyra/generate.py:46-53 with temperature > 0, one row of ``logits`` [rows, V] per draw: logits / temperature,
    keep the k largest (lax.top_k: descending, ties to the lower index), categorical draw over their softmax.

    The reference draws with jax.random.categorical from its key stream; that stream cannot be reproduced here, so the
    draw is restated as the inverse CDF at ``uniforms`` [rows] in [0, 1), taken over the candidates in top_k order: the
    same distribution, a different (caller-supplied) source of randomness.  Returns int32 [rows].
    """
    x = np.asarray(logits, dtype=np.float32) / np.float32(temperature)
    rows, V = x.shape
    k = min(int(k), V)
    out = np.zeros(rows, np.int32)
    for r in range(rows):
        order = np.lexsort((np.arange(V), -x[r]))[:k]  # value descending, then index ascending
        e = np.exp(x[r, order] - x[r, order[0]], dtype=np.float32)
        target = np.float32(uniforms[r]) * np.float32(e.sum(dtype=np.float32))
        run, pick = np.float32(0.0), order[-1]
        for j in range(k):
            run = np.float32(run + e[j])
            if target < run:
                pick = order[j]
                break
        out[r] = pick
    return out
