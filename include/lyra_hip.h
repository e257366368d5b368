/*
 * liblyra_hip - C ABI of the MI355X (gfx950) decode kernels.
 *
 * The reference (ibbyml/lyra) has no FFI: its plugin seam is two Python callables chosen in
 * lyra/kernels/op.py:18-27.  Each entry point below names the reference callable it stands
 * behind.  All pointers are device pointers unless stated otherwise; every call is
 * asynchronous on `stream`, never synchronises, never allocates and keeps no state, so it is
 * re-entrant from any host thread.  Return value: 0 on success, a negative LYRA_E_* code
 * otherwise (nothing has been launched in that case).
 */
#ifndef LYRA_HIP_H
#define LYRA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LYRA_ABI_VERSION 15

/* element types of buffers that cross the ABI */
#define LYRA_DTYPE_BF16 0   /* bfloat16, 2 bytes */
#define LYRA_DTYPE_E4M3FN 1 /* OCP FP8 E4M3 (finite, max 448), 1 byte; needs scales */
#define LYRA_DTYPE_F32 2    /* float32 (outputs only) */
#define LYRA_DTYPE_E5M2 3   /* OCP FP8 E5M2 (max 57344), 1 byte; needs scales; accepted wherever e4m3fn is */
/* OR-ed into rhs_dtype of lyra_decode_gemm_ex / lyra_decode_gemm_partials: rhs is not the reference's [G,K,N] array but
 * the span-major copy of it that lyra_gemm_pack writes (layout 1 or 2 below). */
#define LYRA_RHS_SPAN_MAJOR 0x100     /* layout 1: spans of 128 consecutive columns */
#define LYRA_RHS_SPAN_MAJOR_GLU 0x200 /* layout 2: spans of 64 gate columns + their 64 linear columns (fused_swiglu) */
/* ... and, likewise OR-ed into rhs_dtype: bf16 activations in tiles of 16 rows x 32 columns (1 KB each; the tiles of 16 rows
 * side by side, then the next 16 rows): element (r, c) of an array of C columns (C % 32 == 0) lies at
 *   (((r >> 4) * (C >> 5) + (c >> 5)) * 16 + (r & 15)) * 32 + (c & 31),
 * with room for the rows rounded up to 16.  The 16 lanes that feed one matrix instruction with 16 consecutive rows then
 * read one contiguous KB instead of 16 pieces a row apart, which is what workgroups with many rows (a shared expert's
 * units, the 32- and 64-row blocks of the K-split projections) spend their extra time on.  An internal layout of a fused
 * decode step: lyra_rmsnorm_proj (mode | 4) and the calls below with LYRA_OUT_TILED16 write it, no reference array has it. */
#define LYRA_LHS_TILED16 0x400 /* lhs is tiled: lyra_decode_gemm_ex with several groups or a K-split plan, lyra_decode_gemm_partials */
#define LYRA_OUT_TILED16 0x800 /* out is written tiled (bf16, no residual, output width % 32 == 0): lyra_decode_gemm_ex, same plans */

#define LYRA_OK 0
#define LYRA_E_BADARG (-1)      /* null pointer, non-positive size, N % K != 0 ... */
#define LYRA_E_UNSUPPORTED (-2) /* a shape or dtype the kernels do not cover */
#define LYRA_E_WORKSPACE (-3)   /* workspace pointer missing or too small */
#define LYRA_E_LAUNCH (-4)      /* the HIP runtime refused the launch */
#define LYRA_E_SCRATCH (-5)     /* lyra_decode_attention_static: the call needs more than the static scratch buffer */

typedef void* lyra_stream_t; /* a hipStream_t; NULL = the default stream */

int lyra_abi_version(void);
const char* lyra_strerror(int code);

/*
 * Decode attention: one query token per sequence against the KV cache.
 * Stands behind lyra.kernels.decode_attention.decode_attention
 * (lyra/kernels/decode_attention.py:364-415; maths of decode_attention_reference :311-361
 * and sliding_decode :263-308).
 *
 *   q        [B,N,H] bf16                      (the reference's [B,N,1,H])
 *   k, v     [B,K,S,H] bf16, e4m3fn or e5m2 (both FP8_DTYPES of lyra/nn/quant.py:10), contiguous; kv head of query head n is n / (N/K)
 *   k_scale, v_scale   [B,K,S] float32, one per cached token and kv head (QArray block (1,H),
 *            lyra/model.py:225); NULL iff kv_dtype == LYRA_DTYPE_BF16
 *   sinks    [N] float32 learned sink logits (a virtual key with value 0)
 *   position int32; element b*position_stride is the index of the newest token of row b; keys
 *            0..position are visible (minus the window).  position_stride 0 = one scalar for the
 *            whole batch (the reference's only mode), 1 = ragged batch.  A ragged batch without a window and
 *            with more than 256 (row, kv head) pairs (B <= 256) is worked through longest rows first by
 *            resident workgroups; results do not depend on which launch is taken beyond float32
 *            summation order.
 *   gate     [B,N] bf16 or NULL; out = bf16(bf16(attn) * gate)  (lyra/model.py:343-347)
 *   out      [B,N,H] out_dtype (bf16 or float32)
 *   sliding_window  0 = global layer; w > 0 = only keys j with position-w < j <= position
 *   sm_scale        multiplies q.k (the reference passes H**-0.5)
 *   workspace       at least lyra_decode_attention_workspace(...) bytes, 256-byte aligned.  It holds split
 *                   partials and arrival counters.  The counters must read zero when a call starts and are
 *                   zero again when it ends: zero the buffer once after allocating it (lyra_workspace_init
 *                   or any memset) and it can be reused by every later call, of any shape, on the same stream,
 *                   as long as nothing else writes to it in between.
 * Supported: H in {64,128}; 1 <= N/K <= 16; any B, S >= 1.
 */
int lyra_decode_attention(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                          const float* sinks, const int32_t* position, int position_stride, const void* gate,
                          void* out, void* workspace, size_t workspace_bytes, int B, int N, int K, int S, int H,
                          float sm_scale, int sliding_window, int kv_dtype, int out_dtype, lyra_stream_t stream);

size_t lyra_decode_attention_workspace(int B, int N, int K, int S, int H, int sliding_window);

/*
 * lyra_decode_attention followed, in the same launch, by the model's learned exclusive self attention
 * (lyra/model.py:351-363, enabled by use_learned_xsa, lyra/variants.py:38): after the output gate every query head n
 * loses a learned share of its component along the new token's own value row,
 *     out = t - tanh(xsa_alpha[n]) * <t, v^> * v^,     v^ = v_unit[b, n / (N/K), :]
 *   v_unit    [B,K,H] bf16: the new token's value rows before cache quantisation, scaled to unit length
 *             (lyra_qkv_post writes it)
 *   xsa_alpha [N] float32
 * Both NULL: exactly lyra_decode_attention.  A bf16 output is rounded wherever the JAX code holds a bf16 array (the
 * products inside the inner product, the inner product, tanh(alpha), both products, the difference).
 */
int lyra_decode_attention_xsa(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                              const float* sinks, const int32_t* position, int position_stride, const void* gate,
                              const void* v_unit, const float* xsa_alpha, void* out, void* workspace, size_t workspace_bytes,
                              int B, int N, int K, int S, int H, float sm_scale, int sliding_window, int kv_dtype,
                              int out_dtype, lyra_stream_t stream);

/*
 * lyra_qkv_post_sum and lyra_decode_attention in one launch: what lies between the fused q/k/v projection and the output
 * projection of an attention layer (lyra/model.py:309-347: QK norm, rotary embedding, cache_update :204-212 / qupdate
 * lyra/nn/quant.py:89-98, decode_attention with the output gate).  Every workgroup of the attention kernel first builds
 * the q rows of its kv head from the projection, and the workgroup whose keys include the new token's appends that
 * token's key and value rows to the caches before it reads them.  Arguments as in lyra_qkv_post_sum (qkv / partials /
 * splits, qnorm, knorm, cos_t, sin_t, rope_rows, eps) and lyra_decode_attention; k, v, k_scale, v_scale are written at
 * index position[b] (rows with a position outside [0,S) are not appended).  q is never materialised.
 * Results and cache contents are bit-identical to the two calls.  LYRA_E_UNSUPPORTED (nothing launched) for a ragged
 * batch without a window and with more than 256 (row, kv head) pairs, which lyra_decode_attention hands to its whole-row
 * kernel: call the two entry points then.  No learned exclusive self attention here (lyra_decode_attention_xsa needs the
 * v_unit rows lyra_qkv_post writes).
 */
int lyra_decode_attention_qkv(const void* qkv, const float* partials, int splits, const float* qnorm, const float* knorm,
                              const float* cos_t, const float* sin_t, int rope_rows, float eps, void* k, void* v,
                              float* k_scale, float* v_scale, const float* sinks, const int32_t* position,
                              int position_stride, const void* gate, void* out, void* workspace, size_t workspace_bytes,
                              int B, int N, int K, int S, int H, float sm_scale, int sliding_window, int kv_dtype,
                              int out_dtype, lyra_stream_t stream);
/*
 * The same for a q/k/v projection that has a bias (lyra/model.py:310-313: added to the projection's bf16 result, in
 * bf16) and is handed over as unsummed slices: qkv_bias [(N + 2K) * H] float32 holding bf16 values; every head row is
 * bf16(bf16(sum of slices) + bias) before the QK norm, as lyra_decode_gemm_ex with bit 1 of post_scale leaves it.  Saves
 * the launch that would sum the slices only to add the bias.  qkv_bias needs partials (a summed projection carries its
 * bias already); null = lyra_decode_attention_qkv.
 */
int lyra_decode_attention_qkv_bias(const void* qkv, const float* partials, int splits, const float* qkv_bias, const float* qnorm,
                                   const float* knorm, const float* cos_t, const float* sin_t, int rope_rows, float eps, void* k,
                                   void* v, float* k_scale, float* v_scale, const float* sinks, const int32_t* position,
                                   int position_stride, const void* gate, void* out, void* workspace, size_t workspace_bytes,
                                   int B, int N, int K, int S, int H, float sm_scale, int sliding_window, int kv_dtype,
                                   int out_dtype, lyra_stream_t stream);

/*
 * Ragged batches, rows dealt out by length (an extension of the boundary, like position_stride 1: the reference passes one
 * position for the whole batch, lyra/kernels/decode_attention.py:364-375).  With more (row, kv head) pairs than compute
 * units, which workgroup takes which pair decides how long a launch lasts.  The order of the rows by length changes
 * only when the batch does - every row grows by one token per step - so it is computed once per step, or once per
 * batch, by lyra_attention_rank and handed to every layer's launch:
 *   lyra_attention_rank           row_order[i] = the row with the i-th largest position (ties: lower row first); B <= 8192
 *   lyra_decode_attention_ranked  lyra_decode_attention with that order: the unchunked global-layer launch (position_stride 1,
 *                                 more than 256 pairs) gives the workgroups that share a compute unit the i-th longest and
 *                                 the i-th shortest pair; every other launch ignores the order.  row_order must be a
 *                                 permutation of 0..B-1 (it is not checked); any permutation gives the same results.
 */
int lyra_attention_rank(const int32_t* position, int B, int32_t* row_order, lyra_stream_t stream);
int lyra_decode_attention_ranked(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                 const float* sinks, const int32_t* position, int position_stride, const int32_t* row_order,
                                 const void* gate, void* out, void* workspace, size_t workspace_bytes, int B, int N, int K, int S,
                                 int H, float sm_scale, int sliding_window, int kv_dtype, int out_dtype, lyra_stream_t stream);

/*
 * lyra_decode_attention for callers that cannot allocate device memory or hand over a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments, same kernels and bit-identical results as lyra_decode_attention, minus the workspace: split partials
 * and arrival counters live in a device array of LYRA_STATIC_SCRATCH_BYTES that is part of the library's code object
 * (every GPU the library runs on holds one copy until the process ends).  The call allocates and frees nothing; the
 * first call on a device looks up the array's device address, so make that call outside a capture.  A launch that is
 * not chunked (many (row, kv head) pairs, or a short window) does not touch the array.  A shape whose partials do not
 * fit answers LYRA_E_SCRATCH and launches nothing: use lyra_decode_attention with a workspace for it.  The plan
 * aims at about 256 workgroups per launch, so only launches with 16 query heads per kv head, head size 128 and
 * close to 256 (row, kv head) pairs exceed the 4 MiB (lyra_decode_attention_workspace tells the need of a shape).
 * All calls on one GPU share the array, and the counters a call uses are cleared at its start (a fill kernel on
 * `stream`): calls that overlap on one GPU - different streams, or different host threads without ordering - race.
 */
#define LYRA_STATIC_SCRATCH_BYTES (4u << 20)
int lyra_decode_attention_static(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                 const float* sinks, const int32_t* position, int position_stride, const void* gate,
                                 void* out, int B, int N, int K, int S, int H, float sm_scale, int sliding_window,
                                 int kv_dtype, int out_dtype, lyra_stream_t stream);

/*
 * Zero `workspace_bytes` (a multiple of 4) of a workspace with a fill kernel on `stream` (safe to record
 * into a HIP graph).  No counterpart in the reference; needed once per workspace allocation.
 */
int lyra_workspace_init(void* workspace, size_t workspace_bytes, lyra_stream_t stream);

/*
 * Decode grouped matmul: out[r,:] = epilogue(lhs[r,:] @ rhs[e(r)]) with rows sorted by group.
 * Stands behind lyra.kernels.decode_gemm.decode_gemm (lyra/kernels/decode_gemm.py:404-474;
 * maths of grouped_gemm_reference, lyra/kernels/gemm.py:1575-1617) and, with G == 1, behind
 * lyra.nn.quant.dot for the dense projections (lyra/nn/quant.py:106-108).
 *
 *   lhs         [M,K] bf16
 *   rhs         [G,K,N] bf16, e4m3fn or e5m2, contiguous
 *   rhs_scale   [G,K/bk,N/bn] float32 block scales (QArray block (bk,bn)); NULL iff rhs is bf16.
 *               bk == K, bn == 1 is the per-output-channel layout.
 *   group_sizes [G] int32 on the device; rows of group g are [sum(sizes[:g]), +sizes[g]).
 *               Experts with no rows are never read.  Rows at or beyond sum(sizes) produce
 *               epilogue(0) with the bias of group G-1 (lax.ragged_dot + gemm.py:450-456).
 *   bias        [G,N] float32 or NULL, added in float32 before SwiGLU
 *   fused_swiglu  out[:, j] = (clip(t[:, N/2+j], +-limit) + 1) * g * sigmoid(beta*g),
 *               g = min(t[:, j], limit)  (lyra/kernels/common.py:98-114); out is then [M,N/2]
 *   out         [M,N] or [M,N/2], out_dtype (bf16 or float32)
 *   workspace   at least lyra_decode_gemm_workspace(...) bytes, 256-byte aligned.  Its first 64 KiB hold arrival
 *               counters (units cut into K slices meet there): zero the buffer once after allocating it
 *               (lyra_workspace_init); every call leaves the counters at zero.  Float32 partial products follow.
 * Supported: K % 32 == 0, N % 8 == 0 (N % 16 == 0 with fused_swiglu), G <= 8191; fp8 blocks with bn a
 * power of two, and either (bn % 8 == 0 and (bk % 32 == 0 or bk == K)) or bk == K.  N need not fill its last
 * 128-column span (the reference's kernel wants n % 128 == 0, decode_gemm.py:88, and otherwise takes its XLA path).
 */
int lyra_decode_gemm(const void* lhs, const void* rhs, const float* rhs_scale, int bk, int bn,
                     const int32_t* group_sizes, const float* bias, void* out, void* workspace,
                     size_t workspace_bytes, int M, int G, int K, int N, int rhs_dtype, int out_dtype,
                     int fused_swiglu, float swiglu_beta, float swiglu_limit, lyra_stream_t stream);

size_t lyra_decode_gemm_workspace(int M, int G, int K, int N, int fused_swiglu);
/*
 * Exact workspace bytes of a call whose weights carry scale blocks of bk rows (0 = bf16 weights or one scale per
 * column): what lyra_decode_gemm(_ex) checks workspace_bytes against.  Never more than lyra_decode_gemm_workspace,
 * which covers every scale block of the shape.
 */
size_t lyra_decode_gemm_workspace_for(int M, int G, int K, int N, int bk, int fused_swiglu);

/*
 * lyra_decode_gemm with the two neighbouring model steps fused in (no counterpart kernel in the reference; the
 * model code around its two matmul call sites, lyra/model.py:371-374, 536-567, 631-636):
 *   lhs_row_map [M] int32 or NULL: sorted row r reads lhs[lhs_row_map[r], :] - the token gather that feeds the
 *               expert up-projection (x[permute_map // topk], model.py:536-540); lhs then has as many rows as
 *               the map addresses.
 *   post_scale  bit 0: out = bf16(residual + bf16(bf16(t) * out_scale)), t the plain result - a projection's
 *               output scaled in bf16 and added to the residual stream; residual [M,N] bf16 or NULL (scale only).
 *               residual requires bit 0 and a bf16 output.
 *               bit 1 (one group, no fused_swiglu, bf16 output, bias given): the bias is added after the cast,
 *               t = bf16(bf16(product) + bias), as the model does for the q/k/v, output and dense down
 *               projections (model.py:310-313, 367-368, 629-630: a bf16 bias added to the operator's bf16
 *               result); without it the bias is added to the float32 product (gemm.py:1600-1605).
 *   rhs_dtype   may carry LYRA_RHS_SPAN_MAJOR(_GLU), LYRA_LHS_TILED16 and LYRA_OUT_TILED16 (above).
 */
int lyra_decode_gemm_ex(const void* lhs, const int32_t* lhs_row_map, const void* rhs, const float* rhs_scale, int bk,
                        int bn, const int32_t* group_sizes, const float* bias, const void* residual, float out_scale,
                        int post_scale, void* out, void* workspace, size_t workspace_bytes, int M, int G, int K, int N,
                        int rhs_dtype, int out_dtype, int fused_swiglu, float swiglu_beta, float swiglu_limit,
                        lyra_stream_t stream);

/*
 * Span-major weights (no counterpart in the reference, whose kernels read [G,K,N] as it is: lyra/kernels/decode_gemm.py:
 * 145-298).  A decode matmul streams, per workgroup, one 128-column span of a weight matrix from its first K row to its
 * last; in the row-major [G,K,N] array those are 128-byte pieces N bytes apart - and pieces that straddle two cache
 * lines whenever N (or N/2, where the linear half of a SwiGLU projection starts) is not a multiple of 128 bytes, as
 * with gpt-oss-20b's width 2880.  lyra_gemm_pack copies the weights once, at load time, so that every span is one
 * contiguous, 128-byte aligned run of K rows of 128 elements:
 *   layout 1 (LYRA_RHS_SPAN_MAJOR):      packed[g][s][k][c] = rhs[g][k][128 s + c],           s < ceil(N / 128)
 *   layout 2 (LYRA_RHS_SPAN_MAJOR_GLU):  packed[g][s][k][c] = rhs[g][k][64 s + c]             (c < 64: gate column)
 *                                                          = rhs[g][k][N/2 + 64 s + c - 64]   (c >= 64: its linear column),
 *                                                                                            s < ceil(N / 2 / 64)
 * with zeros where the column does not exist (a last span that N does not fill).  Scales, biases and outputs keep the
 * reference's column order.  lyra_decode_gemm_ex takes layout 2 for several groups with fused_swiglu, layout 1 for
 * several groups without, for the K-split projections of one group (with or without fused_swiglu) and for the
 * general kernel without fused_swiglu (the LM head, also through lyra_decode_gemm_tile_max: bit-identical results; a
 * wavefront then walks one contiguous run instead of K pieces N elements apart), and answers
 * LYRA_E_UNSUPPORTED for any other combination; lyra_decode_gemm_partials takes layout 1.  Results are the same
 * function of the same weights; the float32 summation order over K may differ from the row-major call's.
 *   lyra_gemm_packed_bytes  size of the packed copy (0 for bad arguments)
 *   lyra_gemm_pack          rhs [G,K,N] (rhs_dtype bf16, e4m3fn or e5m2) -> packed; layout 1 or 2; N % 8 == 0 (16 for layout 2)
 */
size_t lyra_gemm_packed_bytes(int G, int K, int N, int rhs_dtype, int layout);
int lyra_gemm_pack(const void* rhs, void* packed, int G, int K, int N, int rhs_dtype, int layout, lyra_stream_t stream);

/*
 * A dense projection (one group, a few MB of weights) runs split over K across all compute units; the float32
 * slices [splits, M, N] are summed by whoever consumes the result.  lyra_decode_gemm(_ex) sums them itself in a
 * second launch.  A decode step saves that launch by handing the unsummed slices to the next kernel of the layer
 * (lyra_qkv_post_sum after the q/k/v projection, lyra_rmsnorm_proj_sum after the output and down projections):
 *   lyra_decode_gemm_splits    number of slices for (M, K, N, bk) - shape only; 0 = this shape does not run split
 *   lyra_decode_gemm_partials  partials[s] = lhs[:, slice s] @ rhs[slice s, :] (weight scales applied), no epilogue;
 *                              partials holds splits * M * N floats, 16-byte aligned.
 * The sum over slices is taken in slice order in float32, then rounded as the projection's bf16 output would be.
 * K % 32 == 0, N % 8 == 0 (a last 128-column span that N does not fill is fine).  A projection with a bias of its own
 * hands the bias to the consumer too: lyra_decode_attention_qkv_bias, lyra_rmsnorm_proj_sum_bias.
 */
int lyra_decode_gemm_splits(int M, int K, int N, int bk);
int lyra_decode_gemm_partials(const void* lhs, const void* rhs, const float* rhs_scale, int bk, int bn,
                              const int32_t* group_sizes, float* partials, size_t partials_bytes, int M, int K, int N,
                              int rhs_dtype, lyra_stream_t stream);

/*
 * The elementwise steps of a decode layer between the two kernels above, one launch each.  They follow the
 * reference's dtype flow exactly: float32 arithmetic inside an op, a bf16 rounding wherever its JAX code holds a
 * bf16 array.
 *
 * lyra_rmsnorm_proj: h = bf16(x * rsqrt(mean(x^2) + eps) * scale) (lyra/model.py:189-191), optionally followed by a
 *   narrow float32 projection of f32(h): y[j] = sum_c h[c] * proj_t[j,c] (+ bias[j]); proj_t [n,C] float32 is the
 *   reference's [C,n] parameter transposed once at load time so that each output reads a contiguous row.  C % 4 == 0.
 *   mode 1: y -> bf16(2 * sigmoid(y)), the per-head output gate (model.py:343-347), y is bf16 [B,n];
 *   mode 2: y float32 [B,n], the router logits (model.py:455-457).  proj_t NULL: norm only.
 *   mode | 4: h is written in tiles of 16 rows x 32 columns (LYRA_LHS_TILED16 above; C % 32 == 0), for the matmul behind it.
 */
int lyra_rmsnorm_proj(const void* x, const float* scale, void* h, const float* proj_t, const float* bias, void* y, int B, int C,
                      int n, int mode, float eps, lyra_stream_t stream);
/* Same, but the row to normalise is first formed from unsummed projection slices (lyra/model.py:371-374, 631-636):
 * x_out = bf16(residual + bf16(bf16(sum_s partials[s]) * out_scale)), partials [splits, B, C] float32; x is ignored.
 * x_out and h must not overlap the inputs (several workgroups read a row while one of them writes its outputs). */
int lyra_rmsnorm_proj_sum(const void* x, const float* partials, int splits, const void* residual, float out_scale, void* x_out,
                          const float* scale, void* h, const float* proj_t, const float* bias, void* y, int B, int C, int n,
                          int mode, float eps, lyra_stream_t stream);
/* Same for a projection with a bias of its own (output and dense-down projections of the gpt-oss variants,
 * lyra/model.py:367-368, 629-630): sum_bias [C] float32 holding bf16 values, and
 * x_out = bf16(residual + bf16(bf16(bf16(sum of slices) + sum_bias) * out_scale)), what lyra_decode_gemm_ex with bit 1 of
 * post_scale and the residual epilogue gives; null = lyra_rmsnorm_proj_sum. */
int lyra_rmsnorm_proj_sum_bias(const void* x, const float* partials, int splits, const float* sum_bias, const void* residual,
                               float out_scale, void* x_out, const float* scale, void* h, const float* proj_t, const float* bias,
                               void* y, int B, int C, int n, int mode, float eps, lyra_stream_t stream);
/* Same, but the row to normalise is the residual update that ends a MoE layer (lyra/model.py:557-567; what lyra_moe_combine
 * computes): x_out = bf16(residual + bf16(bf16(sum_k scores[b,k] * rows[dest[b*topk+k]]) * out_scale)), rows [B*topk, C]
 * bf16 in sorted order, scores [B, topk] float32, dest [B*topk] int32, topk <= 16.  Same aliasing rule. */
/* Same for the first layer of a step: row b is the embedding row table[tokens[b]] (the gather of lyra/model.py:752; table
 * [table_rows, C] bf16, tokens [B] int32), also copied to x_out [B,C] as the residual stream.  A token id outside
 * [0, table_rows) is clamped into the range (jnp.take's "clip" mode; the reference's default mode fills such rows with NaN,
 * lyra/model.py:747): the kernel never reads outside the table. */
int lyra_rmsnorm_proj_embed(const void* table, const int32_t* tokens, int table_rows, void* x_out, const float* scale, void* h,
                            const float* proj_t, const float* bias, void* y, int B, int C, int n, int mode, float eps,
                            lyra_stream_t stream);
int lyra_rmsnorm_proj_combine(const void* rows, const float* scores, const int32_t* dest, int topk, const void* residual,
                              float out_scale, void* x_out, const float* scale, void* h, const float* proj_t, const float* bias,
                              void* y, int B, int C, int n, int mode, float eps, lyra_stream_t stream);

/*
 * lyra_qkv_post: everything between the fused q/k/v projection and the attention kernel (model.py:309-336):
 *   qkv [B,(N+2K)*H] bf16 -> per head rms_norm (qnorm/knorm [H] float32, both NULL = no QK norm) -> half-split
 *   rotary embedding with row position[b] of cos_t/sin_t [rope_rows, H/2] float32 (model.py:183-186) -> q_out
 *   [B,N,H] bf16; k and v rows are appended to the caches [B,K,S,H] at index position[b]: copied (bf16) or
 *   quantised with one scale per row, scale = amax/fmax (1 for a zero row; fmax 448 for e4m3fn, 57344 for e5m2), code = fp8_rne(clip(x/scale))
 *   (lyra/nn/quant.py:68-72, 213-231), scales into k_scale/v_scale [B,K,S].  Rows with position outside [0,S)
 *   are not appended.  H in {64,128}.
 *   v_unit [B,K,H] bf16 or NULL: receives the new value rows scaled to unit length, bf16(v * rsqrt(sum(v^2) + 1e-10))
 *   (model.py:353-354), which lyra_decode_attention_xsa takes.
 */
int lyra_qkv_post(const void* qkv, const float* qnorm, const float* knorm, const float* cos_t, const float* sin_t,
                  const int32_t* position, int position_stride, void* q_out, void* k_cache, void* v_cache, float* k_scale,
                  float* v_scale, void* v_unit, int B, int N, int K, int S, int H, int rope_rows, int kv_dtype, float eps,
                  lyra_stream_t stream);
/* Same, reading the projection as unsummed slices partials [splits, B, (N+2K)*H] float32 (qkv is ignored). */
int lyra_qkv_post_sum(const void* qkv, const float* partials, int splits, const float* qnorm, const float* knorm,
                      const float* cos_t, const float* sin_t, const int32_t* position, int position_stride, void* q_out,
                      void* k_cache, void* v_cache, float* k_scale, float* v_scale, void* v_unit, int B, int N, int K, int S,
                      int H, int rope_rows, int kv_dtype, float eps, lyra_stream_t stream);

/*
 * lyra_moe_route: router top-k, softmax over the chosen logits, shared experts appended with score 1, and the stable
 * sort of assignments by expert (model.py:459-491, 393-417).  logits [tokens,n_routed] float32 ->
 *   scores [tokens,topk] float32, groups [E] int32 (rows per expert), row_map [tokens*topk] int32 (token of each
 *   sorted row = permute_map // topk), dest [tokens*topk] int32 (sorted row of each assignment = unpermute_map);
 *   topk = k_routed + n_shared, E = n_routed + n_shared.  k_routed <= 8, n_routed <= 128.
 *
 * lyra_moe_combine: out[f] = bf16(x[f] + bf16(bf16(sum_k scores[f,k] * rows[dest[f*topk+k]]) * residual_scale))
 *   (model.py:557-567); rows [tokens*topk,C] bf16 in sorted order, x/out [tokens,C] bf16.
 */
int lyra_moe_route(const float* logits, float* scores, int32_t* groups, int32_t* row_map, int32_t* dest, int tokens,
                   int n_routed, int n_shared, int k_routed, lyra_stream_t stream);
int lyra_moe_combine(const void* rows, const float* scores, const int32_t* dest, const void* x, void* out, int tokens, int topk,
                     int C, float residual_scale, lyra_stream_t stream);

/*
 * Greedy sampling (lyra/generate.py:46-53 with temperature <= 0): out[r] = first index of the maximum of
 * x[r, 0:cols], x float32 [rows, ld] (ld >= cols is the padded vocabulary; the padding is not looked at).
 * workspace: lyra_argmax_workspace bytes, 256-byte aligned, zero on first use (it holds arrival counters that
 * every call returns to zero, like the attention workspace).  ld % 4 == 0, x 16-byte aligned.
 * advance (or NULL): an int32 on the device that the launch increments by one once row 0 is decided - the cache position,
 * when the sampler is the last kernel of a decode step (lyra/generate.py:64-85 feeds position + 1 to the next step), so
 * that a captured step can be replayed token after token without host work in between.
 */
int lyra_argmax(const float* x, int32_t* out, void* workspace, size_t workspace_bytes, int rows, int cols, int ld,
                int32_t* advance, lyra_stream_t stream);
size_t lyra_argmax_workspace(int rows, int cols);

/*
 * Temperature / top-k sampling (lyra/generate.py:46-53 with temperature > 0): per row, the k largest of
 * x[r, 0:cols] / temperature (ties go to the lower index, as lax.top_k), softmax over them, and the inverse CDF at
 * uniforms[r] in [0, 1) taken in that order: out[r] = index of the drawn column.  The reference draws with
 * jax.random.categorical from its own key stream; the distribution is the same, the caller supplies the randomness.
 * 1 <= k <= 8; x float32 [rows, ld], ld % 4 == 0, 16-byte aligned; workspace and advance as for lyra_argmax.
 */
int lyra_sample_topk(const float* x, const float* uniforms, int32_t* out, void* workspace, size_t workspace_bytes, int rows,
                     int cols, int ld, int k, float temperature, int32_t* advance, lyra_stream_t stream);
size_t lyra_sample_topk_workspace(int rows, int cols, int k);
/*
 * The same draw with the uniform numbers made inside the launch, so that a captured decode step needs no generator
 * launches of its own: rng is a device array of two uint64, {seed, count}; row r takes
 *   u = (splitmix64(seed ^ (count + 1) * 0x9E3779B97F4A7C15 ^ (r + 1) * 0xD1B54A32D192ED03) >> 40) * 2^-24
 * (splitmix64(z): z = (z ^ z >> 30) * 0xBF58476D1CE4E5B9; z = (z ^ z >> 27) * 0x94D049BB133111EB; z ^ z >> 31), and the
 * launch leaves count + 1 behind once every workgroup has read count.  Like the reference's key stream
 * (lyra/generate.py:53, jax.random.categorical) this is a stream of its own: same distribution, other numbers.
 */
int lyra_sample_topk_rng(const float* x, uint64_t* rng, int32_t* out, void* workspace, size_t workspace_bytes, int rows, int cols,
                         int ld, int k, float temperature, int32_t* advance, lyra_stream_t stream);
/*
 * Samplers for logits whose matmul also left the maximum of every 128-column tile of every row.
 * lyra_decode_gemm_tile_max is lyra_decode_gemm_ex without the residual / scale epilogue and without SwiGLU, for the
 * shapes its plain kernel takes (one group whose weights are too many for the K-split kernel - the LM head,
 * lyra/model.py:784-790 - float32 output): besides `out` it writes tile_max [M, (N + 127) / 128] float32, the maximum
 * of out[row, 128 t .. 128 t + 127] with the bias added, NaNs skipped; LYRA_E_UNSUPPORTED for any other shape (call
 * lyra_decode_gemm_ex and the samplers above).  lyra_argmax_tiles / lyra_sample_topk_tiles return what lyra_argmax /
 * lyra_sample_topk (uniforms given, rng null) / lyra_sample_topk_rng (rng given, uniforms null) return on the same
 * logits, from one launch of one workgroup per row that reads the row's tile maxima and only the tiles that can hold
 * its k best values: 64 x 201088 logits in 6 us instead of 27.  tile_ld: row pitch of tile_max (>= (cols + 127) / 128).
 * The workspace is only used with rng (lyra_sample_topk_workspace bytes, may be the one lyra_sample_topk_rng uses).
 * The logits must be as the matmul left them.
 */
int lyra_decode_gemm_tile_max(const void* lhs, const int32_t* lhs_row_map, const void* rhs, const float* rhs_scale, int bk, int bn,
                              const int32_t* group_sizes, const float* bias, void* out, float* tile_max, void* workspace,
                              size_t workspace_bytes, int M, int G, int K, int N, int rhs_dtype, int out_dtype,
                              lyra_stream_t stream);
int lyra_argmax_tiles(const float* x, const float* tile_max, int32_t* out, int rows, int cols, int ld, int tile_ld,
                      int32_t* advance, lyra_stream_t stream);
int lyra_sample_topk_tiles(const float* x, const float* tile_max, const float* uniforms, uint64_t* rng, int32_t* out,
                           void* workspace, size_t workspace_bytes, int rows, int cols, int ld, int tile_ld, int k,
                           float temperature, int32_t* advance, lyra_stream_t stream);


/*
 * Self-check of the matrix-core register layouts and FP8 conversions the kernels rely on.
 * `report` (device, >= 8 int32) receives mismatch counts; all zeros = pass.  Test hook only.
 */
int lyra_selftest(int32_t* report, lyra_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LYRA_HIP_H */
