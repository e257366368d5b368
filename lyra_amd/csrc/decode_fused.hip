// Small fused kernels around the two decode hot kernels: everything the reference's model code does between
// them for one new token per sequence (lyra/model.py:284-374, 451-567), so that a decode step is a few launches
// per layer instead of hundreds of elementwise ones.  All arithmetic follows the reference's dtype flow: bf16
// activations, float32 maths inside an op, a bf16 rounding wherever the JAX code holds a bf16 array.
#include <algorithm>
#include <cstdlib>

#include <climits>

#include "lyra_device.h"

namespace lyra {

__device__ __forceinline__ float block_sum(float v, float* sm) {  // blockDim.x <= 1024, multiple of 64; sm: 16 floats nobody else uses
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    if (lane == 0) sm[wave] = v;
    __syncthreads();
    float t = lane < nw ? sm[lane] : 0.f;
    return wave_sum(t);
}

// ---- RMS norm (+ a narrow float32 projection of the normalised row) ---------------------------------------
// h = bf16(x * rsqrt(mean(x^2) + eps) * scale)                      lyra/model.py:189-191
// y[j] = sum_c f32(h[c]) * Pt[j, c] (+ bias[j]), j < n               router logits (model.py:455-457) or the
// gate = bf16(2 * sigmoid(y))                                        output gate (model.py:343-347)
// One workgroup per row.  The normalised row stays in LDS; each wavefront then takes output columns in turn and
// reads that column's weights (a contiguous row of the transposed projection) 16 bytes per lane.
struct NormProjParams {
    const uint16_t* x;
    const float* scale;
    uint16_t* h;
    const float* proj_t;  // [n, C] or null
    const float* bias;    // [n] or null
    void* y;              // mode 1: bf16 [B, n] gate; mode 2: float32 [B, n]
    int C, n, mode;
    float eps;
    // optional: the row to normalise is not x but bf16(residual + bf16(bf16(sum_s partials[s]) * out_scale)), the
    // residual update that follows a projection whose K slices have not been summed yet; it is written to x_out
    const float* partials;  // [splits, B, C] or null
    int splits, B;
    const uint16_t* residual;
    float out_scale;
    uint16_t* x_out;
    // or: the row is the residual update that ends a MoE layer (lyra/model.py:557-567),
    // bf16(residual + bf16(bf16(sum_k scores[b,k] * rows[dest[b,k]]) * out_scale)), also written to x_out
    const uint16_t* comb_rows;  // [B * topk, C] expert outputs in sorted order, or null
    const float* comb_scores;   // [B, topk]
    const int32_t* comb_dest;   // [B, topk] sorted row of every assignment
    int comb_topk;              // <= 16
    // or: row b is row row_index[b] of x (the embedding table: the token gather of lyra/model.py:752), copied to x_out
    const int32_t* row_index;   // [B] or null
    int row_limit;              // rows of x when row_index is set: an index outside [0, row_limit) is clamped into it, so a
                                // bad token id (padding such as -1, a stale buffer) reads a valid row instead of faulting
    // with `partials`: the projection's bias [C] (bf16 values as float32), added to the bf16-rounded sum in bf16 before the
    // scale / residual step (lyra/model.py:367-368, 629-630), or null
    const float* sum_bias;
    int per_share;  // projection outputs per workgroup of a row: ceil(n / shares), set by the launch
};

constexpr int kNormThreads = 1024;

// COMBINE: the instantiation whose rows come from a MoE layer's combine step (comb_rows set).
template <bool COMBINE>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_proj_kernel(NormProjParams p) {
    extern __shared__ __align__(16) float sm_h[];  // [C] normalised row (bf16 values as float32), then 16 floats of reduction scratch
    float* sm_red = sm_h + p.C;
    // blockIdx.y: which share of the projection outputs this workgroup computes.  The shares of a row each normalise the
    // row again (cheap: the input comes from L2) so that the projection matrix, which every row needs in full, is pulled
    // through 4 compute units per row instead of one; share 0 writes the row's other outputs.
    const int b = blockIdx.x, share = blockIdx.y, shares = gridDim.y;
    // The weights of the first projection output of this wavefront do not depend on the row: they are requested before
    // anything else, so that they arrive while the row is being read and normalised (otherwise the projection is a
    // second memory round trip behind the norm: 1.4 us of a 4.7 us launch).
    const int per_share = p.per_share, j_end = min(p.n, (share + 1) * per_share);  // (ceil(n / shares), divided on the host)
    const int j_first = share * per_share + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // (the same in every lane)
    u32x4 w_first[8];
    if (p.proj_t && j_first < j_end) {  // (only the wavefronts that have an output: a load that fetches nothing still takes its
        const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(  // turn in the address unit)
            const_cast<float*>(p.proj_t) + (size_t)j_first * p.C, 0, (uint32_t)p.C * 4u, 0x00020000);
#pragma unroll
        for (int i = 0; i < 8; ++i) w_first[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, (i * 256 + (int)(threadIdx.x & 63) * 4) * 4, 0, 0);
    }
    const uint16_t* xr = p.x + (size_t)(p.row_index ? min(max(p.row_index[b], 0), p.row_limit - 1) : b) * p.C;
    // (the norm weights of this thread's first 4 columns, likewise requested ahead of the row)
    const int c_first = min((int)threadIdx.x * 4, p.C - 4);
    const f32x4 sc_first = *(const f32x4*)(p.scale + c_first);
    float ss = 0.f;
    [[maybe_unused]] int comb_row[16];
    [[maybe_unused]] float comb_sc[16];
    if constexpr (COMBINE) {
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            comb_row[k] = k < p.comb_topk ? p.comb_dest[b * p.comb_topk + k] : 0;
            comb_sc[k] = k < p.comb_topk ? p.comb_scores[b * p.comb_topk + k] : 0.f;
        }
    }
    for (int c = threadIdx.x * 4; c < p.C; c += kNormThreads * 4) {  // C % 4 == 0
        u32x2 d;
        if constexpr (COMBINE) {
            // the expert outputs of this token in assignment order, as the combine step adds them
            float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                if (k < p.comb_topk) {
                    const u32x2 e = *(const u32x2*)(p.comb_rows + (size_t)comb_row[k] * p.C + c);
                    t[0] += __uint_as_float(e[0] << 16) * comb_sc[k];
                    t[1] += __uint_as_float(e[0] & 0xFFFF0000u) * comb_sc[k];
                    t[2] += __uint_as_float(e[1] << 16) * comb_sc[k];
                    t[3] += __uint_as_float(e[1] & 0xFFFF0000u) * comb_sc[k];
                }
            }
            const u32x2 r = *(const u32x2*)(p.residual + (size_t)b * p.C + c);
            const float r0 = __uint_as_float(r[0] << 16), r1 = __uint_as_float(r[0] & 0xFFFF0000u);
            const float r2 = __uint_as_float(r[1] << 16), r3 = __uint_as_float(r[1] & 0xFFFF0000u);
            d[0] = pack_bf16(r0 + bf16r(bf16r(t[0]) * p.out_scale), r1 + bf16r(bf16r(t[1]) * p.out_scale));
            d[1] = pack_bf16(r2 + bf16r(bf16r(t[2]) * p.out_scale), r3 + bf16r(bf16r(t[3]) * p.out_scale));
            if (share == 0) *(u32x2*)(p.x_out + (size_t)b * p.C + c) = d;
        } else if (!COMBINE && p.partials) {
            // slices are requested 8 at a time (slices past the last read as zeros) and added in slice order
            const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<float*>(p.partials), 0, (uint32_t)((size_t)p.splits * p.B * p.C * 4), 0x00020000);
            const int slab = p.B * p.C * 4, mine = (b * p.C + c) * 4;
            f32x4 t = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int s0 = 0; s0 < p.splits; s0 += 8) {
                u32x4 u[8];
                if (p.splits - s0 <= 4) {  // (4 or fewer left: no loads for slices that do not exist)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        u[j] = __builtin_amdgcn_raw_buffer_load_b128(pr, s0 + j < p.splits ? (s0 + j) * slab + mine : kNoLoad, 0, 0);
#pragma unroll
                    for (int j = 4; j < 8; ++j) u[j] = u32x4{0u, 0u, 0u, 0u};
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        u[j] = __builtin_amdgcn_raw_buffer_load_b128(pr, s0 + j < p.splits ? (s0 + j) * slab + mine : kNoLoad, 0, 0);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    t[0] += __uint_as_float(u[j][0]); t[1] += __uint_as_float(u[j][1]);
                    t[2] += __uint_as_float(u[j][2]); t[3] += __uint_as_float(u[j][3]);
                }
            }
            const u32x2 r = *(const u32x2*)(p.residual + (size_t)b * p.C + c);
            if (p.sum_bias) {  // (the projection's own bias: bf16(bf16(sum) + bias), as the matmul's epilogue forms it)
                const f32x4 bb = *(const f32x4*)(p.sum_bias + c);
                t[0] = bf16r(bf16r(t[0]) + bb[0]); t[1] = bf16r(bf16r(t[1]) + bb[1]);
                t[2] = bf16r(bf16r(t[2]) + bb[2]); t[3] = bf16r(bf16r(t[3]) + bb[3]);
            }
            const float r0 = __uint_as_float(r[0] << 16), r1 = __uint_as_float(r[0] & 0xFFFF0000u);
            const float r2 = __uint_as_float(r[1] << 16), r3 = __uint_as_float(r[1] & 0xFFFF0000u);
            d[0] = pack_bf16(r0 + bf16r(bf16r(t[0]) * p.out_scale), r1 + bf16r(bf16r(t[1]) * p.out_scale));
            d[1] = pack_bf16(r2 + bf16r(bf16r(t[2]) * p.out_scale), r3 + bf16r(bf16r(t[3]) * p.out_scale));
            if (share == 0) *(u32x2*)(p.x_out + (size_t)b * p.C + c) = d;
        } else {
            d = *(const u32x2*)(xr + c);
            if (p.row_index && share == 0) *(u32x2*)(p.x_out + (size_t)b * p.C + c) = d;
        }
        const float v0 = __uint_as_float(d[0] << 16), v1 = __uint_as_float(d[0] & 0xFFFF0000u);
        const float v2 = __uint_as_float(d[1] << 16), v3 = __uint_as_float(d[1] & 0xFFFF0000u);
        sm_h[c] = v0; sm_h[c + 1] = v1; sm_h[c + 2] = v2; sm_h[c + 3] = v3;
        ss += v0 * v0 + v1 * v1 + v2 * v2 + v3 * v3;
    }
    ss = block_sum(ss, sm_red);
    const float inv = rsqrtf(ss / (float)p.C + p.eps);
    for (int c = threadIdx.x * 4; c < p.C; c += kNormThreads * 4) {  // each thread revisits its own elements
        const f32x4 sc = c == c_first ? sc_first : *(const f32x4*)(p.scale + c);
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = sm_h[c + i] * inv * sc[i];
        u32x2 d;
        d[0] = pack_bf16(v[0], v[1]);
        d[1] = pack_bf16(v[2], v[3]);
        if (share == 0) {
            // (mode bit 2: h in tiles of 16 rows x 32 columns, the layout the expert matmul reads fastest)
            const size_t at = (p.mode & 4) ? ((((size_t)(b >> 4) * (p.C >> 5) + (c >> 5)) * 16 + (b & 15)) << 5) + (c & 31) : (size_t)b * p.C + c;
            *(u32x2*)(p.h + at) = d;
        }
        sm_h[c] = __uint_as_float(d[0] << 16);
        sm_h[c + 1] = __uint_as_float(d[0] & 0xFFFF0000u);
        sm_h[c + 2] = __uint_as_float(d[1] << 16);
        sm_h[c + 3] = __uint_as_float(d[1] & 0xFFFF0000u);
    }
    if (!p.proj_t) return;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    for (int j = j_first; j < j_end; j += kNormThreads / 64) {
        // one output per wavefront at a time; its weight row is requested 8 x 16 bytes per lane at once (offsets past
        // the row read as zeros), so a row of up to 2048 columns costs one memory round trip
        const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.proj_t) + (size_t)j * p.C, 0,
                                                                            (uint32_t)p.C * 4u, 0x00020000);
        float acc = 0.f;
        for (int c0 = 0; c0 < p.C; c0 += 2048) {
            u32x4 w[8];
            if (j == j_first && c0 == 0) {
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = w_first[i];
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, (c0 + i * 256 + lane * 4) * 4, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = min(c0 + i * 256 + lane * 4, p.C - 4);  // (clamped reads meet zero weights)
                const f32x4 hv = *(const f32x4*)(sm_h + c);
                acc += hv[0] * __uint_as_float(w[i][0]) + hv[1] * __uint_as_float(w[i][1]) + hv[2] * __uint_as_float(w[i][2]) +
                       hv[3] * __uint_as_float(w[i][3]);
            }
        }
        float v = wave_sum(acc);
        if (lane == 0) {
            if (p.bias) v += p.bias[j];
            const size_t o = (size_t)b * p.n + j;
            if ((p.mode & 3) == 1) ((uint16_t*)p.y)[o] = f32_to_bf16_bits(2.f / (1.f + __expf(-v)));
            else ((float*)p.y)[o] = v;
        }
    }
}

// ---- after the q/k/v projection: QK norm, RoPE, KV-cache append (quantised) ---------------------------------
// One wavefront per (batch row, head).  Lane i holds elements i and i + H/2 of the head: exactly the pair the
// half-split rotary embedding mixes (lyra/model.py:183-186).
//   q, k: rms_norm over the head (model.py:315-320) -> bf16 -> rotate -> bf16
//   k, v: written at `position` into the cache; FP8 caches quantise the row with block (1, H):
//         scale = amax / fmax (1 if the row is zero; fmax = 448 for e4m3fn, 57344 for e5m2), code = fp8_rne(clip(x / scale))
//         (lyra/nn/quant.py:68-72)
struct QkvPostParams {
    const uint16_t* qkv;  // [B, (N + 2K) * H]
    const float* qnorm;   // [H] or null
    const float* knorm;
    const float* cos_t;   // [seq, H/2]
    const float* sin_t;
    const int32_t* position;
    int pos_stride;
    uint16_t* q_out;      // [B, N, H]
    void* k_cache;        // [B, K, S, H]
    void* v_cache;
    float* k_scale;       // [B, K, S] or null (bf16 cache)
    float* v_scale;
    uint16_t* v_unit;     // [B, K, H] or null: the new value rows scaled to unit length, bf16(v * rsqrt(sum v^2 + 1e-10))
    int B, N, K, S, H, seq;
    float eps;
    const float* partials;  // [splits, B, (N + 2K) * H] K slices of the projection not summed yet, or null (then qkv)
    int splits;
    bool e5m2;  // the 1-byte format of a quantised cache: e5m2 instead of e4m3fn
};

__global__ __launch_bounds__(256) void qkv_post_kernel(QkvPostParams p) {
    const int lane = threadIdx.x & 63;
    const int item = blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, head) over N + 2K heads
    const int heads = p.N + 2 * p.K;
    if (item >= p.B * heads) return;
    const int b = item / heads, hd = item - b * heads;
    const int half = p.H >> 1;
    const bool active = lane < half;
    // Everything that does not depend on the projection is requested first, in the order of its own dependencies - the
    // position, then the rotary row it selects, and the norm weights - so that the row's values, which come last out of
    // the kernel before, are the only thing the wavefront still waits for when they arrive.
    const int pos = p.position[(size_t)b * p.pos_stride];
    const bool is_q = hd < p.N, is_k = !is_q && hd < p.N + p.K;
    const float* ns = is_q ? p.qnorm : (is_k ? p.knorm : nullptr);
    float ns_a = 0.f, ns_c = 0.f, cs = 0.f, sn = 0.f;
    if ((is_q || is_k) && active) {
        if (ns) ns_a = ns[lane], ns_c = ns[lane + half];
        const int rp = min(max(pos, 0), p.seq - 1);
        cs = p.cos_t[(size_t)rp * half + lane];
        sn = p.sin_t[(size_t)rp * half + lane];
    }
    float a = 0.f, c = 0.f;
    if (p.partials) {
        if (active) {
            const size_t slab = (size_t)p.B * heads * p.H;
            const float* src = p.partials + ((size_t)b * heads + hd) * p.H;
            for (int s0 = 0; s0 < p.splits; s0 += 4) {  // 4 slices in flight; added in slice order
                float ua[4], uc[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (s0 + j < p.splits) {
                        ua[j] = src[(s0 + j) * slab + lane];
                        uc[j] = src[(s0 + j) * slab + lane + half];
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (s0 + j < p.splits) {
                        a += ua[j];
                        c += uc[j];
                    }
                }
            }
            a = bf16r(a);  // the projection's output is a bf16 array
            c = bf16r(c);
        }
    } else if (active) {
        const uint16_t* src = p.qkv + ((size_t)b * heads + hd) * p.H;
        a = bf16_bits_to_f32(src[lane]);
        c = bf16_bits_to_f32(src[lane + half]);
    }
    if (is_q || is_k) head_norm_rope(a, c, ns != nullptr, ns_a, ns_c, cs, sn, p.eps, p.H);
    if (is_q) {
        if (active) {
            uint16_t* dst = p.q_out + ((size_t)b * p.N + hd) * p.H;
            dst[lane] = f32_to_bf16_bits(a);
            dst[lane + half] = f32_to_bf16_bits(c);
        }
        return;
    }
    const int kh = is_k ? hd - p.N : hd - p.N - p.K;
    if (!is_k && p.v_unit) {  // lyra/model.py:353-354: float32 sum of squares of the bf16 row, result held in bf16
        const float inv = rsqrtf(wave_sum(a * a + c * c) + 1e-10f);
        if (active) {
            uint16_t* dst = p.v_unit + ((size_t)b * p.K + kh) * p.H;
            dst[lane] = f32_to_bf16_bits(a * inv);
            dst[lane + half] = f32_to_bf16_bits(c * inv);
        }
    }
    if (pos < 0 || pos >= p.S) return;  // nothing to append outside the cache
    const size_t row = ((size_t)b * p.K + kh) * p.S + pos;
    void* cache = is_k ? p.k_cache : p.v_cache;
    float* scales = is_k ? p.k_scale : p.v_scale;
    if (scales) {
        const float amax = wave_max(fmaxf(fabsf(a), fabsf(c)));
        const float fmax = fp8_format_max(p.e5m2);
        const float scale = amax > 0.f ? amax / fmax : 1.f;
        const float inv = 1.0f / scale;
        if (active) {
            uint8_t* dst = (uint8_t*)cache + row * p.H;
            dst[lane] = f32_to_fp8_code(fminf(fmaxf(a * inv, -fmax), fmax), p.e5m2);
            dst[lane + half] = f32_to_fp8_code(fminf(fmaxf(c * inv, -fmax), fmax), p.e5m2);
        }
        if (lane == 0) scales[row] = scale;
    } else if (active) {
        uint16_t* dst = (uint16_t*)cache + row * p.H;
        dst[lane] = f32_to_bf16_bits(a);
        dst[lane + half] = f32_to_bf16_bits(c);
    }
}

// ---- MoE routing: top-k, softmax, shared experts, stable counting sort ------------------------------------
// lyra/model.py:459-491.  One workgroup; a token is routed by a few neighbouring lanes, then every assignment finds its
// destination row: start of its expert's rows + number of earlier assignments to the same expert.
struct RouteParams {
    const float* logits;  // [tokens, n_routed] (bias already added)
    float* scores;        // [tokens, topk]
    int32_t* groups;      // [E]
    int32_t* row_map;     // [tokens * topk]: token of each sorted row   (permute_map // topk)
    int32_t* dest;        // [tokens * topk]: sorted row of each assignment (unpermute_map)
    int tokens, n_routed, n_shared, k_routed;
    int stage_logits;
    int lanes;  // lanes that share the routing of one token: a power of two <= 16
};

// LDS ints the routing needs (host and device agree on this layout): assignments [M], counts [E], starts [E], one pad
// int, one bit per (expert, token) in 64-bit words [E][ceil(tokens / 64)], staged logits [tokens * n_routed] when
// stage_logits.
static inline size_t route_lds_ints(int tokens, int n_routed, int n_shared, int k_routed, int stage_logits) {
    const size_t topk = (size_t)k_routed + n_shared, E = (size_t)n_routed + n_shared, W = ((size_t)tokens + 63) / 64;
    return (size_t)tokens * topk + 2 * E + 2 + 2 * E * W + (stage_logits ? (size_t)tokens * n_routed : 0);
}

// The whole routing by one workgroup of any size (a multiple of 64 threads).  `sm_i`: LDS of route_lds_ints() ints, 8-byte
// aligned.
//
// The stable counting sort needs, for every assignment (token t, expert e), the number of earlier assignments to e.  A
// token picks an expert at most once and assignments are in token order, so that is the number of tokens before t that
// picked e: every pick sets bit t of its expert's mask, and a rank is a population count of the bits below t.
__global__ __launch_bounds__(1024) void moe_route_kernel(RouteParams p) {
    extern __shared__ __align__(16) int sm_i[];
    const int topk = p.k_routed + p.n_shared, E = p.n_routed + p.n_shared, M = p.tokens * topk, W = (p.tokens + 63) >> 6;
    int* sm_expert = sm_i;        // [M]
    int* sm_count = sm_i + M;     // [E]
    int* sm_start = sm_count + E; // [E]
    unsigned long long* sm_mask = (unsigned long long*)(sm_i + ((M + 2 * E + 1) & ~1));  // [E][W]
    float* sm_logits = (float*)(sm_mask + (size_t)E * W);  // [tokens * n_routed] when p.stage_logits (coalesced copy, then row reads)
    for (int e = threadIdx.x; e < E * W; e += blockDim.x) sm_mask[e] = 0ull;
    if (p.stage_logits)
        for (int i = threadIdx.x; i < p.tokens * p.n_routed; i += blockDim.x) sm_logits[i] = p.logits[i];
    __syncthreads();
    // A token is routed by `lanes` neighbouring lanes (a power of two <= 16): each scans the experts sub, sub + lanes, ...
    // for its best candidate, a butterfly of shuffles picks the largest value, on ties the lower index (lax.top_k).
    const int lanes = p.lanes;
    for (int base = 0; base < p.tokens * lanes; base += blockDim.x) {
        const int gid = base + threadIdx.x;
        const int t = min(gid / lanes, p.tokens - 1), sub = gid & (lanes - 1);
        const bool owner = gid < p.tokens * lanes && sub == 0;
        const float* lg = (p.stage_logits ? sm_logits : p.logits) + (size_t)t * p.n_routed;
        float top[8];
        int idx[8];
        unsigned long long taken_lo = 0ull, taken_hi = 0ull;  // up to 128 routed experts
        // (loops over the 8 possible picks are unrolled with a guard, so that top[] and idx[] stay in registers)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j >= p.k_routed) break;
            float best = -INFINITY;
            int bi = INT_MAX;  // nothing found yet
            for (int e = sub; e < p.n_routed; e += lanes) {
                const bool used = e < 64 ? (taken_lo >> e) & 1ull : (taken_hi >> (e - 64)) & 1ull;
                const float v = lg[e];
                if (!used && (bi == INT_MAX || v > best)) {  // strict >: ties go to the lower index
                    best = v;
                    bi = e;
                }
            }
            wave_best(best, bi, [](float& v, int& i, float ov, int oi) {
                if (oi != INT_MAX && (i == INT_MAX || ov > v || (ov == v && oi < i))) {
                    v = ov;
                    i = oi;
                }
            }, lanes);
            if (bi < 64) taken_lo |= 1ull << bi; else taken_hi |= 1ull << (bi - 64);
            top[j] = best;
            idx[j] = bi;
        }
        if (!owner) continue;
        float den = 0.f;
        const float top_max = top[0];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j < p.k_routed) {
                top[j] = __expf(top[j] - top_max);
                den += top[j];
            }
        }
        const unsigned long long bit = 1ull << (t & 63);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j < p.k_routed) {
                p.scores[(size_t)t * topk + j] = top[j] / den;
                sm_expert[t * topk + j] = idx[j];
                atomicOr(&sm_mask[(size_t)idx[j] * W + (t >> 6)], bit);
            }
        }
        for (int s = 0; s < p.n_shared; ++s) {
            p.scores[(size_t)t * topk + p.k_routed + s] = 1.f;  // model.py:476
            sm_expert[t * topk + p.k_routed + s] = p.n_routed + s;
            atomicOr(&sm_mask[(size_t)(p.n_routed + s) * W + (t >> 6)], bit);
        }
    }
    __syncthreads();
    // group sizes and the first row of every expert: the first wavefront counts the bits of 64 experts at a time and
    // scans the counts
    if (threadIdx.x < 64) {
        int carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + (int)threadIdx.x;
            int cnt = 0;
            if (e < E)
                for (int w = 0; w < W; ++w) cnt += __popcll(sm_mask[(size_t)e * W + w]);
            const int incl = wave_scan_inclusive(cnt);
            if (e < E) {
                sm_count[e] = cnt;
                sm_start[e] = carry + incl - cnt;
                p.groups[e] = cnt;
            }
            carry += __builtin_amdgcn_readlane(incl, 63);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < M; i += blockDim.x) {
        const int e = sm_expert[i], t = i / topk;
        int rank = __popcll(sm_mask[(size_t)e * W + (t >> 6)] & ((1ull << (t & 63)) - 1ull));
        for (int w = 0; w < (t >> 6); ++w) rank += __popcll(sm_mask[(size_t)e * W + w]);
        const int d = sm_start[e] + rank;
        p.dest[i] = d;
        p.row_map[d] = t;
    }
}

// ---- MoE combine + residual --------------------------------------------------------------------------------
// out[f] = bf16(x[f] + bf16(bf16(sum_k scores[f,k] * rows[dest[f*topk + k]]) * residual_scale))   model.py:557-567
struct CombineParams {
    const uint16_t* rows;   // [M, C] expert outputs in sorted order
    const float* scores;    // [tokens, topk]
    const int32_t* dest;    // [tokens * topk]
    const uint16_t* x;      // [tokens, C] residual stream
    uint16_t* out;          // [tokens, C]
    int tokens, topk, C;
    float residual_scale;
};

__global__ __launch_bounds__(256) void moe_combine_kernel(CombineParams p) {
    const int f = blockIdx.x;
    for (int c = threadIdx.x * 8; c < p.C; c += blockDim.x * 8) {  // C % 8 == 0: 16 bytes per thread and row
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        for (int k = 0; k < p.topk; ++k) {
            const int r = p.dest[f * p.topk + k];
            const float sc = p.scores[f * p.topk + k];
            const u32x4 d = *(const u32x4*)(p.rows + (size_t)r * p.C + c);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] += __uint_as_float(d[i] << 16) * sc;
                acc[2 * i + 1] += __uint_as_float(d[i] & 0xFFFF0000u) * sc;
            }
        }
        const u32x4 xd = *(const u32x4*)(p.x + (size_t)f * p.C + c);
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float t0 = bf16r(bf16r(acc[2 * i]) * p.residual_scale), t1 = bf16r(bf16r(acc[2 * i + 1]) * p.residual_scale);
            o[i] = pack_bf16(__uint_as_float(xd[i] << 16) + t0, __uint_as_float(xd[i] & 0xFFFF0000u) + t1);
        }
        *(u32x4*)(p.out + (size_t)f * p.C + c) = o;
    }
}

// ---- greedy sampling: first index of the row maximum ---------------------------------------------------------
// lyra/generate.py:46-53 with temperature 0 (argmax over the vocabulary; columns >= cols, the padding of the
// vocabulary, are not looked at).  Grid (chunks, rows): every workgroup reduces one chunk of a row to (max, first
// index) and publishes it; the workgroup that arrives last for the row picks among the chunks.
struct ArgmaxParams {
    const float* x;
    int32_t* out;
    float* part_v;   // [rows, chunks]
    int* part_i;     // [rows, chunks]
    int* arrivals;   // [rows] zero on entry, zero again on exit
    int rows, cols, ld, chunks, chunk_len;
    int32_t* advance;  // or null: a counter (the cache position) that the launch increments by one when row 0 is done
};

__device__ __forceinline__ void take_better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

__global__ __launch_bounds__(256) void argmax_kernel(ArgmaxParams p) {
    __shared__ float sm_v[4];
    __shared__ int sm_i[4];
    __shared__ int sm_last;
    const int c = blockIdx.x, row = blockIdx.y;
    const float* xr = p.x + (size_t)row * p.ld;
    const int lo = c * p.chunk_len, hi = min(lo + p.chunk_len, p.cols);
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    // chunk_len % 4 == 0, ld % 4 == 0: aligned 16-byte loads, four of them in flight per thread; they go through a
    // descriptor of the row's `cols` columns (loads past it return zeros) and columns at or past `hi` are not compared
    const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(xr), 0, (uint32_t)p.cols * 4u, 0x00020000);
    for (int i0 = lo + threadIdx.x * 4; i0 < hi; i0 += 4096) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rr, (i0 + u * 1024) * 4, 0, 0);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int i = i0 + u * 1024 + k;
                if (i < hi) take_better(bv, bi, __uint_as_float(v[u][k]), i);
            }
    }
    wave_best(bv, bi, [](float& v, int& i, float ov, int oi) { take_better(v, i, ov, oi); });
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) {
        sm_v[wave] = bv;
        sm_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) take_better(bv, bi, sm_v[w], sm_i[w]);
        store_agent(&p.part_v[row * p.chunks + c], bv);
        store_agent(&p.part_i[row * p.chunks + c], bi);
        wait_all_memory();
        const int seen = add_agent(&p.arrivals[row], 1);
        sm_last = seen == p.chunks - 1;
        if (sm_last) store_agent(&p.arrivals[row], 0);
    }
    __syncthreads();
    if (!sm_last || threadIdx.x >= 64) return;
    bv = -INFINITY;
    bi = 0x7FFFFFFF;
    for (int k = threadIdx.x; k < p.chunks; k += 64)
        take_better(bv, bi, load_agent(&p.part_v[row * p.chunks + k]), __hip_atomic_load(&p.part_i[row * p.chunks + k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    wave_best(bv, bi, [](float& v, int& i, float ov, int oi) { take_better(v, i, ov, oi); });
    if (threadIdx.x == 0) {
        p.out[row] = bi == 0x7FFFFFFF ? 0 : bi;
        if (p.advance && row == 0) *p.advance += 1;
    }
}

// ---- temperature / top-k sampling ---------------------------------------------------------------------------------
// lyra/generate.py:46-53 with temperature > 0: logits / temperature, keep the k largest (lax.top_k: ties go to the lower
// index), draw from their softmax.  The draw is the inverse CDF at a uniform number the caller supplies per row (the
// reference draws with jax.random.categorical from its own key stream; the distribution is the same).
// Grid (chunks, rows) as for the argmax: every workgroup reduces its chunk to its k best (value, index) pairs, the
// workgroup that arrives last for the row merges the chunks' candidates, forms the softmax and picks the token.
constexpr int kMaxSampleK = 8;

struct SampleParams {
    const float* x;
    const float* uniforms;  // [rows] in [0, 1)
    int32_t* out;
    float* part_v;   // [rows, chunks, k]
    int* part_i;     // [rows, chunks, k]
    int* arrivals;   // [rows] zero on entry, zero again on exit
    int rows, cols, ld, chunks, chunk_len, k;
    float temperature;
    int32_t* advance;  // as in ArgmaxParams
    unsigned long long* rng;  // {seed, count} or null (then uniforms)
    int* arrivals_all;        // rng: counts every workgroup of the launch (zero on entry, zero again on exit)
};

__device__ __forceinline__ unsigned long long splitmix64(unsigned long long z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// Keeps the K best pairs seen so far in (tv, ti), best first.  K is a compile-time constant: with a run-time k the arrays
// are indexed dynamically and leave the registers (the launch then took 81 us over 64 x 201088 logits, the arg-max 14.5).
template <int K>
__device__ __forceinline__ void topk_insert(float (&tv)[kMaxSampleK], int (&ti)[kMaxSampleK], float v, int i) {
    if (!better(v, i, tv[K - 1], ti[K - 1])) return;
#pragma unroll
    for (int j = K - 1; j >= 0; --j) {
        const bool here = better(v, i, tv[j], ti[j]);
        const bool above = j > 0 && better(v, i, tv[j > 0 ? j - 1 : 0], ti[j > 0 ? j - 1 : 0]);
        if (here && above) {  // the pair goes further up: move the entry above down into this slot
            tv[j] = tv[j - 1];
            ti[j] = ti[j - 1];
        } else if (here) {
            tv[j] = v;
            ti[j] = i;
        }
    }
}

// The k best pairs over all threads of a workgroup of `nthreads` (64 or 256) threads, each holding its own k best,
// best first: k rounds of "best head wins, its owner moves on".  Result in sm_tv / sm_ti (valid after the call).
template <int K>
__device__ __forceinline__ void topk_merge(float (&tv)[kMaxSampleK], int (&ti)[kMaxSampleK], int nthreads, float* sm_wv,
                                           int* sm_wi, float* sm_tv, int* sm_ti) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = nthreads >> 6;
    int head = 0;
    for (int r = 0; r < K; ++r) {
        float hv = -INFINITY;
        int hi = 0x7FFFFFFF;
#pragma unroll
        for (int j = 0; j < K; ++j)
            if (j == head) {
                hv = tv[j];
                hi = ti[j];
            }
        float bv = hv;
        int bi = hi;
        wave_best(bv, bi, [](float& v, int& i, float ov, int oi) {
            if (better(ov, oi, v, i)) {
                v = ov;
                i = oi;
            }
        });
        if (lane == 0) {
            sm_wv[wave] = bv;
            sm_wi[wave] = bi;
        }
        __syncthreads();
        for (int w = 0; w < waves; ++w)
            if (better(sm_wv[w], sm_wi[w], bv, bi)) {
                bv = sm_wv[w];
                bi = sm_wi[w];
            }
        if (hi == bi && bi != 0x7FFFFFFF) ++head;  // indices are unique: exactly one thread owns the winner
        if (threadIdx.x == 0) {
            sm_tv[r] = bv;
            sm_ti[r] = bi;
        }
        __syncthreads();
    }
}

// Softmax of logits / temperature over a row's K candidates (best first, a candidate without an index ends the list),
// inverse CDF at the row's uniform number.  (K at compile time: the exponentials stay in registers.)
template <int K>
__device__ __forceinline__ int draw_token(const float* cand_v, const int* cand_i, float temperature, float u) {
    float e[K], total = 0.f;
    const float top = cand_v[0] / temperature;
    int n = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const bool have = n == j && cand_i[j] != 0x7FFFFFFF;
        e[j] = have ? expf(cand_v[j] / temperature - top) : 0.f;
        if (have) {
            total += e[j];
            n = j + 1;
        }
    }
    const float target = u * total;
    float run = 0.f;
    int pick = 0;
    bool found = false;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        if (j < n) {
            if (!found) pick = cand_i[j];  // (the last candidate when the number lies beyond every partial sum)
            run += e[j];
            found = found || target < run;
        }
    }
    return pick;
}

// The uniform number of (seed, draw, row): 24 bits of a splitmix64 of the three.
__device__ __forceinline__ float rng_uniform(const unsigned long long* rng, unsigned long long draw, int row) {
    const unsigned long long seed = __hip_atomic_load(&rng[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long z = splitmix64(seed ^ ((draw + 1) * 0x9E3779B97F4A7C15ull) ^ ((unsigned long long)(row + 1) * 0xD1B54A32D192ED03ull));
    return (float)(z >> 40) * 0x1p-24f;
}

template <int K>
__global__ __launch_bounds__(256) void sample_topk_kernel(SampleParams p) {
    __shared__ float sm_wv[4], sm_tv[kMaxSampleK];
    __shared__ int sm_wi[4], sm_ti[kMaxSampleK];
    __shared__ int sm_last;
    const int c = blockIdx.x, row = blockIdx.y;
    constexpr int k = K;
    // (the draw count is read before this workgroup is counted as arrived, and replaced only after all have been)
    const unsigned long long draw = (p.rng && threadIdx.x == 0) ? __hip_atomic_load(&p.rng[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
    const float* xr = p.x + (size_t)row * p.ld;
    const int lo = c * p.chunk_len, hi = min(lo + p.chunk_len, p.cols);
    float tv[kMaxSampleK];
    int ti[kMaxSampleK];
#pragma unroll
    for (int j = 0; j < kMaxSampleK; ++j) {
        tv[j] = -INFINITY;
        ti[j] = 0x7FFFFFFF;
    }
    // chunk_len % 4 == 0, ld % 4 == 0: aligned 16-byte loads, four of them in flight per thread.
    // Two passes over the chunk.  Keeping K best pairs per thread costs ~15 instructions per pair and element, and with 64
    // lanes some lane nearly always has a new candidate, so the wavefront would run the insertion for nearly every element
    // (60 us for 64 x 201088 logits, the arg-max takes 14.5).  The first pass therefore takes one maximum per thread; the
    // K-th largest of the workgroup's 256 maxima is a lower bound `floor_v` of the chunk's K-th best value (K elements at
    // least that large exist).  The second pass reads the chunk again (from the caches) and only looks closer at values
    // >= floor_v - a handful per chunk unless many logits are equal, in which case it is merely slow.
    const int n_vec = (hi - lo) >> 2;
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(xr + lo), 0, (uint32_t)n_vec * 16u, 0x00020000);
    float mx = -INFINITY;
    for (int j0 = threadIdx.x; j0 < n_vec; j0 += 1024) {
        u32x4 raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) raw[u] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (j0 + 256 * u) * 16, 0, 0);  // (past the end: zeros, unused)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float m4 = fmaxf(fmaxf(__uint_as_float(raw[u][0]), __uint_as_float(raw[u][1])),
                                   fmaxf(__uint_as_float(raw[u][2]), __uint_as_float(raw[u][3])));
            mx = j0 + 256 * u < n_vec ? fmaxf(mx, m4) : mx;
        }
    }
    for (int i = lo + 4 * n_vec + threadIdx.x; i < hi; i += 256) mx = fmaxf(mx, xr[i]);  // (a last chunk whose end is not a multiple of 4)
    tv[0] = mx;
    ti[0] = mx > -INFINITY ? (int)threadIdx.x : 0x7FFFFFFF;
    topk_merge<K>(tv, ti, 256, sm_wv, sm_wi, sm_tv, sm_ti);
    const float floor_v = sm_tv[K - 1];  // (-inf when fewer than K threads saw a finite value: everything is looked at)
    __syncthreads();  // (sm_tv is written again below)
    tv[0] = -INFINITY;
    ti[0] = 0x7FFFFFFF;
    for (int j0 = threadIdx.x; j0 < n_vec; j0 += 1024) {
        u32x4 raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) raw[u] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (j0 + 256 * u) * 16, 0, 0);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int jj = j0 + 256 * u;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float v = __uint_as_float(raw[u][q]);
                if (jj < n_vec && v >= floor_v) topk_insert<K>(tv, ti, v, lo + 4 * jj + q);
            }
        }
    }
    for (int i = lo + 4 * n_vec + threadIdx.x; i < hi; i += 256) {
        const float v = xr[i];
        if (v >= floor_v) topk_insert<K>(tv, ti, v, i);
    }
    topk_merge<K>(tv, ti, 256, sm_wv, sm_wi, sm_tv, sm_ti);
    if (threadIdx.x < k) {
        store_agent(&p.part_v[((size_t)row * p.chunks + c) * k + threadIdx.x], sm_tv[threadIdx.x]);
        store_agent(&p.part_i[((size_t)row * p.chunks + c) * k + threadIdx.x], sm_ti[threadIdx.x]);
    }
    wait_all_memory();
    __syncthreads();
    if (threadIdx.x == 0) {
        const int seen = add_agent(&p.arrivals[row], 1);
        sm_last = seen == p.chunks - 1;
        if (sm_last) store_agent(&p.arrivals[row], 0);
        if (p.rng) {
            const int total = (int)(gridDim.x * gridDim.y);
            if (add_agent(p.arrivals_all, 1) == total - 1) {  // every workgroup has read the count: the next launch's is count + 1
                store_agent(p.arrivals_all, 0);
                __hip_atomic_store(&p.rng[1], draw + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __syncthreads();
    if (!sm_last) return;
    // merge the candidates of all chunks (every thread takes some, then the same k rounds)
#pragma unroll
    for (int j = 0; j < kMaxSampleK; ++j) {
        tv[j] = -INFINITY;
        ti[j] = 0x7FFFFFFF;
    }
    for (int q = threadIdx.x; q < p.chunks * k; q += 256) {
        const float v = load_agent(&p.part_v[(size_t)row * p.chunks * k + q]);
        const int i = __hip_atomic_load(&p.part_i[(size_t)row * p.chunks * k + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (i != 0x7FFFFFFF) topk_insert<K>(tv, ti, v, i);
    }
    topk_merge<K>(tv, ti, 256, sm_wv, sm_wi, sm_tv, sm_ti);
    if (threadIdx.x == 0) {
        p.out[row] = draw_token<K>(sm_tv, sm_ti, p.temperature, p.rng ? rng_uniform(p.rng, draw, row) : p.uniforms[row]);
        if (p.advance && row == 0) *p.advance += 1;
    }
}

// ---- the two samplers over logits whose producer also left the maximum of every 128-column tile ------------------
// (GemmParams::tile_max of the matmul that wrote them.)  One workgroup per row reads the row's tile maxima - 1571 numbers
// for 201088 logits - and then only the tiles that can hold what it looks for: the first tile with the row maximum
// (greedy), or the tiles whose maximum reaches the k-th largest tile maximum (k tiles, unless values repeat).  Results are
// those of argmax_kernel / sample_topk_kernel on the same logits.
struct TileSampleParams {
    const float* x;
    const float* tile_max;  // [rows, tile_ld]
    const float* uniforms;
    int32_t* out;
    int rows, cols, ld, tile_ld;
    float temperature;
    int32_t* advance;
    unsigned long long* rng;
    int* arrivals_all;
};

// Maximum of tile t over the row's first `cols` columns: the producer's number, or - the one tile that `cols` cuts - a
// walk over its valid columns.
__device__ __forceinline__ float tile_value(const float* tm, const float* xr, int t, int cols) {
    if (128 * t + 128 <= cols) return tm[t];
    float m = -INFINITY;
    for (int c = 128 * t; c < cols; ++c) m = fmaxf(m, xr[c]);
    return m;
}

__global__ __launch_bounds__(256) void argmax_tiles_kernel(TileSampleParams p) {
    __shared__ float sm_v[4];
    __shared__ int sm_i[4];
    const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float* xr = p.x + (size_t)row * p.ld;
    const float* tm = p.tile_max + (size_t)row * p.tile_ld;
    const int n_tiles = (p.cols + 127) >> 7;
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int t = threadIdx.x; t < n_tiles; t += 256) take_better(bv, bi, tile_value(tm, xr, t, p.cols), t);
    wave_best(bv, bi, [](float& v, int& i, float ov, int oi) { take_better(v, i, ov, oi); });
    if (lane == 0) {
        sm_v[wave] = bv;
        sm_i[wave] = bi;
    }
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < 4; ++w) take_better(bv, bi, sm_v[w], sm_i[w]);
    // the first tile that holds the row maximum: its first column with that value
    const int tile = bi;
    bv = -INFINITY;
    bi = 0x7FFFFFFF;
    if (tile != 0x7FFFFFFF && lane < 32) {
        const int c0 = 128 * tile + 4 * lane;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (c0 + q < p.cols) take_better(bv, bi, xr[c0 + q], c0 + q);
    }
    wave_best(bv, bi, [](float& v, int& i, float ov, int oi) { take_better(v, i, ov, oi); });
    if (lane == 0) {
        p.out[row] = bi == 0x7FFFFFFF ? 0 : bi;
        if (p.advance && row == 0) *p.advance += 1;
    }
}

constexpr int kTileList = 1024;  // tiles a workgroup lists for a closer look; more (many equal logits): a slower walk

// The tile maxima that thread `tid` looks at in one batch: tiles base + tid + 256 j, j < 8 (-inf past the last tile).
// All eight are requested before any is used; the one tile that `cols` cuts is walked by its owner.
__device__ __forceinline__ void load_tile_values(float (&m)[8], const float* tm, const float* xr, int base, int n_tiles, int cols) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int t = base + (int)threadIdx.x + 256 * j;
        const float v = tm[min(t, n_tiles - 1)];
        m[j] = t < n_tiles ? v : -INFINITY;
    }
    if (cols & 127) {
        const int cut = cols >> 7, rel = cut - base - (int)threadIdx.x;
        if (rel >= 0 && rel < 2048 && (rel & 255) == 0) {
            const float v = tile_value(tm, xr, cut, cols);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (rel == 256 * j) m[j] = v;
        }
    }
}

constexpr int kCandMax = 256;  // values a workgroup collects for the final ranking; more (many equal logits): the slower walk

template <int K>
__global__ __launch_bounds__(256) void sample_tiles_kernel(TileSampleParams p) {
    __shared__ float sm_wv[4], sm_tv[kMaxSampleK], sm_g[16], sm_cv[kCandMax];
    __shared__ int sm_wi[4], sm_ti[kMaxSampleK], sm_ci[kCandMax];
    __shared__ int sm_list[kTileList];
    __shared__ int sm_count, sm_ncand;
    __shared__ float sm_floor;
    const int tid = threadIdx.x, row = blockIdx.x, wave = tid >> 6, lane = tid & 63;
    // (the draw count is read before this workgroup is counted as arrived, and replaced only after all have been)
    const unsigned long long draw = (p.rng && tid == 0) ? __hip_atomic_load(&p.rng[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
    const float* xr = p.x + (size_t)row * p.ld;
    const float* tm = p.tile_max + (size_t)row * p.tile_ld;
    const int n_tiles = (p.cols + 127) >> 7;
    const bool one_batch = n_tiles <= 2048;  // (then the second look still holds the first one's values)
    if (tid == 0) sm_count = sm_ncand = 0;
    if (tid < kMaxSampleK) {
        sm_tv[tid] = -INFINITY;
        sm_ti[tid] = 0x7FFFFFFF;
    }
    // A lower bound of the row's K-th best value: the K-th largest of the 16 maxima that groups of 16 threads find
    // among their tiles - K different tiles hold a value at least that large.  (Not the K-th largest tile maximum itself:
    // that costs K rounds over the workgroup, this costs one, and lists a few tiles more.)
    float m[8], mine = -INFINITY;
    for (int base = 0; base < n_tiles; base += 2048) {
        load_tile_values(m, tm, xr, base, n_tiles, p.cols);
#pragma unroll
        for (int j = 0; j < 8; ++j) mine = fmaxf(mine, m[j]);
    }
    mine = row16_max(mine);
    if ((tid & 15) == 0) sm_g[tid >> 4] = mine;
    __syncthreads();
    int seen = 0;
    if (p.rng && tid == 0) {  // (its own read of the count has returned: every load above has)
        wait_all_memory();
        seen = add_agent(p.arrivals_all, 1);
    }
    if (tid < 16) {
        const float v = sm_g[tid];
        int rank = 0;
#pragma unroll
        for (int j = 0; j < 16; ++j) rank += (sm_g[j] > v || (sm_g[j] == v && j < tid)) ? 1 : 0;
        if (rank == K - 1) sm_floor = v;  // (-inf when fewer than K groups hold a finite value: every tile is looked at)
    }
    __syncthreads();
    const float floor_v = sm_floor;
    for (int base = 0; base < n_tiles; base += 2048) {
        if (!one_batch) load_tile_values(m, tm, xr, base, n_tiles, p.cols);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int t = base + tid + 256 * j;
            if (t < n_tiles && m[j] >= floor_v) {
                const int slot = atomicAdd(&sm_count, 1);
                if (slot < kTileList) sm_list[slot] = t;
            }
        }
    }
    __syncthreads();
    const int count = sm_count;
    bool ranked = false;
    if (count <= kTileList) {  // a wavefront per listed tile, 32 lanes x 4 columns: values >= the bound go on a list
        const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(xr), 0, (uint32_t)p.cols * 4u, 0x00020000);
        for (int e = wave; e < count; e += 4) {
            const int c0 = 128 * sm_list[e] + 4 * (lane & 31);
            const u32x4 raw = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, c0 * 4, 0, 0);  // (past `cols`: zeros, unused)
            if (lane < 32) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float v = __uint_as_float(raw[q]);
                    if (c0 + q < p.cols && v >= floor_v) {
                        const int slot = atomicAdd(&sm_ncand, 1);
                        if (slot < kCandMax) {
                            sm_cv[slot] = v;
                            sm_ci[slot] = c0 + q;
                        }
                    }
                }
            }
        }
        __syncthreads();
        const int ncand = sm_ncand;
        if (ncand <= kCandMax) {  // rank by counting: how many candidates come before mine
            if (tid < ncand) {
                const float v = sm_cv[tid];
                const int i = sm_ci[tid];
                int rank = 0;
                for (int j = 0; j < ncand; ++j) rank += better(sm_cv[j], sm_ci[j], v, i) ? 1 : 0;
                if (rank < K) {
                    sm_tv[rank] = v;
                    sm_ti[rank] = i;
                }
            }
            ranked = true;
            __syncthreads();
        }
    }
    if (!ranked) {  // many equal values: every thread walks the tiles it looked at and keeps its K best, then K rounds
        float tv[kMaxSampleK];
        int ti[kMaxSampleK];
#pragma unroll
        for (int j = 0; j < kMaxSampleK; ++j) {
            tv[j] = -INFINITY;
            ti[j] = 0x7FFFFFFF;
        }
        for (int t = tid; t < n_tiles; t += 256) {
            if (!(tile_value(tm, xr, t, p.cols) >= floor_v)) continue;
            for (int c = 128 * t; c < min(128 * t + 128, p.cols); ++c) {
                const float v = xr[c];
                if (v >= floor_v) topk_insert<K>(tv, ti, v, c);
            }
        }
        __syncthreads();
        topk_merge<K>(tv, ti, 256, sm_wv, sm_wi, sm_tv, sm_ti);
    }
    if (tid == 0) {
        p.out[row] = draw_token<K>(sm_tv, sm_ti, p.temperature, p.rng ? rng_uniform(p.rng, draw, row) : p.uniforms[row]);
        if (p.advance && row == 0) *p.advance += 1;
        if (p.rng && seen == (int)gridDim.x - 1) {  // every workgroup has read the count
            store_agent(p.arrivals_all, 0);
            __hip_atomic_store(&p.rng[1], draw + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace lyra

namespace lyra {
static int launch_rmsnorm_proj(const NormProjParams& p0, int B, lyra_stream_t stream) {
    NormProjParams p = p0;
    const size_t lds = ((size_t)p.C + 16) * sizeof(float);
    static const int shares_env = [] { const char* e = getenv("LYRA_NORM_SHARES"); return e ? atoi(e) : 4; }();  // tuning override
    const int shares = (p.proj_t && p.n >= 8 && B <= 256) ? std::max(1, std::min(shares_env, p.n)) : 1;
    p.per_share = (p.n + shares - 1) / shares;
    if (p.comb_rows) hipLaunchKernelGGL(rmsnorm_proj_kernel<true>, dim3(B, shares), dim3(kNormThreads), lds, (hipStream_t)stream, p);
    else hipLaunchKernelGGL(rmsnorm_proj_kernel<false>, dim3(B, shares), dim3(kNormThreads), lds, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}
}  // namespace lyra

extern "C" int lyra_rmsnorm_proj(const void* x, const float* scale, void* h, const float* proj_t, const float* bias, void* y,
                                 int B, int C, int n, int mode, float eps, lyra_stream_t stream) {
    return lyra_rmsnorm_proj_sum(x, nullptr, 0, nullptr, 1.0f, nullptr, scale, h, proj_t, bias, y, B, C, n, mode, eps, stream);
}

extern "C" int lyra_rmsnorm_proj_sum(const void* x, const float* partials, int splits, const void* residual, float out_scale,
                                     void* x_out, const float* scale, void* h, const float* proj_t, const float* bias, void* y,
                                     int B, int C, int n, int mode, float eps, lyra_stream_t stream) {
    return lyra_rmsnorm_proj_sum_bias(x, partials, splits, nullptr, residual, out_scale, x_out, scale, h, proj_t, bias, y, B, C, n, mode,
                                      eps, stream);
}

extern "C" int lyra_rmsnorm_proj_sum_bias(const void* x, const float* partials, int splits, const float* sum_bias, const void* residual,
                                          float out_scale, void* x_out, const float* scale, void* h, const float* proj_t,
                                          const float* bias, void* y, int B, int C, int n, int mode, float eps, lyra_stream_t stream) {
    using namespace lyra;
    if (sum_bias && (!partials || ((uintptr_t)sum_bias % 16))) return LYRA_E_BADARG;
    if (partials ? (!residual || !x_out || splits <= 0) : !x) return LYRA_E_BADARG;
    if (partials && (double)splits * B * C * 4 >= 2147483648.0) return LYRA_E_UNSUPPORTED;
    if (!scale || !h || B <= 0 || C <= 0) return LYRA_E_BADARG;
    if (proj_t && (!y || n <= 0 || ((mode & 3) != 1 && (mode & 3) != 2))) return LYRA_E_BADARG;
    if ((mode & ~7) || ((mode & 4) && C % 32)) return LYRA_E_UNSUPPORTED;
    if (C % 4 || C > 32768) return LYRA_E_UNSUPPORTED;
    NormProjParams p{(const uint16_t*)x, scale, (uint16_t*)h, proj_t, bias, y, C, proj_t ? n : 0, mode, eps,
                     partials, splits, B, (const uint16_t*)residual, out_scale, (uint16_t*)x_out, nullptr, nullptr, nullptr, 0, nullptr, 0,
                     sum_bias};
    return launch_rmsnorm_proj(p, B, stream);
}

extern "C" int lyra_rmsnorm_proj_embed(const void* table, const int32_t* tokens, int table_rows, void* x_out, const float* scale, void* h,
                                       const float* proj_t, const float* bias, void* y, int B, int C, int n, int mode, float eps,
                                       lyra_stream_t stream) {
    using namespace lyra;
    if (!table || !tokens || !x_out || table_rows <= 0) return LYRA_E_BADARG;
    if (!scale || !h || B <= 0 || C <= 0) return LYRA_E_BADARG;
    if (proj_t && (!y || n <= 0 || ((mode & 3) != 1 && (mode & 3) != 2))) return LYRA_E_BADARG;
    if ((mode & ~7) || ((mode & 4) && C % 32)) return LYRA_E_UNSUPPORTED;
    if (C % 4 || C > 32768) return LYRA_E_UNSUPPORTED;
    NormProjParams p{(const uint16_t*)table, scale, (uint16_t*)h, proj_t, bias, y, C, proj_t ? n : 0, mode, eps,
                     nullptr, 0, B, nullptr, 1.0f, (uint16_t*)x_out, nullptr, nullptr, nullptr, 0, tokens, table_rows};
    return launch_rmsnorm_proj(p, B, stream);
}

extern "C" int lyra_rmsnorm_proj_combine(const void* rows, const float* scores, const int32_t* dest, int topk, const void* residual,
                                         float out_scale, void* x_out, const float* scale, void* h, const float* proj_t,
                                         const float* bias, void* y, int B, int C, int n, int mode, float eps, lyra_stream_t stream) {
    using namespace lyra;
    if (!rows || !scores || !dest || !residual || !x_out || topk <= 0) return LYRA_E_BADARG;
    if (!scale || !h || B <= 0 || C <= 0) return LYRA_E_BADARG;
    if (proj_t && (!y || n <= 0 || ((mode & 3) != 1 && (mode & 3) != 2))) return LYRA_E_BADARG;
    if ((mode & ~7) || ((mode & 4) && C % 32)) return LYRA_E_UNSUPPORTED;
    if (C % 4 || C > 32768 || topk > 16) return LYRA_E_UNSUPPORTED;
    NormProjParams p{nullptr, scale, (uint16_t*)h, proj_t, bias, y, C, proj_t ? n : 0, mode, eps,
                     nullptr, 0, B, (const uint16_t*)residual, out_scale, (uint16_t*)x_out,
                     (const uint16_t*)rows, scores, dest, topk, nullptr, 0};
    return launch_rmsnorm_proj(p, B, stream);
}

extern "C" int lyra_qkv_post(const void* qkv, const float* qnorm, const float* knorm, const float* cos_t, const float* sin_t,
                             const int32_t* position, int position_stride, void* q_out, void* k_cache, void* v_cache,
                             float* k_scale, float* v_scale, void* v_unit, int B, int N, int K, int S, int H, int rope_rows,
                             int kv_dtype, float eps, lyra_stream_t stream) {
    return lyra_qkv_post_sum(qkv, nullptr, 0, qnorm, knorm, cos_t, sin_t, position, position_stride, q_out, k_cache, v_cache, k_scale,
                             v_scale, v_unit, B, N, K, S, H, rope_rows, kv_dtype, eps, stream);
}

extern "C" int lyra_qkv_post_sum(const void* qkv, const float* partials, int splits, const float* qnorm, const float* knorm,
                                 const float* cos_t, const float* sin_t, const int32_t* position, int position_stride, void* q_out,
                                 void* k_cache, void* v_cache, float* k_scale, float* v_scale, void* v_unit, int B, int N, int K,
                                 int S, int H, int rope_rows, int kv_dtype, float eps, lyra_stream_t stream) {
    using namespace lyra;
    if (partials ? splits <= 0 : !qkv) return LYRA_E_BADARG;
    if (!cos_t || !sin_t || !position || !q_out || !k_cache || !v_cache) return LYRA_E_BADARG;
    if (B <= 0 || N <= 0 || K <= 0 || S <= 0 || rope_rows <= 0) return LYRA_E_BADARG;
    if (H != 64 && H != 128) return LYRA_E_UNSUPPORTED;
    if ((qnorm == nullptr) != (knorm == nullptr)) return LYRA_E_BADARG;
    const bool fp8 = kv_dtype == LYRA_DTYPE_E4M3FN || kv_dtype == LYRA_DTYPE_E5M2;
    if (!fp8 && kv_dtype != LYRA_DTYPE_BF16) return LYRA_E_UNSUPPORTED;
    if (fp8 != (k_scale != nullptr) || fp8 != (v_scale != nullptr)) return LYRA_E_BADARG;
    if (position_stride != 0 && position_stride != 1) return LYRA_E_BADARG;
    QkvPostParams p{(const uint16_t*)qkv, qnorm, knorm, cos_t, sin_t, position, position_stride, (uint16_t*)q_out,
                    k_cache, v_cache, k_scale, v_scale, (uint16_t*)v_unit, B, N, K, S, H, rope_rows, eps, partials, splits,
                    kv_dtype == LYRA_DTYPE_E5M2};
    const int items = B * (N + 2 * K);
    hipLaunchKernelGGL(qkv_post_kernel, dim3((items + 3) / 4), dim3(256), 0, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

extern "C" int lyra_moe_route(const float* logits, float* scores, int32_t* groups, int32_t* row_map, int32_t* dest, int tokens,
                              int n_routed, int n_shared, int k_routed, lyra_stream_t stream) {
    using namespace lyra;
    if (!logits || !scores || !groups || !row_map || !dest) return LYRA_E_BADARG;
    if (tokens <= 0 || n_routed <= 0 || n_shared < 0 || k_routed <= 0) return LYRA_E_BADARG;
    if (k_routed > 8 || k_routed > n_routed || n_routed > 128) return LYRA_E_UNSUPPORTED;
    const int topk = k_routed + n_shared, E = n_routed + n_shared;
    int lanes = 1;
    while (lanes < 16 && 2 * lanes <= n_routed && (long)tokens * 2 * lanes <= 1024) lanes *= 2;
    const int threads = std::min(1024, std::max(64, (std::max(tokens * topk, tokens * lanes) + 63) / 64 * 64));
    // assignments, counts and starts, the (expert, token) bit masks of the ranking step (+ the logits when they fit)
    size_t lds = route_lds_ints(tokens, n_routed, n_shared, k_routed, 0) * sizeof(int);
    if (lds > 60000) return LYRA_E_UNSUPPORTED;
    const int stage = route_lds_ints(tokens, n_routed, n_shared, k_routed, 1) * sizeof(int) <= 64000;
    if (stage) lds = route_lds_ints(tokens, n_routed, n_shared, k_routed, 1) * sizeof(int);
    RouteParams p{logits, scores, groups, row_map, dest, tokens, n_routed, n_shared, k_routed, stage, lanes};
    hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(threads), lds, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

extern "C" int lyra_moe_combine(const void* rows, const float* scores, const int32_t* dest, const void* x, void* out, int tokens,
                                int topk, int C, float residual_scale, lyra_stream_t stream) {
    using namespace lyra;
    if (!rows || !scores || !dest || !x || !out || tokens <= 0 || topk <= 0 || C <= 0) return LYRA_E_BADARG;
    if (C % 8) return LYRA_E_UNSUPPORTED;
    CombineParams p{(const uint16_t*)rows, scores, dest, (const uint16_t*)x, (uint16_t*)out, tokens, topk, C, residual_scale};
    hipLaunchKernelGGL(moe_combine_kernel, dim3(tokens), dim3(256), 0, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

namespace lyra {
// The arrival counters take a fixed region at the start of the workspace whatever the shape, so that calls of
// different shapes sharing one workspace never leave partial results where another call expects zeroed counters.
constexpr size_t kArgmaxCounterBytes = 65536 * sizeof(int);
static int argmax_chunks(int rows, int cols) {
    static const int wgs_env = [] { const char* e = getenv("LYRA_ARGMAX_WGS"); return e ? atoi(e) : 0; }();  // tuning override
    const int want = std::max(1, (wgs_env > 0 ? wgs_env : 512) / std::max(1, rows));  // ~2 workgroups per compute unit
    const int most = std::max(1, (cols + 4095) / 4096);                // at least 4096 columns per workgroup
    return std::min(std::min(want, most), 64);
}
}  // namespace lyra

extern "C" size_t lyra_argmax_workspace(int rows, int cols) {
    if (rows <= 0 || cols <= 0) return 0;
    return lyra::kArgmaxCounterBytes + ((size_t)rows * lyra::argmax_chunks(rows, cols) * 8 + 255) / 256 * 256;
}

extern "C" int lyra_argmax(const float* x, int32_t* out, void* workspace, size_t workspace_bytes, int rows, int cols, int ld,
                           int32_t* advance, lyra_stream_t stream) {
    using namespace lyra;
    if (!x || !out || rows <= 0 || cols <= 0 || ld < cols) return LYRA_E_BADARG;
    if (ld % 4 || ((uintptr_t)x % 16) || rows > 65535 || cols > (1 << 28)) return LYRA_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < lyra_argmax_workspace(rows, cols) || ((uintptr_t)workspace % 256)) return LYRA_E_WORKSPACE;
    ArgmaxParams p;
    p.x = x;
    p.out = out;
    p.advance = advance;
    p.rows = rows;
    p.cols = cols;
    p.ld = ld;
    p.chunks = argmax_chunks(rows, cols);
    p.chunk_len = ((cols + p.chunks - 1) / p.chunks + 3) / 4 * 4;
    p.chunks = (cols + p.chunk_len - 1) / p.chunk_len;
    const size_t counters = kArgmaxCounterBytes;
    p.arrivals = (int*)workspace;
    p.part_v = (float*)((char*)workspace + counters);
    p.part_i = (int*)(p.part_v + (size_t)rows * argmax_chunks(rows, cols));
    hipLaunchKernelGGL(argmax_kernel, dim3(p.chunks, rows), dim3(256), 0, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

extern "C" size_t lyra_sample_topk_workspace(int rows, int cols, int k) {
    if (rows <= 0 || cols <= 0 || k <= 0) return 0;
    return lyra::kArgmaxCounterBytes + ((size_t)rows * lyra::argmax_chunks(rows, cols) * k * 8 + 255) / 256 * 256;
}

namespace lyra {
static int run_sample_topk(const float* x, const float* uniforms, unsigned long long* rng, int32_t* out, void* workspace,
                           size_t workspace_bytes, int rows, int cols, int ld, int k, float temperature, int32_t* advance,
                           lyra_stream_t stream);
}

extern "C" int lyra_sample_topk(const float* x, const float* uniforms, int32_t* out, void* workspace, size_t workspace_bytes, int rows,
                                int cols, int ld, int k, float temperature, int32_t* advance, lyra_stream_t stream) {
    if (!uniforms) return LYRA_E_BADARG;
    return lyra::run_sample_topk(x, uniforms, nullptr, out, workspace, workspace_bytes, rows, cols, ld, k, temperature, advance, stream);
}

extern "C" int lyra_sample_topk_rng(const float* x, uint64_t* rng, int32_t* out, void* workspace, size_t workspace_bytes, int rows,
                                    int cols, int ld, int k, float temperature, int32_t* advance, lyra_stream_t stream) {
    if (!rng || ((uintptr_t)rng % 8)) return LYRA_E_BADARG;
    return lyra::run_sample_topk(x, nullptr, (unsigned long long*)rng, out, workspace, workspace_bytes, rows, cols, ld, k, temperature,
                                 advance, stream);
}

extern "C" int lyra_argmax_tiles(const float* x, const float* tile_max, int32_t* out, int rows, int cols, int ld, int tile_ld,
                                 int32_t* advance, lyra_stream_t stream) {
    using namespace lyra;
    if (!x || !tile_max || !out || rows <= 0 || cols <= 0 || ld < cols || tile_ld < (cols + 127) / 128) return LYRA_E_BADARG;
    TileSampleParams p{x, tile_max, nullptr, out, rows, cols, ld, tile_ld, 0.f, advance, nullptr, nullptr};
    hipLaunchKernelGGL(argmax_tiles_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

extern "C" int lyra_sample_topk_tiles(const float* x, const float* tile_max, const float* uniforms, uint64_t* rng, int32_t* out,
                                      void* workspace, size_t workspace_bytes, int rows, int cols, int ld, int tile_ld, int k,
                                      float temperature, int32_t* advance, lyra_stream_t stream) {
    using namespace lyra;
    if (!x || !tile_max || !out || rows <= 0 || cols <= 0 || ld < cols || tile_ld < (cols + 127) / 128 || k <= 0 || !(temperature > 0.f))
        return LYRA_E_BADARG;
    if ((uniforms != nullptr) == (rng != nullptr) || ((uintptr_t)rng % 8)) return LYRA_E_BADARG;  // one source of uniform numbers
    if (k > kMaxSampleK || ld % 4 || ((uintptr_t)x % 16)) return LYRA_E_UNSUPPORTED;
    // (the generator's launch counter lives where lyra_sample_topk_rng keeps its own: the two may share a workspace)
    if (rng && (!workspace || workspace_bytes < kArgmaxCounterBytes || ((uintptr_t)workspace % 256))) return LYRA_E_WORKSPACE;
    TileSampleParams p{x, tile_max, uniforms, out, rows, cols, ld, tile_ld, temperature, advance, (unsigned long long*)rng,
                       rng ? (int*)workspace + 65535 : nullptr};
    const dim3 grid(rows), block(256);
    switch (std::min(k, cols)) {
        case 1: hipLaunchKernelGGL(sample_tiles_kernel<1>, grid, block, 0, (hipStream_t)stream, p); break;
        case 2: hipLaunchKernelGGL(sample_tiles_kernel<2>, grid, block, 0, (hipStream_t)stream, p); break;
        case 3: hipLaunchKernelGGL(sample_tiles_kernel<3>, grid, block, 0, (hipStream_t)stream, p); break;
        case 4: hipLaunchKernelGGL(sample_tiles_kernel<4>, grid, block, 0, (hipStream_t)stream, p); break;
        case 5: hipLaunchKernelGGL(sample_tiles_kernel<5>, grid, block, 0, (hipStream_t)stream, p); break;
        case 6: hipLaunchKernelGGL(sample_tiles_kernel<6>, grid, block, 0, (hipStream_t)stream, p); break;
        case 7: hipLaunchKernelGGL(sample_tiles_kernel<7>, grid, block, 0, (hipStream_t)stream, p); break;
        default: hipLaunchKernelGGL(sample_tiles_kernel<8>, grid, block, 0, (hipStream_t)stream, p); break;
    }
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

namespace lyra {
static int run_sample_topk(const float* x, const float* uniforms, unsigned long long* rng, int32_t* out, void* workspace,
                           size_t workspace_bytes, int rows, int cols, int ld, int k, float temperature, int32_t* advance,
                           lyra_stream_t stream) {
    if (!x || !out || rows <= 0 || cols <= 0 || ld < cols || k <= 0 || !(temperature > 0.f)) return LYRA_E_BADARG;
    if (ld % 4 || ((uintptr_t)x % 16) || rows > 65535 || k > kMaxSampleK) return LYRA_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < lyra_sample_topk_workspace(rows, cols, k) || ((uintptr_t)workspace % 256))
        return LYRA_E_WORKSPACE;
    SampleParams p;
    p.x = x;
    p.uniforms = uniforms;
    p.out = out;
    p.advance = advance;
    p.rows = rows;
    p.cols = cols;
    p.ld = ld;
    p.k = std::min(k, cols);
    p.temperature = temperature;
    p.chunks = argmax_chunks(rows, cols);
    p.chunk_len = ((cols + p.chunks - 1) / p.chunks + 3) / 4 * 4;
    p.chunks = (cols + p.chunk_len - 1) / p.chunk_len;
    p.arrivals = (int*)workspace;
    p.rng = rng;
    p.arrivals_all = (int*)workspace + 65535;  // (rows <= 65535: the last counter of the region belongs to no row)
    p.part_v = (float*)((char*)workspace + kArgmaxCounterBytes);
    p.part_i = (int*)(p.part_v + (size_t)rows * argmax_chunks(rows, cols) * k);
    const dim3 grid(p.chunks, rows), block(256);
    switch (p.k) {
        case 1: hipLaunchKernelGGL(sample_topk_kernel<1>, grid, block, 0, (hipStream_t)stream, p); break;
        case 2: hipLaunchKernelGGL(sample_topk_kernel<2>, grid, block, 0, (hipStream_t)stream, p); break;
        case 3: hipLaunchKernelGGL(sample_topk_kernel<3>, grid, block, 0, (hipStream_t)stream, p); break;
        case 4: hipLaunchKernelGGL(sample_topk_kernel<4>, grid, block, 0, (hipStream_t)stream, p); break;
        case 5: hipLaunchKernelGGL(sample_topk_kernel<5>, grid, block, 0, (hipStream_t)stream, p); break;
        case 6: hipLaunchKernelGGL(sample_topk_kernel<6>, grid, block, 0, (hipStream_t)stream, p); break;
        case 7: hipLaunchKernelGGL(sample_topk_kernel<7>, grid, block, 0, (hipStream_t)stream, p); break;
        default: hipLaunchKernelGGL(sample_topk_kernel<8>, grid, block, 0, (hipStream_t)stream, p); break;
    }
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}
}  // namespace lyra
