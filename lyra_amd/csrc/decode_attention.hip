// Decode attention for gfx950: one query token per sequence, grouped-query heads, learned sinks,
// global or sliding-window layers, BF16 or block-scaled FP8 (e4m3fn) KV cache, ragged positions.
//
// Maths (lyra/kernels/decode_attention.py:311-361, Appendix form):
//   s_j = sm_scale * <q, K^[j]>  for visible j;  m = max(max_j s_j, sink);
//   out = sum_j exp(s_j - m) V^[j] / (exp(sink - m) + sum_j exp(s_j - m))
// with K^ = f32(Kq) * k_scale[j] for an FP8 cache.  The per-token scale factors out of both
// contractions, so the kernel multiplies raw FP8 values on the matrix cores (converted exactly to
// BF16 in registers) and applies k_scale to the logits and v_scale to the probabilities in float32.
//
// Work decomposition (flash-decoding): workgroup = (chunk of the visible range, kv head, batch row);
// its 4 wavefronts walk 32-token tiles round-robin, each keeping its own running (max, sum, out);
// they are merged through LDS, and chunks are merged by a second kernel with wavefront shuffles.
//
// Matrix-core mapping, per 32-token tile and wavefront (lane = 16*kb + x):
//   S^T[token, head]  = K[16 tokens x H] . Q^T[H x 16 heads]   (A = K tile, B = Q^T, heads padded to 16)
//   O^T[col, head]   += V^T[16 cols x 32 tokens] . P^T[32 tokens x 16 heads]
// The accumulator layout of the first product (lane x holds head x, tokens 4*kb+r) is exactly the B
// operand layout of the second, so probabilities never leave their lane.
#include <algorithm>

#include "lyra_device.h"

namespace lyra {

struct AttnParams {
    const uint16_t* q;
    const uint8_t* k;
    const uint8_t* v;
    const float* ks;
    const float* vs;
    const float* sinks;
    const int32_t* position;
    int pos_stride;
    const uint16_t* gate;
    void* out;
    float* part_o;   // [B,K,n_chunks,G,H]
    float* part_ml;  // [B,K,n_chunks,G,2]
    int B, N, K, S, G;
    float scale_log2;  // sm_scale * log2(e)
    int sw;
    int chunk;     // tokens per workgroup, multiple of 128
    int n_chunks;  // grid.x
    int out_f32;
    int scale_vec4;  // S % 4 == 0 -> scales are fetched as float4
};

constexpr int kAttnWaves = 4;
constexpr int kTile = 32;

// Visible key range of one batch row; bit-exact restatement of the mask
// (key <= pos) & (key > pos - sw)   (decode_attention.py:285-286, :338-340).
struct Range {
    int lo, hi, start;  // [lo, hi] visible, start = lo rounded down to a tile
};
__device__ __forceinline__ Range visible_range(int pos, int sw, int S) {
    Range r;
    r.hi = min(pos, S - 1);
    r.lo = sw > 0 ? max(0, pos - sw + 1) : 0;
    r.start = r.lo & ~(kTile - 1);
    return r;
}

// out = cast(attn) * gate in the output dtype: a bf16 output is rounded before and after the
// multiplication, as "t *= gate.astype(dtype)" does on a bf16 array (lyra/model.py:347).
__device__ __forceinline__ void store_out(const AttnParams& p, size_t idx, float val, float gate) {
    if (p.out_f32) {
        ((float*)p.out)[idx] = p.gate ? val * gate : val;
    } else {
        if (p.gate) val = bf16_bits_to_f32(f32_to_bf16_bits(val)) * gate;
        ((uint16_t*)p.out)[idx] = f32_to_bf16_bits(val);
    }
}

template <int H, bool FP8>
struct RawTile {
    static constexpr int ES = FP8 ? 1 : 2;
    static constexpr int KW = ES * H / 16;  // dwords of one K row held by a lane (a quarter row)
    static constexpr int VW = ES * H / 64;  // dwords of one V row held by a lane (H/16 columns)
    uint32_t k[2][KW];
    uint32_t v[8][VW];
    float ks[8];
    float vs[8];
};

template <int H, bool FP8>
__device__ __forceinline__ void load_tile(RawTile<H, FP8>& t, const AttnParams& p, const uint8_t* kbase,
                                          const uint8_t* vbase, const float* ksbase, const float* vsbase, int base,
                                          int lane) {
    constexpr int ES = RawTile<H, FP8>::ES;
    constexpr int KW = RawTile<H, FP8>::KW;
    constexpr int VW = RawTile<H, FP8>::VW;
    const int x = lane & 15, kb = lane >> 4;
    const int last = p.S - 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int tok = min(base + 16 * j + x, last);
        const uint8_t* row = kbase + (size_t)tok * (H * ES) + kb * (KW * 4);
#pragma unroll
        for (int w = 0; w < KW; w += 4) {
            u32x4 d = *(const u32x4*)(row + w * 4);
            t.k[j][w] = d[0];
            t.k[j][w + 1] = d[1];
            t.k[j][w + 2] = d[2];
            t.k[j][w + 3] = d[3];
        }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int tok0 = base + 16 * j + 4 * kb;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tok = min(tok0 + r, last);
            const uint8_t* row = vbase + (size_t)tok * (H * ES) + x * (VW * 4);
            if constexpr (VW == 1) {
                t.v[4 * j + r][0] = *(const uint32_t*)row;
            } else if constexpr (VW == 2) {
                u32x2 d = *(const u32x2*)row;
                t.v[4 * j + r][0] = d[0];
                t.v[4 * j + r][1] = d[1];
            } else {
                u32x4 d = *(const u32x4*)row;
                t.v[4 * j + r][0] = d[0];
                t.v[4 * j + r][1] = d[1];
                t.v[4 * j + r][2] = d[2];
                t.v[4 * j + r][3] = d[3];
            }
        }
        if constexpr (FP8) {
            if (p.scale_vec4) {
                const int g0 = min(tok0, p.S - 4);  // S % 4 == 0: the group of 4 is inside or wholly outside
                f32x4 a = *(const f32x4*)(ksbase + g0);
                f32x4 b = *(const f32x4*)(vsbase + g0);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    t.ks[4 * j + r] = a[r];
                    t.vs[4 * j + r] = b[r];
                }
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int tok = min(tok0 + r, last);
                    t.ks[4 * j + r] = ksbase[tok];
                    t.vs[4 * j + r] = vsbase[tok];
                }
            }
        }
    }
}

// One tile of online softmax.  MASKED tiles straddle the ends of the visible range: logits of
// invisible keys become -inf and their V rows / scales are zeroed so that unwritten cache memory
// (which may decode to NaN) cannot reach the accumulators.
template <int H, bool FP8, bool MASKED>
__device__ __forceinline__ void process_tile(RawTile<H, FP8>& t, const bf16x8 (&qop)[H / 32], int base, int lo, int hi,
                                             float scale_log2, int lane, float& m, float& lsum, f32x4 (&o)[H / 16]) {
    constexpr int NC = H / 32;  // k-steps of the S^T product
    constexpr int CB = H / 16;  // 16-column blocks of O^T
    const int kb = lane >> 4;

    f32x4 s[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            bf16x8 a;
            if constexpr (FP8) {
                a = fp8x8_to_bf16x8(t.k[j][2 * c], t.k[j][2 * c + 1]);
            } else {
                Pack8 pk;
                pk.u[0] = t.k[j][4 * c];
                pk.u[1] = t.k[j][4 * c + 1];
                pk.u[2] = t.k[j][4 * c + 2];
                pk.u[3] = t.k[j][4 * c + 3];
                a = pk.v;
            }
            s[j] = mfma_16x16x32(a, qop[c], s[j]);
        }
    }

    bool vis[8];
    float sv[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int tok = base + 16 * (i >> 2) + 4 * kb + (i & 3);
        vis[i] = !MASKED || (tok >= lo && tok <= hi);
        float x = s[i >> 2][i & 3] * scale_log2;
        if constexpr (FP8) x *= t.ks[i];
        sv[i] = vis[i] ? x : -INFINITY;
        tmax = fmaxf(tmax, sv[i]);
    }
    tmax = group4_max(tmax);
    const float m_new = fmaxf(m, tmax);
    if (__ballot(m_new > m) != 0ull) {
        const float alpha = fast_exp2(m - m_new);
        lsum *= alpha;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            o[c][0] *= alpha;
            o[c][1] *= alpha;
            o[c][2] *= alpha;
            o[c][3] *= alpha;
        }
        m = m_new;
    }

    float pv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float pr = fast_exp2(sv[i] - m);
        lsum += pr;
        float w = pr;
        if constexpr (FP8) w *= t.vs[i];
        pv[i] = vis[i] ? w : 0.f;
    }
    Pack8 pop;
#pragma unroll
    for (int i = 0; i < 4; ++i) pop.u[i] = pack_bf16(pv[2 * i], pv[2 * i + 1]);

    if constexpr (MASKED) {
        constexpr int VW = RawTile<H, FP8>::VW;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int w = 0; w < VW; ++w) t.v[i][w] = vis[i] ? t.v[i][w] : 0u;
    }

    // V^T operand: element i of column c is V[token i, c]; the bf16 pack step pairs two tokens, which
    // transposes the row-major cache for free.
    if constexpr (FP8) {
#pragma unroll
        for (int c = 0; c < CB; c += 2) {
            Pack8 v0, v1;
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const f32x2 fa = fp8x2_to_f32(t.v[i][c >> 2], (c & 2) != 0);
                const f32x2 fb = fp8x2_to_f32(t.v[i + 1][c >> 2], (c & 2) != 0);
                v0.u[i >> 1] = pack_bf16(fa[0], fb[0]);
                v1.u[i >> 1] = pack_bf16(fa[1], fb[1]);
            }
            o[c] = mfma_16x16x32(v0.v, pop.v, o[c]);
            o[c + 1] = mfma_16x16x32(v1.v, pop.v, o[c + 1]);
        }
    } else {
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            Pack8 vv;
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const uint32_t a = t.v[i][c >> 1], b = t.v[i + 1][c >> 1];
                vv.u[i >> 1] = (c & 1) ? __builtin_amdgcn_perm(b, a, 0x07060302u) : __builtin_amdgcn_perm(b, a, 0x05040100u);
            }
            o[c] = mfma_16x16x32(vv.v, pop.v, o[c]);
        }
    }
}

template <int H, bool FP8>
__global__ __launch_bounds__(kAttnWaves * 64) void decode_attention_kernel(AttnParams p) {
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int NC = H / 32;
    constexpr int CB = H / 16;
    constexpr int HP = H + 4;  // LDS row pitch in floats
    extern __shared__ float smem[];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = lane & 15, kb = lane >> 4;
    const int c_idx = blockIdx.x, kh = blockIdx.y, b = blockIdx.z;
    const int G = p.G;

    const int pos = p.position[(size_t)b * p.pos_stride];
    const Range rg = visible_range(pos, p.sw, p.S);
    const int c_lo = rg.start + c_idx * p.chunk;
    if (c_lo > rg.hi) {  // chunk holds no visible key (whole workgroup leaves together)
        if (p.n_chunks == 1)  // position < 0: only the sink is attended and its value is 0
            for (int idx = threadIdx.x; idx < G * H; idx += kAttnWaves * 64)
                store_out(p, ((size_t)b * p.N + kh * G) * H + idx, 0.f, 1.f);
        return;
    }
    const int c_hi = min(c_lo + p.chunk, rg.hi + 1);
    const int n_tiles = (c_hi - c_lo + kTile - 1) / kTile;

    // Q^T operand: lane (head x, k-group kb) holds q[head][kb*H/4 + 8c + i]; K lanes hold the same columns.
    bf16x8 qop[NC];
    {
        const uint16_t* qrow = p.q + ((size_t)b * p.N + kh * G + min(x, G - 1)) * H + kb * (H / 4);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            u32x4 d = *(const u32x4*)(qrow + 8 * c);
            if (x >= G) d = u32x4{0u, 0u, 0u, 0u};
            qop[c] = __builtin_bit_cast(bf16x8, d);
        }
    }
    const float sink2 = x < G ? p.sinks[kh * G + x] * kLog2e : 0.f;
    float m = fmaxf(sink2, -1e30f);  // finite start: fully masked tiles cannot produce inf - inf
    float lsum = 0.f;
    f32x4 o[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) o[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    const size_t head_row = ((size_t)b * p.K + kh) * p.S;
    const uint8_t* kbase = p.k + head_row * (H * ES);
    const uint8_t* vbase = p.v + head_row * (H * ES);
    const float* ksbase = FP8 ? p.ks + head_row : nullptr;
    const float* vsbase = FP8 ? p.vs + head_row : nullptr;

    RawTile<H, FP8> cur, nxt;
    int tile = wave;
    if (tile < n_tiles) load_tile<H, FP8>(cur, p, kbase, vbase, ksbase, vsbase, c_lo + tile * kTile, lane);
    for (; tile < n_tiles; tile += kAttnWaves) {
        const int base = c_lo + tile * kTile;
        const bool more = tile + kAttnWaves < n_tiles;
        if (more) load_tile<H, FP8>(nxt, p, kbase, vbase, ksbase, vsbase, base + kAttnWaves * kTile, lane);
        if (base >= rg.lo && base + kTile - 1 <= rg.hi)
            process_tile<H, FP8, false>(cur, qop, base, rg.lo, rg.hi, p.scale_log2, lane, m, lsum, o);
        else
            process_tile<H, FP8, true>(cur, qop, base, rg.lo, rg.hi, p.scale_log2, lane, m, lsum, o);
        if (more) cur = nxt;
    }
    lsum = group4_sum(lsum);

    // ---- merge the 4 wavefronts through LDS -------------------------------------------------
    float* sm_o = smem;                                  // [waves][G][HP]
    float* sm_m = smem + kAttnWaves * G * HP;            // [waves][16]
    float* sm_l = sm_m + kAttnWaves * 16;                // [waves][16]
    if (x < G) {
        float* dst = sm_o + ((size_t)wave * G + x) * HP;
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[(4 * kb + r) * CB + c] = o[c][r];
        if (kb == 0) {
            sm_m[wave * 16 + x] = m;
            sm_l[wave * 16 + x] = lsum;
        }
    }
    __syncthreads();

    const bool final_out = p.n_chunks == 1;
    for (int idx = threadIdx.x; idx < G * H; idx += kAttnWaves * 64) {
        const int g = idx / H, col = idx - g * H;
        float mm = sm_m[g];
#pragma unroll
        for (int w = 1; w < kAttnWaves; ++w) mm = fmaxf(mm, sm_m[w * 16 + g]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float f = fast_exp2(sm_m[w * 16 + g] - mm);
            acc += sm_o[((size_t)w * G + g) * HP + col] * f;
            l += sm_l[w * 16 + g] * f;
        }
        const int n = kh * G + g;
        if (final_out) {
            const float sk = p.sinks[n] * kLog2e;
            const float den = l + fast_exp2(sk - mm);  // mm >= sink by construction
            const float gate = p.gate ? bf16_bits_to_f32(p.gate[(size_t)b * p.N + n]) : 1.f;
            store_out(p, ((size_t)b * p.N + n) * H + col, acc / den, gate);
        } else {
            const size_t item = ((size_t)b * p.K + kh) * p.n_chunks + c_idx;
            p.part_o[(item * G + g) * H + col] = acc;
            if (col == 0) {
                p.part_ml[(item * G + g) * 2] = mm;
                p.part_ml[(item * G + g) * 2 + 1] = l;
            }
        }
    }
}

// Merge of the per-chunk partials: one wavefront per (batch row, query head).  Lanes first span the
// chunks (log-sum-exp weights by wavefront shuffles), then the H output columns.
template <int H>
__global__ __launch_bounds__(64) void decode_attention_merge_kernel(AttnParams p) {
    const int lane = threadIdx.x;
    const int b = blockIdx.x / p.N, n = blockIdx.x - b * p.N;
    const int G = p.G, kh = n / G, g = n - kh * G;
    const int pos = p.position[(size_t)b * p.pos_stride];
    const Range rg = visible_range(pos, p.sw, p.S);
    int nvalid = rg.hi >= rg.lo ? (rg.hi + 1 - rg.start + p.chunk - 1) / p.chunk : 0;
    nvalid = min(nvalid, p.n_chunks);

    const size_t item0 = ((size_t)b * p.K + kh) * p.n_chunks;
    const float sk = p.sinks[n] * kLog2e;
    float mm = fmaxf(sk, -1e30f);
    for (int c = lane; c < nvalid; c += 64) mm = fmaxf(mm, p.part_ml[((item0 + c) * G + g) * 2]);
    mm = wave_max(mm);
    float den = 0.f;
    for (int c = lane; c < nvalid; c += 64) {
        const float* ml = p.part_ml + ((item0 + c) * G + g) * 2;
        den += ml[1] * fast_exp2(ml[0] - mm);
    }
    den = wave_sum(den) + fast_exp2(sk - mm);
    const float inv = 1.f / den;

    float acc[H / 64];
#pragma unroll
    for (int i = 0; i < H / 64; ++i) acc[i] = 0.f;
    for (int c0 = 0; c0 < nvalid; c0 += 64) {
        const int c = c0 + lane;
        const float wl = c < nvalid ? fast_exp2(p.part_ml[((item0 + c) * G + g) * 2] - mm) : 0.f;
        const int cnt = min(64, nvalid - c0);
        for (int cc = 0; cc < cnt; ++cc) {
            const float w = __shfl(wl, cc, 64);
            const float* po = p.part_o + ((item0 + c0 + cc) * G + g) * H;
#pragma unroll
            for (int i = 0; i < H / 64; ++i) acc[i] += w * po[lane + 64 * i];
        }
    }
    const float gate = p.gate ? bf16_bits_to_f32(p.gate[(size_t)b * p.N + n]) : 1.f;
#pragma unroll
    for (int i = 0; i < H / 64; ++i) {
        store_out(p, ((size_t)b * p.N + n) * H + lane + 64 * i, acc[i] * inv, gate);
    }
}

// ---- host side ---------------------------------------------------------------------------------
struct AttnPlan {
    int chunk, n_chunks;
};

// Split so that the launch has a few workgroups per compute unit even at small batch, never below
// one 128-token pass per workgroup.  Depends only on shapes, so plan and workspace size agree.
static AttnPlan plan_attention(int B, int K, int S, int sliding_window) {
    int span = S;  // longest visible range, measured from its tile-aligned start
    if (sliding_window > 0) span = std::min(S, sliding_window + kTile - 1);
    const int unit = kAttnWaves * kTile;
    const int max_chunks = (span + unit - 1) / unit;
    const long pairs = (long)B * K;
    const long target = 256L * 8;  // workgroups
    long want = (target + pairs - 1) / pairs;
    int n_chunks = (int)std::max(1L, std::min((long)max_chunks, want));
    int chunk = (span + n_chunks - 1) / n_chunks;
    chunk = (chunk + unit - 1) / unit * unit;
    n_chunks = (span + chunk - 1) / chunk;
    return AttnPlan{chunk, n_chunks};
}

}  // namespace lyra

extern "C" size_t lyra_decode_attention_workspace(int B, int N, int K, int S, int H, int sliding_window) {
    if (B <= 0 || N <= 0 || K <= 0 || S <= 0 || H <= 0 || N % K) return 0;
    const lyra::AttnPlan pl = lyra::plan_attention(B, K, S, sliding_window);
    if (pl.n_chunks == 1) return 256;
    const size_t items = (size_t)B * K * pl.n_chunks * (N / K);
    size_t bytes = items * H * sizeof(float);
    bytes = (bytes + 255) / 256 * 256;
    bytes += items * 2 * sizeof(float);
    return (bytes + 255) / 256 * 256;
}

extern "C" int lyra_decode_attention(const void* q, const void* k, const void* v, const float* k_scale,
                                     const float* v_scale, const float* sinks, const int32_t* position,
                                     int position_stride, const void* gate, void* out, void* workspace,
                                     size_t workspace_bytes, int B, int N, int K, int S, int H, float sm_scale,
                                     int sliding_window, int kv_dtype, int out_dtype, lyra_stream_t stream) {
    using namespace lyra;
    if (!q || !k || !v || !sinks || !position || !out) return LYRA_E_BADARG;
    if (B <= 0 || N <= 0 || K <= 0 || S <= 0 || H <= 0 || N % K || sliding_window < 0) return LYRA_E_BADARG;
    if (position_stride != 0 && position_stride != 1) return LYRA_E_BADARG;
    if (kv_dtype != LYRA_DTYPE_BF16 && kv_dtype != LYRA_DTYPE_E4M3FN) return LYRA_E_UNSUPPORTED;
    if (out_dtype != LYRA_DTYPE_BF16 && out_dtype != LYRA_DTYPE_F32) return LYRA_E_UNSUPPORTED;
    const bool fp8 = kv_dtype == LYRA_DTYPE_E4M3FN;
    if (fp8 != (k_scale != nullptr) || fp8 != (v_scale != nullptr)) return LYRA_E_BADARG;
    const int G = N / K;
    if ((H != 64 && H != 128) || G > 16) return LYRA_E_UNSUPPORTED;
    if (K > 65535 || B > 65535) return LYRA_E_UNSUPPORTED;

    const AttnPlan pl = plan_attention(B, K, S, sliding_window);
    AttnParams p;
    p.q = (const uint16_t*)q;
    p.k = (const uint8_t*)k;
    p.v = (const uint8_t*)v;
    p.ks = k_scale;
    p.vs = v_scale;
    p.sinks = sinks;
    p.position = position;
    p.pos_stride = position_stride;
    p.gate = (const uint16_t*)gate;
    p.out = out;
    p.part_o = nullptr;
    p.part_ml = nullptr;
    p.B = B; p.N = N; p.K = K; p.S = S; p.G = G;
    p.scale_log2 = sm_scale * kLog2e;
    p.sw = sliding_window;
    p.chunk = pl.chunk;
    p.n_chunks = pl.n_chunks;
    p.out_f32 = out_dtype == LYRA_DTYPE_F32;
    p.scale_vec4 = (S % 4 == 0) && (((uintptr_t)k_scale | (uintptr_t)v_scale) % 16 == 0);
    if (pl.n_chunks > 1) {
        const size_t need = lyra_decode_attention_workspace(B, N, K, S, H, sliding_window);
        if (!workspace || workspace_bytes < need || ((uintptr_t)workspace % 256)) return LYRA_E_WORKSPACE;
        const size_t items = (size_t)B * K * pl.n_chunks * G;
        size_t obytes = (items * H * sizeof(float) + 255) / 256 * 256;
        p.part_o = (float*)workspace;
        p.part_ml = (float*)((char*)workspace + obytes);
    }

    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(pl.n_chunks, K, B), block(kAttnWaves * 64);
    const size_t lds = ((size_t)kAttnWaves * G * (H + 4) + 2 * kAttnWaves * 16) * sizeof(float);
    if (H == 128) {
        if (fp8) hipLaunchKernelGGL((decode_attention_kernel<128, true>), grid, block, lds, st, p);
        else hipLaunchKernelGGL((decode_attention_kernel<128, false>), grid, block, lds, st, p);
    } else {
        if (fp8) hipLaunchKernelGGL((decode_attention_kernel<64, true>), grid, block, lds, st, p);
        else hipLaunchKernelGGL((decode_attention_kernel<64, false>), grid, block, lds, st, p);
    }
    if (hipGetLastError() != hipSuccess) return LYRA_E_LAUNCH;
    if (pl.n_chunks > 1) {
        const dim3 mgrid(B * N), mblock(64);
        if (H == 128) hipLaunchKernelGGL((decode_attention_merge_kernel<128>), mgrid, mblock, 0, st, p);
        else hipLaunchKernelGGL((decode_attention_merge_kernel<64>), mgrid, mblock, 0, st, p);
        if (hipGetLastError() != hipSuccess) return LYRA_E_LAUNCH;
    }
    return LYRA_OK;
}
