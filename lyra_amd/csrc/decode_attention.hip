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
// they are merged through LDS.  Chunks are merged by whichever workgroup of the (batch row, kv head)
// finishes last (an arrival counter in the workspace), so one launch does everything.
//
// Matrix-core mapping, per 32-token tile and wavefront (lane = 16*kb + x):
//   S^T[token, head]  = K[16 tokens x H] . Q^T[H x 16 heads]   (A = K tile, B = Q^T, heads padded to 16)
//   O^T[col, head]   += V^T[16 cols x 32 tokens] . P^T[32 tokens x 16 heads]
// The accumulator layout of the first product (lane x holds head x, tokens 4*kb+r) is exactly the B
// operand layout of the second, so probabilities never leave their lane.
#include <algorithm>
#include <cstdlib>
#include <mutex>

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
    int* arrivals;   // [B,K] zero on entry, zero again on exit
    int B, N, K, S, G;
    float scale_log2;  // sm_scale * log2(e)
    int sw;
    int chunk;     // tokens per workgroup, multiple of 128
    int n_chunks;  // grid.x
    int out_f32;
    int scale_vec4;  // S % 4 == 0 -> scales are fetched as float4
    // learned exclusive self attention (lyra/model.py:351-363), both null when the model has none
    const uint16_t* xsa_v;   // [B,K,H] bf16: the new token's value rows scaled to unit length
    const float* xsa_alpha;  // [N]
    int xsa_lds;             // float offset of the staging area [G*H + 16] in dynamic LDS
    // lyra_decode_attention_qkv: the step in front of the attention (QK norm, rotary embedding, cache append) is done by
    // this launch; q is then not read.  The caches behind k, v, ks, vs are written (one row per batch row and kv head).
    const float* qkv_partials;  // [splits, B, (N + 2K) * H] float32 slices of the q/k/v projection, or null (then qkv)
    const uint16_t* qkv;        // [B, (N + 2K) * H] bf16
    int qkv_splits;
    const float* qkv_bias;      // with the slices: the projection's bias [(N + 2K) * H] (bf16 values as float32), or null
    const float* qnorm;  // [H] or null (both)
    const float* knorm;
    const float* cos_t;  // [rope_rows, H/2]
    const float* sin_t;
    int rope_rows;
    float norm_eps;
    // lyra_decode_attention_ranked: batch rows from longest to shortest ([B]), or null.  With it the unchunked launch deals
    // its (row, kv head) pairs out so that the workgroups that share a compute unit hold a long and a short row.
    const int32_t* row_order;
};

constexpr int kTile = 32;
constexpr int kMaxRankedRows = 256;  // batch rows the whole-row kernel can rank by length (one per thread)
constexpr int kMergeStageFloats = 3 * 1024 + 16;  // LDS floats used when the last workgroup merges chunks

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

// The value the output gate leaves, as the JAX code holds it: a bf16 output is rounded before and after the multiplication.
__device__ __forceinline__ float gated(const AttnParams& p, float val, float gate) {
    if (p.out_f32) return p.gate ? val * gate : val;
    val = bf16_bits_to_f32(f32_to_bf16_bits(val));
    return p.gate ? bf16_bits_to_f32(f32_to_bf16_bits(val * gate)) : val;
}

// Learned exclusive self attention on the G finished heads of one (batch row, kv head) (lyra/model.py:351-363):
//   out = t - tanh(alpha_n) * <t, v^> * v^,   v^ = the new token's value row of this kv head at unit length.
// sm_t [G*H] holds t after the gate (written by the caller, one element per thread and step), sm_coef [16] is scratch.
// A bf16 output follows the dtype flow of the JAX code: the products inside the inner product, the inner product,
// tanh(alpha), both products and the difference are each rounded to bf16; a float32 output rounds nowhere.
// Every thread of the workgroup must call it (two barriers).
template <int H>
__device__ __forceinline__ void xsa_finish(const AttnParams& p, float* sm_t, float* sm_coef, int b, int kh, int tid, int threads) {
    const int lane = tid & 63, wave = tid >> 6, waves = threads >> 6;
    const int G = p.G;
    const bool r16 = !p.out_f32;
    auto rnd = [r16](float x) { return r16 ? bf16_bits_to_f32(f32_to_bf16_bits(x)) : x; };
    const uint16_t* vn = p.xsa_v + ((size_t)b * p.K + kh) * H;
    __syncthreads();
    for (int g = wave; g < G; g += waves) {
        float acc = 0.f;
#pragma unroll
        for (int c = lane; c < H; c += 64) acc += rnd(sm_t[g * H + c] * bf16_bits_to_f32(vn[c]));
        acc = wave_sum(acc);
        if (lane == 0) sm_coef[g] = rnd(rnd(tanhf(p.xsa_alpha[kh * G + g])) * rnd(acc));
    }
    __syncthreads();
    for (int idx = tid; idx < G * H; idx += threads) {
        const int g = idx / H, col = idx - g * H;
        const float r = sm_t[idx] - rnd(sm_coef[g] * bf16_bits_to_f32(vn[col]));
        const size_t o = ((size_t)b * p.N + kh * G + g) * H + col;
        if (p.out_f32) ((float*)p.out)[o] = r;
        else ((uint16_t*)p.out)[o] = f32_to_bf16_bits(r);
    }
}

// Raw (still quantised) operands of one 32-token tile as this lane holds them.
template <int H, int FP8>
struct RawK {
    static constexpr int ES = FP8 ? 1 : 2;
    static constexpr int KW = ES * H / 16;  // dwords of one K row held by a lane: 16-byte pieces at p * 64 + kb * 16
    uint32_t k[2][KW];
};
struct RawS {  // per-token scales of the 8 tokens whose logits this lane holds
    float ks[8];
    float vs[8];
};
template <int H, int FP8>
struct RawV {
    static constexpr int ES = FP8 ? 1 : 2;
    static constexpr int VW = ES * H / 64;  // dwords of one V row held by a lane (H/16 columns)
    uint32_t v[8][VW];
};

// Buffer descriptors of one (batch row, kv head) slab.  Loads past the end of the slab return 0, and the
// per-lane byte offsets are computed once: inside the loop only the tile offset (a scalar) changes.
struct Slab {
    __amdgpu_buffer_rsrc_t k, v, ks, vs;
    int voff_k, voff_v, voff_s;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

template <int H, int FP8>
__device__ __forceinline__ void load_k(RawK<H, FP8>& t, const Slab& sl, int base, bool live) {
    constexpr int ES = RawK<H, FP8>::ES;
    constexpr int KW = RawK<H, FP8>::KW;
    constexpr int RB = H * ES;  // bytes per cached row
    const int soff = __builtin_amdgcn_readfirstlane(live ? base * RB : 0);
    const int voff = live ? sl.voff_k : kNoLoad;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int w = 0; w < KW; w += 4) {
            const u32x4 d = __builtin_amdgcn_raw_buffer_load_b128(sl.k, voff + j * 16 * RB + (w / 4) * 64, soff, kStream);
            t.k[j][w] = d[0];
            t.k[j][w + 1] = d[1];
            t.k[j][w + 2] = d[2];
            t.k[j][w + 3] = d[3];
        }
}

template <bool VEC4>
__device__ __forceinline__ void load_s(RawS& t, const Slab& sl, int base, bool live) {
    const int ssoff = __builtin_amdgcn_readfirstlane(live ? base * 4 : 0);
    const int voff = live ? sl.voff_s : kNoLoad;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if constexpr (VEC4) {
            const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(sl.ks, voff + j * 64, ssoff, kStream);
            const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(sl.vs, voff + j * 64, ssoff, kStream);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                t.ks[4 * j + r] = __uint_as_float(a[r]);
                t.vs[4 * j + r] = __uint_as_float(b[r]);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                t.ks[4 * j + r] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(sl.ks, voff + j * 64 + r * 4, ssoff, kStream));
                t.vs[4 * j + r] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(sl.vs, voff + j * 64 + r * 4, ssoff, kStream));
            }
        }
    }
}

template <int H, int FP8>
__device__ __forceinline__ void load_v(RawV<H, FP8>& t, const Slab& sl, int base, bool live) {
    constexpr int ES = RawV<H, FP8>::ES;
    constexpr int VW = RawV<H, FP8>::VW;
    constexpr int RB = H * ES;
    const int soff = __builtin_amdgcn_readfirstlane(live ? base * RB : 0);
    const int voff = live ? sl.voff_v : kNoLoad;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int off = voff + (16 * (i >> 2) + (i & 3)) * RB;
        if constexpr (VW == 1) {
            t.v[i][0] = __builtin_amdgcn_raw_buffer_load_b32(sl.v, off, soff, kStream);
        } else if constexpr (VW == 2) {
            const u32x2 d = __builtin_amdgcn_raw_buffer_load_b64(sl.v, off, soff, kStream);
            t.v[i][0] = d[0];
            t.v[i][1] = d[1];
        } else {
            const u32x4 d = __builtin_amdgcn_raw_buffer_load_b128(sl.v, off, soff, kStream);
            t.v[i][0] = d[0];
            t.v[i][1] = d[1];
            t.v[i][2] = d[2];
            t.v[i][3] = d[3];
        }
    }
}

// Running state of one wavefront: per lane the max and partial sum of head (lane & 15), and the
// transposed output tile O^T[col, head] in matrix-core accumulator layout.
template <int H>
struct Acc {
    float m, lsum;
    f32x4 o[H / 16];
};

// First third of a tile: S^T = K Q^T on the matrix cores (raw FP8 values, scales applied later).
template <int H, int FP8>
__device__ __forceinline__ void tile_logits(const RawK<H, FP8>& t, const uint16_t* sm_q, int lane, f32x4 (&s)[2]) {
    constexpr int NC = H / 32;
    constexpr int QP = H + 8;  // LDS pitch of a q row in bf16 elements
    const int x = lane & 15, kb = lane >> 4;
    bf16x8 qop[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        // k index of the 8 values chunk c takes from this lane's K pieces: piece p of a lane is the 16 bytes at
        // p * 64 + kb * 16 of the row, so that one load instruction covers a contiguous 64 bytes of each of its 16 rows
        const int k0 = FP8 ? (c >> 1) * 64 + kb * 16 + 8 * (c & 1) : c * 32 + kb * 8;
        qop[c] = *(const bf16x8*)(sm_q + x * QP + k0);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            bf16x8 a;
            if constexpr (FP8) {
                a = fp8x8_to_bf16x8<FP8>(t.k[j][2 * c], t.k[j][2 * c + 1]);
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
}

// Second third: the online-softmax update, producing the probability operand (already multiplied by the
// V scales).  MASKED tiles straddle the ends of the visible range: logits of invisible keys become -inf
// and their probabilities exactly 0.
template <int H, int FP8, bool MASKED>
__device__ __forceinline__ bf16x8 tile_softmax(const f32x4 (&s)[2], const RawS& t, int base, int lo, int hi, float scale_log2,
                                               int lane, Acc<H>& acc, uint32_t& vis_bits) {
    constexpr int CB = H / 16;
    const int kb = lane >> 4;
    float sv[8];
    float tmax = -INFINITY;
    vis_bits = 0xFFu;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float v = s[i >> 2][i & 3];
        if constexpr (FP8) v *= t.ks[i] * scale_log2;
        else v *= scale_log2;
        if constexpr (MASKED) {
            const int tok = base + 16 * (i >> 2) + 4 * kb + (i & 3);
            const bool ok = tok >= lo && tok <= hi;
            if (!ok) {
                v = -INFINITY;
                vis_bits &= ~(1u << i);
            }
        }
        sv[i] = v;
        tmax = fmaxf(tmax, v);
    }
    tmax = group4_max(tmax);
    const float m_new = fmaxf(acc.m, tmax);
    if (__ballot(m_new > acc.m) != 0ull) {
        const float alpha = fast_exp2(acc.m - m_new);
        acc.lsum *= alpha;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            acc.o[c][0] *= alpha;
            acc.o[c][1] *= alpha;
            acc.o[c][2] *= alpha;
            acc.o[c][3] *= alpha;
        }
        acc.m = m_new;
    }
    float pv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float pr = fast_exp2(sv[i] - acc.m);
        acc.lsum += pr;
        float w = pr;
        if constexpr (FP8) w *= t.vs[i];
        if constexpr (MASKED) w = (vis_bits >> i) & 1u ? w : 0.f;  // a garbage scale times 0 must stay 0
        pv[i] = w;
    }
    Pack8 pop;
#pragma unroll
    for (int i = 0; i < 4; ++i) pop.u[i] = pack_bf16(pv[2 * i], pv[2 * i + 1]);
    return pop.v;
}

// Last third of a tile: O^T += V^T P^T.  Element i of column c of the V^T operand is V[token i, c]; the
// bf16 pack step pairs two tokens, which transposes the row-major cache for free.  In MASKED tiles the
// rows of invisible keys are zeroed first so unwritten cache memory (possibly NaN) cannot reach O.
template <int H, int FP8, bool MASKED>
__device__ __forceinline__ void tile_values(RawV<H, FP8>& t, bf16x8 pop, uint32_t vis_bits, Acc<H>& acc) {
    constexpr int CB = H / 16;
    if constexpr (MASKED) {
        constexpr int VW = RawV<H, FP8>::VW;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int w = 0; w < VW; ++w) t.v[i][w] = (vis_bits >> i) & 1u ? t.v[i][w] : 0u;
    }
    if constexpr (FP8) {
#pragma unroll
        for (int c = 0; c < CB; c += 2) {
            Pack8 v0, v1;
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const f32x2 fa = codes2_to_f32<FP8>(t.v[i][c >> 2], (c & 2) != 0);
                const f32x2 fb = codes2_to_f32<FP8>(t.v[i + 1][c >> 2], (c & 2) != 0);
                v0.u[i >> 1] = pack_bf16(fa[0], fb[0]);
                v1.u[i >> 1] = pack_bf16(fa[1], fb[1]);
            }
            acc.o[c] = mfma_16x16x32(v0.v, pop, acc.o[c]);
            acc.o[c + 1] = mfma_16x16x32(v1.v, pop, acc.o[c + 1]);
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
            acc.o[c] = mfma_16x16x32(vv.v, pop, acc.o[c]);
        }
    }
}

// ---- what lyra_qkv_post does for one (batch row, kv head), inside the attention launch -------------------------------
// Same arithmetic in the same order, so results and cache contents are bit-identical to the two launches.  Wavefront w
// takes the query heads w, w + WAVES, ... of the G: sum of the projection's slices, QK norm, rotary embedding -> row t of
// the q tile in LDS.  The last wavefront also finishes the new token's key and value rows (norm, rotary embedding,
// quantisation) and leaves their bytes in LDS.  All of this is requested when the kernel starts, next to the first cache
// tiles, and done before the barrier that releases the wavefronts into their loops.  Behind the barrier, in the workgroup
// whose chunk holds the new token's key, the wavefront that will read that key's tile copies the two rows into the
// caches: they are written and read by one wavefront, whose memory operations are served in the order it issued them, so
// nobody waits for the stores.
constexpr int kHeadSlices = 8;   // slices of a head held in registers
constexpr int kFirstSlices = 4;  // ... of which are requested when the kernel starts
struct HeadSlices {
    float a[kHeadSlices], c[kHeadSlices];  // the first slices of elements `lane` and `lane + H/2`
    uint16_t qa, qc;                       // ... or the two elements of the summed projection (bf16)
};

// Requests the slices of head hd for this lane (elements `lane` and `lane + H/2`).  Every load is issued whatever the
// arguments - through descriptors, with an offset outside them for what does not exist (slices beyond the last, the other
// of the two input forms, idle lanes) - so that no load sits inside a branch and the compiler keeps an exact count of
// what is in flight.
// The slices come in two requests, J0 = 0 and J0 = kFirstSlices: projections of many rows have at most kFirstSlices, and a
// load that returns nothing still takes its turn in the address unit.
template <int H, int J0 = 0>
__device__ __forceinline__ void request_head(const AttnParams& p, __amdgpu_buffer_rsrc_t part_rsrc, __amdgpu_buffer_rsrc_t qkv_rsrc,
                                             int b, int hd, bool live, int lane, HeadSlices& hs) {
    constexpr int half = H / 2;
    const int heads = p.N + 2 * p.K;
    const bool on = live && lane < half;
    const int slab = p.B * heads * H;                 // floats per slice (the host keeps splits * slab * 4 below 2^31)
    const int at = (b * heads + hd) * H + lane;       // element `lane` of the head within a slice
#pragma unroll
    for (int j = J0; j < (J0 == 0 ? kFirstSlices : kHeadSlices); ++j) {
        const int off = on && j < p.qkv_splits ? (j * slab + at) * 4 : kNoLoad;
        hs.a[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(part_rsrc, off, 0, 0));
        hs.c[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(part_rsrc, off, half * 4, 0));
    }
    if constexpr (J0 != 0) return;
#pragma unroll
    for (int j = kFirstSlices; j < kHeadSlices; ++j) hs.a[j] = hs.c[j] = 0.f;
    // the summed form of the projection (bf16); a null descriptor when the slices are given
    const int off16 = on ? at * 2 : kNoLoad;
    hs.qa = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(qkv_rsrc, off16, 0, 0);
    hs.qc = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(qkv_rsrc, off16, half * 2, 0);
}

// The projection's bf16 output for this lane's two elements of head hd: the slices added in slice order, then rounded.
template <int H>
__device__ __forceinline__ void sum_head(const AttnParams& p, __amdgpu_buffer_rsrc_t part_rsrc, int b, int hd, int lane,
                                         const HeadSlices& hs, float& a, float& c) {
    constexpr int half = H / 2;
    if (!p.qkv_partials) {
        a = bf16_bits_to_f32(hs.qa);
        c = bf16_bits_to_f32(hs.qc);
        return;
    }
    a = 0.f + hs.a[0];
    c = 0.f + hs.c[0];
#pragma unroll
    for (int j = 1; j < kHeadSlices; ++j) {
        if (j < p.qkv_splits) {
            a += hs.a[j];
            c += hs.c[j];
        }
    }
    if (p.qkv_splits > kHeadSlices) {  // (more slices than are requested at once: the rest one by one)
        const int heads = p.N + 2 * p.K;
        const int slab = p.B * heads * H, at = (b * heads + hd) * H + lane;
        for (int j = kHeadSlices; j < p.qkv_splits; ++j) {
            const int off = lane < half ? (j * slab + at) * 4 : kNoLoad;
            a += __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(part_rsrc, off, 0, 0));
            c += __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(part_rsrc, off, half * 4, 0));
        }
    }
    a = bf16r(a);
    c = bf16r(c);
    if (p.qkv_bias) {
        // lyra/model.py:310-313: the bias is added to the projection's bf16 result, in bf16.  Fetched here, in the one
        // branch of the front step that holds loads: launches without a bias (every lyra variant) skip it, and two more
        // requests per head at kernel start cost those 0.3 us per sliding-window launch.
        const int heads = p.N + 2 * p.K;
        const __amdgpu_buffer_rsrc_t bias_rsrc = make_rsrc(p.qkv_bias, (uint32_t)heads * (uint32_t)H * 4u);
        const int offb = lane < half ? (hd * H + lane) * 4 : kNoLoad;
        a = bf16r(a + __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(bias_rsrc, offb, 0, 0)));
        c = bf16r(c + __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(bias_rsrc, offb, half * 4, 0)));
    }
}

// The cache bytes of one finished row (this lane's elements a, c) of the key (slot 0) or value (slot 1) head, left in
// LDS: H codes and the row's scale for an FP8 cache, H bf16 values otherwise.  stage: [2][H * ES] bytes, then 2 floats.
template <int H, int FP8>
__device__ __forceinline__ void stage_row(uint8_t* stage, int slot, int lane, float a, float c) {
    constexpr int half = H / 2, ES = FP8 ? 1 : 2;
    const bool active = lane < half;
    if constexpr (FP8) {
        const float amax = wave_max(fmaxf(fabsf(a), fabsf(c)));
        constexpr bool e5m2 = FP8 == 2;
        const float fmax = fp8_format_max(e5m2);
        const float scale = amax > 0.f ? amax / fmax : 1.f;
        const float inv = 1.0f / scale;
        if (active) {
            uint8_t* dst = stage + slot * H;
            dst[lane] = f32_to_fp8_code(fminf(fmaxf(a * inv, -fmax), fmax), e5m2);
            dst[lane + half] = f32_to_fp8_code(fminf(fmaxf(c * inv, -fmax), fmax), e5m2);
        }
        if (lane == 0) ((float*)(stage + 2 * H * ES))[slot] = scale;
    } else if (active) {
        uint16_t* dst = (uint16_t*)stage + slot * H;
        dst[lane] = f32_to_bf16_bits(a);
        dst[lane + half] = f32_to_bf16_bits(c);
    }
}

// Copies the two staged rows into the caches at key `pos` of this workgroup's slab (one dword per lane and row).  Every
// wavefront issues the stores, through the slab's descriptors and with an offset outside them where nothing is to be
// written (`live` false: not the wavefront that owns the new key), so that no memory operation sits inside a branch:
// behind a branch the compiler no longer knows how many operations are in flight and makes the tile loop wait for all of
// them in every pass.
template <int H, int FP8>
__device__ __forceinline__ void append_staged(const Slab& sl, const uint8_t* stage, int pos, bool live, int lane) {
    constexpr int ES = FP8 ? 1 : 2, DW = H * ES / 4;  // dwords per row (16 to 64)
    const bool on = live && lane < DW;
    const uint32_t kd = ((const uint32_t*)stage)[lane & (DW - 1)], vd = ((const uint32_t*)stage)[DW + (lane & (DW - 1))];
    const int off = on ? pos * (H * ES) + lane * 4 : kNoLoad;
    __builtin_amdgcn_raw_buffer_store_b32(kd, sl.k, off, 0, 0);
    __builtin_amdgcn_raw_buffer_store_b32(vd, sl.v, off, 0, 0);
    if constexpr (FP8) {
        const float* sc = (const float*)(stage + 2 * H * ES);
        const int soff = live && lane == 0 ? pos * 4 : kNoLoad;
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sc[0]), sl.ks, soff, 0, 0);
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sc[1]), sl.vs, soff, 0, 0);
    }
}

// QKV: the launch also does the step in front of the attention (lyra_decode_attention_qkv).
template <int H, int FP8, bool VEC4, int WAVES, bool EARLY, int DEPTH, bool QKV = false>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(DEPTH > 1 ? 2 : (WAVES >= 8 ? 4 : 3))))
void decode_attention_kernel(AttnParams p) {
    static_assert(!QKV || DEPTH == 1, "the fused front step knows one register set per wavefront");
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int CB = H / 16;
    constexpr int HP = H + 4;  // LDS row pitch of the merge buffer in floats
    constexpr int QP = H + 8;  // LDS row pitch of q in bf16 elements
    extern __shared__ float smem[];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = lane & 15, kb = lane >> 4;
    const int c_idx = blockIdx.x;
    int kh = blockIdx.y, b = blockIdx.z;
    const int G = p.G;
    if (p.row_order) {
        // Workgroups are started in the order of their linear index (kv head fastest), 256 at a time, one per compute
        // unit: workgroup L of a round shares its unit with workgroup L of the next.  Pairs are ranked by length (row
        // order[r / K], kv head r % K); even rounds take them from the front of their stretch, odd rounds from the back.
        const int L = (int)blockIdx.z * p.K + (int)blockIdx.y, n_pairs = p.B * p.K;
        const int round = L >> 8, i = L & 255;
        const int last = min(n_pairs, (round + 1) << 8) - 1;  // (last rank of this round's stretch)
        const int r = (round & 1) ? last - i : (round << 8) + i;
        kh = r % p.K;
        b = __builtin_amdgcn_readfirstlane(p.row_order[r / p.K]);
    }

    // The position first: loads return in the order they were issued, so requested behind the cache tiles and the
    // projection slices it would arrive last, and everything that follows from it (rotary row, window, the owner of the
    // new key) would start that much later.
    const uint32_t pos_raw = __builtin_amdgcn_raw_buffer_load_b32(
        make_rsrc(p.position, (uint32_t)(p.pos_stride ? p.B : 1) * 4u), 0, b * p.pos_stride * 4, 0);
    __builtin_amdgcn_sched_barrier(0);

    const size_t head_row = ((size_t)b * p.K + kh) * p.S;
    Slab sl;
    sl.k = make_rsrc(p.k + head_row * (H * ES), (uint32_t)p.S * (H * ES));
    sl.v = make_rsrc(p.v + head_row * (H * ES), (uint32_t)p.S * (H * ES));
    sl.ks = make_rsrc(FP8 ? p.ks + head_row : nullptr, FP8 ? (uint32_t)p.S * 4u : 0u);
    sl.vs = make_rsrc(FP8 ? p.vs + head_row : nullptr, FP8 ? (uint32_t)p.S * 4u : 0u);
    sl.voff_k = x * (H * ES) + kb * 16;
    sl.voff_v = 4 * kb * (H * ES) + x * (H * ES / 16);
    sl.voff_s = 16 * kb;

    // q of this kv head's G query heads (thread t: row t / (H/8), 16-byte piece t % (H/8); rows >= G lie past the end of
    // the descriptor and read as zeros) and the sink logits: requested first, so that their arrival does not wait for
    // the cache tiles behind them (loads return in order).
    const int q_row = threadIdx.x / (H / 8), q_piece = threadIdx.x % (H / 8);
    u32x4 q_raw = u32x4{0u, 0u, 0u, 0u};
    [[maybe_unused]] const int qkv_heads = p.N + 2 * p.K;
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t part_rsrc = make_rsrc(
        p.qkv_partials, p.qkv_partials ? (uint32_t)p.qkv_splits * (uint32_t)p.B * (uint32_t)qkv_heads * (uint32_t)H * 4u : 0u);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t qkv_rsrc =
        make_rsrc(p.qkv, (QKV && !p.qkv_partials) ? (uint32_t)p.B * (uint32_t)qkv_heads * (uint32_t)H * 2u : 0u);
    [[maybe_unused]] HeadSlices hq, hkv;  // QKV: the projection slices of this wavefront's first query head (head `wave` of the G)
    [[maybe_unused]] float qn_a = 0.f, qn_c = 0.f, kn_a = 0.f, kn_c = 0.f;
    if constexpr (!QKV) {
        const __amdgpu_buffer_rsrc_t qrsrc = make_rsrc(p.q + ((size_t)b * p.N + kh * G) * H, (uint32_t)(G * H * 2));
        q_raw = __builtin_amdgcn_raw_buffer_load_b128(qrsrc, (q_row * H + q_piece * 8) * 2, 0, 0);
    }
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(p.sinks + kh * G, (uint32_t)(G * 4));
    const float sink_raw = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(srsrc, x * 4, 0, 0));
    // ... and the output gates of these heads (an absent gate reads as zeros and is replaced by 1 below)
    const __amdgpu_buffer_rsrc_t grsrc = make_rsrc(p.gate ? p.gate + (size_t)b * p.N + kh * G : nullptr, p.gate ? (uint32_t)(G * 2) : 0u);
    const uint16_t gate_raw = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(grsrc, x * 2, 0, 0);
    __builtin_amdgcn_sched_barrier(0);

    // First tile of this wavefront: requested next.  Without a sliding window the chunk starts at a
    // key that does not depend on the position, so the request does not wait for the position to arrive (keys past
    // the end of the slab read as zeros, tiles past the visible range are simply not used).
    RawK<H, FP8> rk[DEPTH];
    RawS rs[DEPTH];
    RawV<H, FP8> rv[DEPTH];
    int tile = wave;
    constexpr bool early = EARLY;  // no sliding window
    if constexpr (early) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int early_base = c_idx * p.chunk + (tile + d * WAVES) * kTile;
            load_k<H, FP8>(rk[d], sl, early_base, true);
            if constexpr (FP8) load_s<VEC4>(rs[d], sl, early_base, true);
            load_v<H, FP8>(rv[d], sl, early_base, true);
        }
    }
    if constexpr (QKV) {
        // (behind the cache tiles: those come from memory and gate the loop, these from the caches)
        request_head<H>(p, part_rsrc, qkv_rsrc, b, kh * G + wave, wave < G, lane, hq);
        // (the last wavefront: the key head too, the one before it the value head; used only where the chunk turns out to
        // hold the new key)
        request_head<H>(p, part_rsrc, qkv_rsrc, b, wave == WAVES - 1 ? p.N + kh : p.N + p.K + kh, wave >= WAVES - 2, lane, hkv);
        const __amdgpu_buffer_rsrc_t qn_rsrc = make_rsrc(p.qnorm, p.qnorm ? (uint32_t)H * 4u : 0u);
        const __amdgpu_buffer_rsrc_t kn_rsrc = make_rsrc(p.knorm, p.knorm ? (uint32_t)H * 4u : 0u);
        const int noff = lane < H / 2 ? lane * 4 : kNoLoad;
        qn_a = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(qn_rsrc, noff, 0, 0));
        qn_c = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(qn_rsrc, noff, H / 2 * 4, 0));
        kn_a = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(kn_rsrc, noff, 0, 0));
        kn_c = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(kn_rsrc, noff, H / 2 * 4, 0));
    }

    const int pos = __builtin_amdgcn_readfirstlane((int)pos_raw);  // (waited for here, with everything above in flight)
    const Range rg = visible_range(pos, p.sw, p.S);
    const int c_lo = rg.start + c_idx * p.chunk;
    if (c_lo > rg.hi) {  // chunk holds no visible key (whole workgroup leaves together)
        // First chunk empty = no chunk of this row holds a key (position < 0): only the sink is attended and its value is
        // 0.  No workgroup of the row then reaches the merge, so the first one writes the zeros, however many chunks the
        // launch has; the arrival counter is not touched and stays zero.
        if (c_idx == 0)
            for (int idx = threadIdx.x; idx < G * H; idx += WAVES * 64)
                store_out(p, ((size_t)b * p.N + kh * G) * H + idx, 0.f, 1.f);
        wait_all_memory();
        return;
    }
    const int c_hi = min(c_lo + p.chunk, rg.hi + 1);
    const int n_tiles = (c_hi - c_lo + kTile - 1) / kTile;
    // QKV: this workgroup appends the new token's key and value when its chunk holds them, through the wavefront that
    // reads that key's tile (kv_wave); when the tile is that wavefront's first, it is requested a second time after the
    // rows have been written (`redo`).
    [[maybe_unused]] const bool owner = QKV && pos >= 0 && pos < p.S && pos >= c_lo && pos < c_lo + p.chunk;
    [[maybe_unused]] const int kv_wave = owner ? ((pos - c_lo) / kTile) % WAVES : -1;
    [[maybe_unused]] const bool redo = owner && wave == kv_wave && (pos - c_lo) / kTile < WAVES;
    [[maybe_unused]] float rope_cs = 0.f, rope_sn = 0.f;
    if constexpr (!early) {  // sliding window: the first key follows from the position
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const bool live = tile + d * WAVES < n_tiles;
            const int base = c_lo + (tile + d * WAVES) * kTile;
            load_k<H, FP8>(rk[d], sl, base, live);
            if constexpr (FP8) load_s<VEC4>(rs[d], sl, base, live);
            load_v<H, FP8>(rv[d], sl, base, live);
        }
    }

    uint16_t* sm_q = (uint16_t*)smem;
    static_assert(WAVES * 64 >= 16 * (H / 8), "one q piece per thread");
    if constexpr (QKV) {
        if (q_row >= G) *(u32x4*)(sm_q + q_row * QP + q_piece * 8) = q_raw;  // zeros
        constexpr int half = H / 2;
        if (p.qkv_splits > kFirstSlices) {  // (projections of few rows are cut into more slices)
            request_head<H, kFirstSlices>(p, part_rsrc, qkv_rsrc, b, kh * G + wave, wave < G, lane, hq);
            request_head<H, kFirstSlices>(p, part_rsrc, qkv_rsrc, b, wave == WAVES - 1 ? p.N + kh : p.N + p.K + kh,
                                          owner && wave >= WAVES - 2, lane, hkv);
        }
        {
            const int rp = min(max(pos, 0), p.rope_rows - 1);
            const uint32_t rope_bytes = (uint32_t)p.rope_rows * (uint32_t)half * 4u;
            const int roff = lane < half ? (rp * half + lane) * 4 : kNoLoad;
            rope_cs = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(make_rsrc(p.cos_t, rope_bytes), roff, 0, 0));
            rope_sn = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(make_rsrc(p.sin_t, rope_bytes), roff, 0, 0));
        }
        for (int t = wave; t < G; t += WAVES) {
            if (t != wave) {  // (more than WAVES query heads per kv head)
                // both requests, in this order: the first one clears the slots the second one fills (which it leaves
                // at zero, without memory traffic, when the projection has no more than kFirstSlices slices)
                request_head<H>(p, part_rsrc, qkv_rsrc, b, kh * G + t, true, lane, hq);
                request_head<H, kFirstSlices>(p, part_rsrc, qkv_rsrc, b, kh * G + t, true, lane, hq);
            }
            float a, c;
            sum_head<H>(p, part_rsrc, b, kh * G + t, lane, hq, a, c);
            head_norm_rope(a, c, p.qnorm != nullptr, qn_a, qn_c, rope_cs, rope_sn, p.norm_eps, H);
            if (lane < half) {
                sm_q[t * QP + lane] = f32_to_bf16_bits(a);
                sm_q[t * QP + lane + half] = f32_to_bf16_bits(c);
            }
        }
        if (owner && wave >= WAVES - 2) {  // the new token's key and value rows, as the caches will hold them
            uint8_t* stage = (uint8_t*)(smem + p.xsa_lds);
            const bool is_k = wave == WAVES - 1;
            float a, c;
            sum_head<H>(p, part_rsrc, b, is_k ? p.N + kh : p.N + p.K + kh, lane, hkv, a, c);
            if (is_k) head_norm_rope(a, c, p.knorm != nullptr, kn_a, kn_c, rope_cs, rope_sn, p.norm_eps, H);
            stage_row<H, FP8>(stage, is_k ? 0 : 1, lane, a, c);
        }
    } else {
        *(u32x4*)(sm_q + q_row * QP + q_piece * 8) = q_raw;  // every thread stores (rows >= G hold zeros; rows >= 16 are never read)
    }

    Acc<H> acc;
    const float sink2 = x < G ? sink_raw * kLog2e : 0.f;
    acc.m = fmaxf(sink2, -1e30f);  // finite start: fully masked tiles cannot produce inf - inf
    acc.lsum = 0.f;
#pragma unroll
    for (int c = 0; c < CB; ++c) acc.o[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    if constexpr (QKV) {
        // Everything requested so far is needed by now.  Waiting for all of it here, on every path, also tells the compiler
        // what is in flight when the tile loop starts: after the branches of the front step it otherwise assumes the worst
        // and makes every pass of the loop wait for nearly all of its loads at once (47 instead of 38 us per launch).
        wait_all_memory();
        append_staged<H, FP8>(sl, (const uint8_t*)(smem + p.xsa_lds), pos, wave == kv_wave, lane);  // (0 <= pos < S where live)
        if (redo) {  // the first tile of this wavefront holds the rows just appended: requested again (now from the caches)
            const int base = c_lo + wave * kTile;
            load_k<H, FP8>(rk[0], sl, base, true);
            if constexpr (FP8) load_s<VEC4>(rs[0], sl, base, true);
            load_v<H, FP8>(rv[0], sl, base, true);
            wait_all_memory();  // (leaves this rare path with nothing in flight, like no path the compiler has to guess about)
        }
    }

    // Loads for a tile past the end are issued all the same, with a lane offset no buffer contains (they return zeros
    // without touching memory): the number of loads in flight is then identical on every path and each wait covers
    // exactly the loads it needs.
    // Software pipeline over this wavefront's tiles (wave, wave + WAVES, ...: a fixed assignment, so results are
    // bit-reproducible from run to run) with DEPTH register sets (1 as instantiated: two tiles in flight per wavefront
    // measured no faster): each operand of the next tile of a set is requested right after the last use of the
    // current one, so the loads fly during the rest of the iteration.
    while (tile < n_tiles) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int cur = tile + d * WAVES;         // tile held in register set d (zeros past the end: skipped)
            const int next_tile = cur + DEPTH * WAVES;  // tile requested into the same set
            const int base = c_lo + cur * kTile;
            const int next = c_lo + next_tile * kTile;
            const bool more = next_tile < n_tiles;
            const bool live = cur < n_tiles;
            const bool full = base >= rg.lo && base + kTile - 1 <= rg.hi;
            f32x4 s[2];
            if (live) tile_logits<H, FP8>(rk[d], sm_q, lane, s);
            __builtin_amdgcn_sched_barrier(0);
            load_k<H, FP8>(rk[d], sl, next, more);
            __builtin_amdgcn_sched_barrier(0);
            uint32_t vis = 0;
            bf16x8 pop;
            if (live) {
                if (full) pop = tile_softmax<H, FP8, false>(s, rs[d], base, rg.lo, rg.hi, p.scale_log2, lane, acc, vis);
                else pop = tile_softmax<H, FP8, true>(s, rs[d], base, rg.lo, rg.hi, p.scale_log2, lane, acc, vis);
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (FP8) load_s<VEC4>(rs[d], sl, next, more);
            __builtin_amdgcn_sched_barrier(0);
            if (live) {
                if (full) tile_values<H, FP8, false>(rv[d], pop, vis, acc);
                else tile_values<H, FP8, true>(rv[d], pop, vis, acc);
            }
            __builtin_amdgcn_sched_barrier(0);
            load_v<H, FP8>(rv[d], sl, next, more);
            __builtin_amdgcn_sched_barrier(0);
        }
        tile += DEPTH * WAVES;
    }
    acc.lsum = group4_sum(acc.lsum);

    // ---- merge the wavefronts through LDS ---------------------------------------------------
    __syncthreads();  // everyone is done reading q
    float* sm_o = smem;                             // [waves][G][HP]
    float* sm_m = smem + WAVES * G * HP;            // [waves][16]
    float* sm_l = sm_m + WAVES * 16;                // [waves][16]
    float* sm_sink = sm_l + WAVES * 16;             // [16] sink logit (base 2) and output gate of every head: the final
    float* sm_gate = sm_sink + 16;                  // [16] loop below then reads no global memory between its stores
    if (wave == 0 && kb == 0 && x < G) {
        sm_sink[x] = sink2;
        sm_gate[x] = p.gate ? bf16_bits_to_f32(gate_raw) : 1.f;
    }
    if (x < G) {
        float* dst = sm_o + ((size_t)wave * G + x) * HP;
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[(4 * kb + r) * CB + c] = acc.o[c][r];
        if (kb == 0) {
            sm_m[wave * 16 + x] = acc.m;
            sm_l[wave * 16 + x] = acc.lsum;
        }
    }
    __syncthreads();

    const bool final_out = p.n_chunks == 1;
    for (int idx = threadIdx.x; idx < G * H; idx += WAVES * 64) {
        const int g = idx / H, col = idx - g * H;
        float mm = sm_m[g];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) mm = fmaxf(mm, sm_m[w * 16 + g]);
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float f = fast_exp2(sm_m[w * 16 + g] - mm);
            o += sm_o[((size_t)w * G + g) * HP + col] * f;
            l += sm_l[w * 16 + g] * f;
        }
        const int n = kh * G + g;
        if (final_out) {
            const float den = l + fast_exp2(sm_sink[g] - mm);  // mm >= sink by construction
            if (p.xsa_v) smem[p.xsa_lds + idx] = gated(p, o / den, sm_gate[g]);
            else store_out(p, ((size_t)b * p.N + n) * H + col, o / den, sm_gate[g]);
        } else {
            const size_t item = ((size_t)b * p.K + kh) * p.n_chunks + c_idx;
            store_agent(p.part_o + (item * G + g) * H + col, o);
            if (col == 0) {
                store_agent(p.part_ml + (item * G + g) * 2, mm);
                store_agent(p.part_ml + (item * G + g) * 2 + 1, l);
            }
        }
    }
    if (final_out) {
        if (p.xsa_v) xsa_finish<H>(p, smem + p.xsa_lds, smem + p.xsa_lds + G * H, b, kh, threadIdx.x, WAVES * 64);
        return;
    }

    // ---- merge the chunks: the workgroup that arrives last reads every partial of this kv head ----
    const int n_valid = min((rg.hi + 1 - rg.start + p.chunk - 1) / p.chunk, p.n_chunks);
    __shared__ int sm_last;
    wait_all_memory();  // this lane's partials have reached device-wide visibility
    __syncthreads();    // ... and so have everybody else's in this workgroup, before the arrival is counted
    if (threadIdx.x == 0) {
        const int seen = add_agent(&p.arrivals[b * p.K + kh], 1);
        sm_last = seen == n_valid - 1;
        if (sm_last) store_agent(&p.arrivals[b * p.K + kh], 0);  // leave the counter ready for the next launch
    }
    __syncthreads();
    if (!sm_last) return;
    // weights of the chunks: every thread fetches one (max, sum) pair, then LDS holds exp2(m_c - m*) and the
    // denominator per head; the output columns are then gathered with all loads of a thread in flight at once
    const size_t item0 = ((size_t)b * p.K + kh) * p.n_chunks;
    float* sm_w = smem;                 // [n_valid][G] weight of chunk c for head g
    float* sm_den = smem + 1024;        // [G]
    float* sm_cm = smem + 1024 + 16;    // [n_valid][G] chunk maxima
    float* sm_cl = sm_cm + 1024;        // [n_valid][G] chunk sums
    const bool staged = n_valid * G <= 1024;
    if (staged) {
        for (int i = threadIdx.x; i < n_valid * G; i += WAVES * 64) {
            const float* ml = p.part_ml + (item0 * G + i) * 2;
            sm_cm[i] = load_agent(ml);
            sm_cl[i] = load_agent(ml + 1);
        }
        __syncthreads();
        if (threadIdx.x < G) {
            const int g = threadIdx.x;
            const float sk = p.sinks[kh * G + g] * kLog2e;
            float mm = fmaxf(sk, -1e30f);
            for (int c = 0; c < n_valid; ++c) mm = fmaxf(mm, sm_cm[c * G + g]);
            float den = fast_exp2(sk - mm);
            for (int c = 0; c < n_valid; ++c) {
                const float f = fast_exp2(sm_cm[c * G + g] - mm);
                sm_w[c * G + g] = f;
                den += sm_cl[c * G + g] * f;
            }
            sm_den[g] = den;
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < G * H; idx += WAVES * 64) {
            const int g = idx / H, col = idx - g * H;
            const int n = kh * G + g;
            float o = 0.f;
            for (int c0 = 0; c0 < n_valid; c0 += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    v[u] = c0 + u < n_valid ? load_agent(p.part_o + ((item0 + c0 + u) * G + g) * H + col) : 0.f;
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (c0 + u < n_valid) o += v[u] * sm_w[(c0 + u) * G + g];
            }
            const float gate = p.gate ? bf16_bits_to_f32(p.gate[(size_t)b * p.N + n]) : 1.f;
            if (p.xsa_v) smem[p.xsa_lds + idx] = gated(p, o / sm_den[g], gate);
            else store_out(p, ((size_t)b * p.N + n) * H + col, o / sm_den[g], gate);
        }
        if (p.xsa_v) xsa_finish<H>(p, smem + p.xsa_lds, smem + p.xsa_lds + G * H, b, kh, threadIdx.x, WAVES * 64);
        return;
    }
    // more chunks than the staging area holds: plain per-thread loops (long contexts at tiny batch)
    for (int idx = threadIdx.x; idx < G * H; idx += WAVES * 64) {
        const int g = idx / H, col = idx - g * H;
        const int n = kh * G + g;
        const float sk = p.sinks[n] * kLog2e;
        float mm = fmaxf(sk, -1e30f);
        for (int c = 0; c < n_valid; ++c) mm = fmaxf(mm, load_agent(p.part_ml + ((item0 + c) * G + g) * 2));
        float o = 0.f, den = fast_exp2(sk - mm);
        for (int c = 0; c < n_valid; ++c) {
            const float* ml = p.part_ml + ((item0 + c) * G + g) * 2;
            const float f = fast_exp2(load_agent(ml) - mm);
            den += load_agent(ml + 1) * f;
            o += load_agent(p.part_o + ((item0 + c) * G + g) * H + col) * f;
        }
        const float gate = p.gate ? bf16_bits_to_f32(p.gate[(size_t)b * p.N + n]) : 1.f;
        if (p.xsa_v) smem[p.xsa_lds + idx] = gated(p, o / den, gate);
        else store_out(p, ((size_t)b * p.N + n) * H + col, o / den, gate);
    }
    if (p.xsa_v) xsa_finish<H>(p, smem + p.xsa_lds, smem + p.xsa_lds + G * H, b, kh, threadIdx.x, WAVES * 64);
}

// ---- whole rows, longest first ------------------------------------------------------------------
// For launches with more (batch row, kv head) pairs than compute units and no sliding window.  One workgroup per compute
// unit stays resident and works through several pairs, each from its first key to its last (no chunks, no merge across
// workgroups).  With one position per batch row the rows are ranked by length first (descending, ties by row index) and
// dealt out in serpentine order - workgroup w takes entries w, 2W-1-w, 2W+w, 4W-1-w, ... of the ranked list of pairs - so
// every workgroup gets long and short rows in turn and all finish together; handed out in launch order instead, two long
// rows that land on the same compute unit set the time of the launch (gpt-oss shape, lengths 256...4096: 39 us, of which
// only 24 us are the average unit's share).  The first tile of the next pair is requested before the current pair's
// wavefronts are merged, so a compute unit keeps streaming across pairs.
template <int H, int FP8>
struct PairState {
    Slab sl;
    int b, kh, pos;
    u32x4 q_raw;
    float sink_raw;
    uint16_t gate_raw;
};

template <int H, int FP8, bool VEC4>
__device__ __forceinline__ void request_pair(const AttnParams& p, int pair, bool live_pair, const int* sm_pos, const int* sm_order,
                                             int tid, int lane, int wave, PairState<H, FP8>& st, RawK<H, FP8>& rk, RawS& rs,
                                             RawV<H, FP8>& rv) {
    constexpr int ES = FP8 ? 1 : 2;
    const int x = lane & 15, kb = lane >> 4;
    const int G = p.G;
    const int row_rank = pair / p.K;
    st.kh = pair - row_rank * p.K;
    st.b = __builtin_amdgcn_readfirstlane(sm_order[row_rank]);
    st.pos = __builtin_amdgcn_readfirstlane(sm_pos[st.b]);
    const size_t head_row = ((size_t)st.b * p.K + st.kh) * p.S;
    st.sl.k = make_rsrc(p.k + head_row * (H * ES), (uint32_t)p.S * (H * ES));
    st.sl.v = make_rsrc(p.v + head_row * (H * ES), (uint32_t)p.S * (H * ES));
    st.sl.ks = make_rsrc(FP8 ? p.ks + head_row : nullptr, FP8 ? (uint32_t)p.S * 4u : 0u);
    st.sl.vs = make_rsrc(FP8 ? p.vs + head_row : nullptr, FP8 ? (uint32_t)p.S * 4u : 0u);
    st.sl.voff_k = x * (H * ES) + kb * 16;
    st.sl.voff_v = 4 * kb * (H * ES) + x * (H * ES / 16);
    st.sl.voff_s = 16 * kb;
    // q, sinks and gates first (loads return in order), then this wavefront's first tile
    const __amdgpu_buffer_rsrc_t qrsrc = make_rsrc(p.q + ((size_t)st.b * p.N + st.kh * G) * H, (uint32_t)(G * H * 2));
    const int q_row = tid / (H / 8), q_piece = tid % (H / 8);
    st.q_raw = __builtin_amdgcn_raw_buffer_load_b128(qrsrc, (q_row * H + q_piece * 8) * 2, 0, 0);
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(p.sinks + st.kh * G, (uint32_t)(G * 4));
    st.sink_raw = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(srsrc, x * 4, 0, 0));
    const __amdgpu_buffer_rsrc_t grsrc =
        make_rsrc(p.gate ? p.gate + (size_t)st.b * p.N + st.kh * G : nullptr, p.gate ? (uint32_t)(G * 2) : 0u);
    st.gate_raw = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(grsrc, x * 2, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    const bool live = live_pair && wave * kTile <= min(st.pos, p.S - 1);
    load_k<H, FP8>(rk, st.sl, wave * kTile, live);
    if constexpr (FP8) load_s<VEC4>(rs, st.sl, wave * kTile, live);
    load_v<H, FP8>(rv, st.sl, wave * kTile, live);
}

template <int H, int FP8, bool VEC4, int WAVES>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(WAVES / 4, WAVES / 4)))  // one workgroup per compute unit
void decode_attention_rows_kernel(AttnParams p) {
    constexpr int CB = H / 16;
    constexpr int HP = H + 4;  // LDS row pitch of the merge buffer in floats
    constexpr int QP = H + 8;  // LDS row pitch of q in bf16 elements
    extern __shared__ float smem[];
    __shared__ int sm_pos[kMaxRankedRows];
    __shared__ int sm_order[kMaxRankedRows];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int x = lane & 15, kb = lane >> 4;
    const int G = p.G;
    const int n_pairs = p.B * p.K;
    const int n_wg = gridDim.x;  // <= n_pairs

    // rank the rows: thread t places row t
    int mine = 0;
    if (tid < p.B) {
        mine = p.position[(size_t)tid * p.pos_stride];
        sm_pos[tid] = mine;
    }
    __syncthreads();
    if (tid < p.B) {
        int rank = tid;
        if (p.pos_stride != 0) {
            rank = 0;
            for (int j = 0; j < p.B; ++j) {
                const int other = sm_pos[j];
                rank += (other > mine) || (other == mine && j < tid);
            }
        }
        sm_order[rank] = tid;
    }
    __syncthreads();

    PairState<H, FP8> st;
    RawK<H, FP8> rk;
    RawS rs;
    RawV<H, FP8> rv;
    int round = 0;
    request_pair<H, FP8, VEC4>(p, (int)blockIdx.x, true, sm_pos, sm_order, tid, lane, wave, st, rk, rs, rv);

    uint16_t* sm_q = (uint16_t*)smem;
    static_assert(WAVES * 64 >= 16 * (H / 8), "one q piece per thread");
    const int q_row = tid / (H / 8), q_piece = tid % (H / 8);
    for (;;) {
        const Range rg = visible_range(st.pos, 0, p.S);
        const int n_tiles = (rg.hi + kTile) / kTile;  // 0 when the position is negative: only the sink is attended
        *(u32x4*)(sm_q + q_row * QP + q_piece * 8) = st.q_raw;

        Acc<H> acc;
        const float sink2 = x < G ? st.sink_raw * kLog2e : 0.f;
        acc.m = fmaxf(sink2, -1e30f);
        acc.lsum = 0.f;
#pragma unroll
        for (int c = 0; c < CB; ++c) acc.o[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();

        // same software pipeline as decode_attention_kernel: tiles wave, wave + WAVES, ... of the row
        for (int tile = wave; tile < n_tiles; tile += WAVES) {
            const int base = tile * kTile;
            const int next = base + WAVES * kTile;
            const bool more = tile + WAVES < n_tiles;
            const bool full = base + kTile - 1 <= rg.hi;
            f32x4 s[2];
            tile_logits<H, FP8>(rk, sm_q, lane, s);
            __builtin_amdgcn_sched_barrier(0);
            load_k<H, FP8>(rk, st.sl, next, more);
            __builtin_amdgcn_sched_barrier(0);
            uint32_t vis = 0;
            bf16x8 pop;
            if (full) pop = tile_softmax<H, FP8, false>(s, rs, base, 0, rg.hi, p.scale_log2, lane, acc, vis);
            else pop = tile_softmax<H, FP8, true>(s, rs, base, 0, rg.hi, p.scale_log2, lane, acc, vis);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (FP8) load_s<VEC4>(rs, st.sl, next, more);
            __builtin_amdgcn_sched_barrier(0);
            if (full) tile_values<H, FP8, false>(rv, pop, vis, acc);
            else tile_values<H, FP8, true>(rv, pop, vis, acc);
            __builtin_amdgcn_sched_barrier(0);
            load_v<H, FP8>(rv, st.sl, next, more);
            __builtin_amdgcn_sched_barrier(0);
        }
        acc.lsum = group4_sum(acc.lsum);

        // what the merge needs of the finished pair, then the requests of the next one (none after the last: the loads
        // are still issued, with lane offsets that touch no memory, so both paths have the same loads in flight)
        const int done_b = st.b, done_kh = st.kh;
        const float done_gate = p.gate ? bf16_bits_to_f32(st.gate_raw) : 1.f;
        ++round;
        const int next_pair = round * n_wg + ((round & 1) ? n_wg - 1 - (int)blockIdx.x : (int)blockIdx.x);
        const bool has_next = next_pair < n_pairs;
        request_pair<H, FP8, VEC4>(p, has_next ? next_pair : 0, has_next, sm_pos, sm_order, tid, lane, wave, st, rk, rs, rv);

        // ---- merge the wavefronts through LDS (as in decode_attention_kernel) ----
        __syncthreads();  // everyone is done reading q
        float* sm_o = smem;                   // [waves][G][HP]
        float* sm_m = smem + WAVES * G * HP;  // [waves][16]
        float* sm_l = sm_m + WAVES * 16;      // [waves][16]
        float* sm_sink = sm_l + WAVES * 16;   // [16]
        float* sm_gate = sm_sink + 16;        // [16]
        if (wave == 0 && kb == 0 && x < G) {
            sm_sink[x] = sink2;
            sm_gate[x] = done_gate;
        }
        if (x < G) {
            float* dst = sm_o + ((size_t)wave * G + x) * HP;
#pragma unroll
            for (int c = 0; c < CB; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[(4 * kb + r) * CB + c] = acc.o[c][r];
            if (kb == 0) {
                sm_m[wave * 16 + x] = acc.m;
                sm_l[wave * 16 + x] = acc.lsum;
            }
        }
        __syncthreads();
        for (int idx = tid; idx < G * H; idx += WAVES * 64) {
            const int g = idx / H, col = idx - g * H;
            float mm = sm_m[g];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) mm = fmaxf(mm, sm_m[w * 16 + g]);
            float o = 0.f, l = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float f = fast_exp2(sm_m[w * 16 + g] - mm);
                o += sm_o[((size_t)w * G + g) * HP + col] * f;
                l += sm_l[w * 16 + g] * f;
            }
            const float den = l + fast_exp2(sm_sink[g] - mm);  // mm >= sink by construction
            if (p.xsa_v) smem[p.xsa_lds + idx] = gated(p, o / den, sm_gate[g]);
            else store_out(p, ((size_t)done_b * p.N + done_kh * G + g) * H + col, o / den, sm_gate[g]);
        }
        if (p.xsa_v) xsa_finish<H>(p, smem + p.xsa_lds, smem + p.xsa_lds + G * H, done_b, done_kh, tid, WAVES * 64);
        if (!has_next) break;
        __syncthreads();  // the merge buffer has been read: q of the next pair may replace it
    }
}

// ---- host side ---------------------------------------------------------------------------------
struct AttnPlan {
    int chunk, n_chunks, waves;
};
constexpr long kMaxSplitPairs = 16384;  // (batch row, kv head) pairs beyond which a launch is never chunked

static long env_long(const char* name) {
    const char* e = getenv(name);
    return e ? atol(e) : 0L;
}

// Split so that the launch fills the 256 compute units even at small batch, never below one pass of the
// workgroup's wavefronts.  Depends only on shapes, so plan and workspace size agree.
static AttnPlan plan_attention(int B, int K, int S, int sliding_window) {
    static const long target_env = env_long("LYRA_ATTN_TARGET_WGS");  // tuning overrides, read once
    static const long waves_env = env_long("LYRA_ATTN_WAVES");
    int span = S;  // longest visible range, measured from its tile-aligned start
    if (sliding_window > 0) span = std::min(S, sliding_window + kTile - 1);
    const long pairs = (long)B * K;
    AttnPlan pl;
    pl.waves = 4;
    if (waves_env == 4 || waves_env == 8 || waves_env == 16) pl.waves = (int)waves_env;
    const int unit = pl.waves * kTile;
    const int max_chunks = (span + unit - 1) / unit;
    const long target = target_env > 0 ? target_env : 256;  // workgroups: one per compute unit
    long want = (target + pairs - 1) / pairs;
    if (span <= 2 * 128) want = 1;  // a window of a few tiles: one workgroup, no merge
    if (pairs > kMaxSplitPairs) want = 1;
    int n_chunks = (int)std::max(1L, std::min((long)max_chunks, want));
    int chunk = (span + n_chunks - 1) / n_chunks;
    chunk = (chunk + unit - 1) / unit * unit;
    pl.n_chunks = (span + chunk - 1) / chunk;
    pl.chunk = chunk;
    return pl;
}

}  // namespace lyra

namespace lyra {
struct AttnWorkspace {
    size_t arrivals_bytes, o_bytes, ml_bytes;
    size_t total() const { return arrivals_bytes + o_bytes + ml_bytes; }
};
static AttnWorkspace attention_workspace(int B, int N, int K, int H, const AttnPlan& pl) {
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    AttnWorkspace w;
    // fixed size whatever the shape, so calls of different shapes sharing one workspace never leave
    // partial results where another call's counters live (chunking only happens below kMaxSplitPairs pairs)
    w.arrivals_bytes = kMaxSplitPairs * sizeof(int);
    const size_t items = (size_t)B * K * pl.n_chunks * (N / K);
    w.o_bytes = up(items * H * sizeof(float));
    w.ml_bytes = up(items * 2 * sizeof(float));
    return w;
}
__global__ void zero_fill_kernel(uint32_t* p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}
}  // namespace lyra

extern "C" size_t lyra_decode_attention_workspace(int B, int N, int K, int S, int H, int sliding_window) {
    if (B <= 0 || N <= 0 || K <= 0 || S <= 0 || H <= 0 || N % K) return 0;
    const lyra::AttnPlan pl = lyra::plan_attention(B, K, S, sliding_window);
    if (pl.n_chunks == 1) return 256;
    return lyra::attention_workspace(B, N, K, H, pl).total();
}

extern "C" int lyra_workspace_init(void* workspace, size_t workspace_bytes, lyra_stream_t stream) {
    if (!workspace || workspace_bytes % 4 || ((uintptr_t)workspace % 4)) return LYRA_E_BADARG;
    if (workspace_bytes == 0) return LYRA_OK;
    const size_t n = workspace_bytes / 4;
    const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 4096);
    hipLaunchKernelGGL(lyra::zero_fill_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)workspace, n);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

namespace lyra {
// Validates and launches; shared by the entry point that takes the caller's workspace and the one that uses the static
// scratch buffer.  too_small is what an insufficient workspace is reported as.
// The step in front of the attention, when the launch is to do it (lyra_decode_attention_qkv).
struct QkvFront {
    const void* qkv;
    const float* partials;
    int splits;
    const float* bias;  // of the projection whose slices `partials` are, or null
    const float *qnorm, *knorm, *cos_t, *sin_t;
    int rope_rows;
    float eps;
};

static int run_attention(const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                         const float* sinks, const int32_t* position, int position_stride, const void* gate, void* out,
                         void* workspace, size_t workspace_bytes, int too_small, bool clear_counters, const void* xsa_v,
                         const float* xsa_alpha, int B, int N, int K, int S, int H, float sm_scale, int sliding_window,
                         int kv_dtype, int out_dtype, lyra_stream_t stream, const QkvFront* front = nullptr,
                         const int32_t* row_order = nullptr) {
    if ((!q && !front) || !k || !v || !sinks || !position || !out) return LYRA_E_BADARG;
    if (front) {
        if ((front->partials ? front->splits <= 0 : !front->qkv) || !front->cos_t || !front->sin_t || front->rope_rows <= 0)
            return LYRA_E_BADARG;
        if ((front->qnorm == nullptr) != (front->knorm == nullptr)) return LYRA_E_BADARG;
        if (xsa_v) return LYRA_E_UNSUPPORTED;  // the unit-length value row is handed over by lyra_qkv_post only
        const double width = (double)(N + 2 * K) * H;
        if ((double)std::max(front->splits, 1) * B * width * 4 >= 2147483648.0 || (double)front->rope_rows * H * 2 >= 2147483648.0)
            return LYRA_E_UNSUPPORTED;  // (byte offsets into the slices and the rotary tables are 32-bit)
    }
    if (B <= 0 || N <= 0 || K <= 0 || S <= 0 || H <= 0 || N % K || sliding_window < 0) return LYRA_E_BADARG;
    if (position_stride != 0 && position_stride != 1) return LYRA_E_BADARG;
    if ((xsa_v == nullptr) != (xsa_alpha == nullptr)) return LYRA_E_BADARG;
    if (kv_dtype != LYRA_DTYPE_BF16 && kv_dtype != LYRA_DTYPE_E4M3FN && kv_dtype != LYRA_DTYPE_E5M2) return LYRA_E_UNSUPPORTED;
    if (out_dtype != LYRA_DTYPE_BF16 && out_dtype != LYRA_DTYPE_F32) return LYRA_E_UNSUPPORTED;
    const bool fp8 = kv_dtype != LYRA_DTYPE_BF16, e5m2 = kv_dtype == LYRA_DTYPE_E5M2;
    if (fp8 != (k_scale != nullptr) || fp8 != (v_scale != nullptr)) return LYRA_E_BADARG;
    const int G = N / K;
    if ((H != 64 && H != 128) || G > 16) return LYRA_E_UNSUPPORTED;
    if (K > 65535 || B > 65535) return LYRA_E_UNSUPPORTED;

    AttnPlan pl = plan_attention(B, K, S, sliding_window);
    // ranked rows: only the unchunked global-layer launch with one position per row and more pairs than compute units deals
    // pairs out by length; every other launch ignores the order
    const bool ranked = row_order && position_stride == 1 && sliding_window == 0 && pl.n_chunks == 1 && (long)B * K > 256 && !front;
    if (ranked) {
        static const long ranked_waves_env = env_long("LYRA_ATTN_RANKED_WAVES");  // tuning override, read once
        pl.waves = (ranked_waves_env == 4 || ranked_waves_env == 8) ? (int)ranked_waves_env : (H == 64 ? 8 : 4);
    }
    AttnParams p;
    p.row_order = ranked ? row_order : nullptr;
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
    const bool vec4 = (S % 4 == 0) && (((uintptr_t)k_scale | (uintptr_t)v_scale) % 16 == 0);
    p.scale_vec4 = vec4;
    p.xsa_v = (const uint16_t*)xsa_v;
    p.xsa_alpha = xsa_alpha;
    p.xsa_lds = 0;
    p.qkv_partials = nullptr;
    p.qkv = nullptr;
    p.qkv_splits = 0;
    p.qkv_bias = nullptr;
    p.qnorm = p.knorm = p.cos_t = p.sin_t = nullptr;
    p.rope_rows = 0;
    p.norm_eps = 0.f;
    if (front) {
        p.qkv_partials = front->partials;
        p.qkv = (const uint16_t*)front->qkv;
        p.qkv_splits = front->splits;
        p.qkv_bias = front->partials ? front->bias : nullptr;
        p.qnorm = front->qnorm;
        p.knorm = front->knorm;
        p.cos_t = front->cos_t;
        p.sin_t = front->sin_t;
        p.rope_rows = front->rope_rows;
        p.norm_eps = front->eps;
    }
    p.arrivals = nullptr;
    if (pl.n_chunks > 1) {
        const AttnWorkspace w = attention_workspace(B, N, K, H, pl);
        if (!workspace || ((uintptr_t)workspace % 256)) return LYRA_E_WORKSPACE;
        if (workspace_bytes < w.total()) return too_small;
        p.arrivals = (int*)workspace;
        p.part_o = (float*)((char*)workspace + w.arrivals_bytes);
        p.part_ml = (float*)((char*)workspace + w.arrivals_bytes + w.o_bytes);
    }

    hipStream_t st = (hipStream_t)stream;
    if (clear_counters && p.arrivals) {  // a fill kernel, not a memset node: safe to record into a graph
        const size_t n = (size_t)B * K;
        hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 64)), dim3(256), 0, st,
                           (uint32_t*)p.arrivals, n);
        if (hipGetLastError() != hipSuccess) return LYRA_E_LAUNCH;
    }
    const dim3 grid(pl.n_chunks, K, B), block(pl.waves * 64);
    const size_t lds_merge = ((size_t)pl.waves * G * (H + 4) + 2 * pl.waves * 16 + 32) * sizeof(float);
    const size_t lds_q = (size_t)(pl.waves * 64 / (H / 8)) * (H + 8) * sizeof(uint16_t);  // one 16-byte piece of q per thread
    const size_t lds_stage = pl.n_chunks > 1 ? kMergeStageFloats * sizeof(float) : 0;
    // behind the rest: the staging area of the exclusive-self-attention step, or (front step) of the new key and value rows
    const size_t lds_xsa = xsa_v ? ((size_t)G * H + 16) * sizeof(float) : (front ? (size_t)2 * H * 2 + 16 : 0);
    const size_t lds_base = (std::max(std::max(lds_merge, lds_q), lds_stage) + 15) / 16 * 16;
    const size_t lds = lds_base + lds_xsa;
    p.xsa_lds = (int)(lds_base / sizeof(float));
    // Whole-row launch: more (row, kv head) pairs than compute units, no window.  LYRA_ATTN_ROWS=0 switches it off,
    // =1 takes it only for one position per row (rows of different lengths), =2 also for a shared position;
    // LYRA_ATTN_ROWS_WAVES (4 or 8) overrides the wavefront count.
    static const char* rows_env = getenv("LYRA_ATTN_ROWS");
    static const long rows_mode = rows_env ? atol(rows_env) : 1;
    static const long rows_waves_env = env_long("LYRA_ATTN_ROWS_WAVES");
    const bool rows = !ranked && rows_mode > 0 && (position_stride == 1 || rows_mode > 1) && sliding_window == 0 && pl.n_chunks == 1 &&
                      (long)B * K > 256 && B <= kMaxRankedRows;
    // the front step exists in the chunked kernel with 4 wavefronts only; the caller takes the two launches otherwise
    if (front && (rows || pl.waves != 4)) return LYRA_E_UNSUPPORTED;
    if (rows) {
        const int waves = (rows_waves_env == 4 || rows_waves_env == 8) ? (int)rows_waves_env : (H == 64 ? 8 : 4);
        const size_t lds_need = std::max(((size_t)waves * G * (H + 4) + 2 * waves * 16 + 32) * sizeof(float),
                                         (size_t)(waves * 64 / (H / 8)) * (H + 8) * sizeof(uint16_t));
        // more than half of a compute unit's 160 KB: one workgroup per unit
        const size_t lds_need_x = (lds_need + 15) / 16 * 16;
        p.xsa_lds = (int)(lds_need_x / sizeof(float));
        const size_t lds_r = std::max(lds_need_x + lds_xsa, (size_t)81 * 1024);
        const dim3 grid_r(256), block_r(waves * 64);
#define LYRA_LAUNCH_ATTN_R(HH, F, V, W)                                                                        \
    do {                                                                                                      \
        auto kern = decode_attention_rows_kernel<HH, F, V, W>;                                                \
        static const hipError_t attr =                                                                        \
            hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);    \
        if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                         \
        hipLaunchKernelGGL(kern, grid_r, block_r, lds_r, st, p);                                              \
    } while (0)
#define LYRA_LAUNCH_ATTN_RW(HH, F, V)                    \
    do {                                                 \
        if (waves == 4) LYRA_LAUNCH_ATTN_R(HH, F, V, 4); \
        else LYRA_LAUNCH_ATTN_R(HH, F, V, 8);            \
    } while (0)
        // (the second argument is the cache format: 0 bf16, 1 e4m3fn, 2 e5m2)
        if (H == 128) {
            if (!fp8) LYRA_LAUNCH_ATTN_RW(128, 0, false);
            else if (e5m2 && vec4) LYRA_LAUNCH_ATTN_RW(128, 2, true);
            else if (e5m2) LYRA_LAUNCH_ATTN_RW(128, 2, false);
            else if (vec4) LYRA_LAUNCH_ATTN_RW(128, 1, true);
            else LYRA_LAUNCH_ATTN_RW(128, 1, false);
        } else {
            if (!fp8) LYRA_LAUNCH_ATTN_RW(64, 0, false);
            else if (e5m2 && vec4) LYRA_LAUNCH_ATTN_RW(64, 2, true);
            else if (e5m2) LYRA_LAUNCH_ATTN_RW(64, 2, false);
            else if (vec4) LYRA_LAUNCH_ATTN_RW(64, 1, true);
            else LYRA_LAUNCH_ATTN_RW(64, 1, false);
        }
#undef LYRA_LAUNCH_ATTN_RW
#undef LYRA_LAUNCH_ATTN_R
        if (hipGetLastError() != hipSuccess) return LYRA_E_LAUNCH;
        return LYRA_OK;
    }
#define LYRA_LAUNCH_ATTN_W(HH, F, V, W)                                                                        \
    do {                                                                                                      \
        if (sliding_window == 0) hipLaunchKernelGGL((decode_attention_kernel<HH, F, V, W, true, 1>), grid, block, lds, st, p); \
        else hipLaunchKernelGGL((decode_attention_kernel<HH, F, V, W, false, 1>), grid, block, lds, st, p);      \
    } while (0)
#define LYRA_LAUNCH_ATTN(HH, F, V)                              \
    do {                                                        \
        if (front) {                                            \
            if (sliding_window == 0) hipLaunchKernelGGL((decode_attention_kernel<HH, F, V, 4, true, 1, true>), grid, block, lds, st, p); \
            else hipLaunchKernelGGL((decode_attention_kernel<HH, F, V, 4, false, 1, true>), grid, block, lds, st, p); \
        } else if (pl.waves == 4) LYRA_LAUNCH_ATTN_W(HH, F, V, 4); \
        else if (pl.waves == 8) LYRA_LAUNCH_ATTN_W(HH, F, V, 8); \
        else LYRA_LAUNCH_ATTN_W(HH, F, V, 16);                  \
    } while (0)
    if (H == 128) {
        if (!fp8) LYRA_LAUNCH_ATTN(128, 0, false);
        else if (e5m2 && vec4) LYRA_LAUNCH_ATTN(128, 2, true);
        else if (e5m2) LYRA_LAUNCH_ATTN(128, 2, false);
        else if (vec4) LYRA_LAUNCH_ATTN(128, 1, true);
        else LYRA_LAUNCH_ATTN(128, 1, false);
    } else {
        if (!fp8) LYRA_LAUNCH_ATTN(64, 0, false);
        else if (e5m2 && vec4) LYRA_LAUNCH_ATTN(64, 2, true);
        else if (e5m2) LYRA_LAUNCH_ATTN(64, 2, false);
        else if (vec4) LYRA_LAUNCH_ATTN(64, 1, true);
        else LYRA_LAUNCH_ATTN(64, 1, false);
    }
#undef LYRA_LAUNCH_ATTN
#undef LYRA_LAUNCH_ATTN_W
    if (hipGetLastError() != hipSuccess) return LYRA_E_LAUNCH;
    return LYRA_OK;
}

// ---- static scratch for callers that cannot allocate -----------------------------------------------
// One copy of this array lives on every GPU the library is loaded on, from load until the process ends.  Host code never
// uses the array's name as an address: the device address is asked for once per device and kept.
static __device__ __align__(256) unsigned char scratch[LYRA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, null until first asked for
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device, or null if the runtime cannot tell.
static void* static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace lyra

extern "C" int lyra_decode_attention_qkv(const void* qkv, const float* partials, int splits, const float* qnorm,
                                         const float* knorm, const float* cos_t, const float* sin_t, int rope_rows, float eps,
                                         void* k, void* v, float* k_scale, float* v_scale, const float* sinks,
                                         const int32_t* position, int position_stride, const void* gate, void* out,
                                         void* workspace, size_t workspace_bytes, int B, int N, int K, int S, int H,
                                         float sm_scale, int sliding_window, int kv_dtype, int out_dtype,
                                         lyra_stream_t stream) {
    return lyra_decode_attention_qkv_bias(qkv, partials, splits, nullptr, qnorm, knorm, cos_t, sin_t, rope_rows, eps, k, v, k_scale,
                                          v_scale, sinks, position, position_stride, gate, out, workspace, workspace_bytes, B, N, K, S,
                                          H, sm_scale, sliding_window, kv_dtype, out_dtype, stream);
}

extern "C" int lyra_decode_attention_qkv_bias(const void* qkv, const float* partials, int splits, const float* qkv_bias,
                                              const float* qnorm, const float* knorm, const float* cos_t, const float* sin_t,
                                              int rope_rows, float eps, void* k, void* v, float* k_scale, float* v_scale,
                                              const float* sinks, const int32_t* position, int position_stride, const void* gate,
                                              void* out, void* workspace, size_t workspace_bytes, int B, int N, int K, int S, int H,
                                              float sm_scale, int sliding_window, int kv_dtype, int out_dtype,
                                              lyra_stream_t stream) {
    if (qkv_bias && !partials) return LYRA_E_BADARG;  // (a summed projection already carries its bias)
    const lyra::QkvFront front{qkv, partials, splits, qkv_bias, qnorm, knorm, cos_t, sin_t, rope_rows, eps};
    return lyra::run_attention(nullptr, k, v, k_scale, v_scale, sinks, position, position_stride, gate, out, workspace,
                               workspace_bytes, LYRA_E_WORKSPACE, false, nullptr, nullptr, B, N, K, S, H, sm_scale,
                               sliding_window, kv_dtype, out_dtype, stream, &front);
}

extern "C" int lyra_decode_attention(const void* q, const void* k, const void* v, const float* k_scale,
                                     const float* v_scale, const float* sinks, const int32_t* position,
                                     int position_stride, const void* gate, void* out, void* workspace,
                                     size_t workspace_bytes, int B, int N, int K, int S, int H, float sm_scale,
                                     int sliding_window, int kv_dtype, int out_dtype, lyra_stream_t stream) {
    return lyra::run_attention(q, k, v, k_scale, v_scale, sinks, position, position_stride, gate, out, workspace, workspace_bytes,
                               LYRA_E_WORKSPACE, false, nullptr, nullptr, B, N, K, S, H, sm_scale, sliding_window, kv_dtype,
                               out_dtype, stream);
}

namespace lyra {
// rank[i] = the row with the i-th largest position (ties: the lower row first); one workgroup, thread t places row t
__global__ __launch_bounds__(1024) void attention_rank_kernel(const int32_t* position, int B, int32_t* order) {
    extern __shared__ int sm_rank_pos[];
    for (int i = threadIdx.x; i < B; i += blockDim.x) sm_rank_pos[i] = position[i];
    __syncthreads();
    for (int t = threadIdx.x; t < B; t += blockDim.x) {
        const int mine = sm_rank_pos[t];
        int rank = 0;
        for (int j = 0; j < B; ++j) {
            const int other = sm_rank_pos[j];
            rank += (other > mine) || (other == mine && j < t);
        }
        order[rank] = t;
    }
}
}  // namespace lyra

extern "C" int lyra_attention_rank(const int32_t* position, int B, int32_t* row_order, lyra_stream_t stream) {
    if (!position || !row_order || B <= 0) return LYRA_E_BADARG;
    if (B > 8192) return LYRA_E_UNSUPPORTED;
    const int threads = std::min(1024, (B + 63) / 64 * 64);
    hipLaunchKernelGGL(lyra::attention_rank_kernel, dim3(1), dim3(threads), (size_t)B * sizeof(int), (hipStream_t)stream, position, B,
                       row_order);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

extern "C" int lyra_decode_attention_ranked(const void* q, const void* k, const void* v, const float* k_scale,
                                            const float* v_scale, const float* sinks, const int32_t* position,
                                            int position_stride, const int32_t* row_order, const void* gate, void* out,
                                            void* workspace, size_t workspace_bytes, int B, int N, int K, int S, int H,
                                            float sm_scale, int sliding_window, int kv_dtype, int out_dtype, lyra_stream_t stream) {
    if (!row_order) return LYRA_E_BADARG;
    return lyra::run_attention(q, k, v, k_scale, v_scale, sinks, position, position_stride, gate, out, workspace, workspace_bytes,
                               LYRA_E_WORKSPACE, false, nullptr, nullptr, B, N, K, S, H, sm_scale, sliding_window, kv_dtype,
                               out_dtype, stream, nullptr, row_order);
}

extern "C" int lyra_decode_attention_xsa(const void* q, const void* k, const void* v, const float* k_scale,
                                         const float* v_scale, const float* sinks, const int32_t* position,
                                         int position_stride, const void* gate, const void* v_unit, const float* xsa_alpha,
                                         void* out, void* workspace, size_t workspace_bytes, int B, int N, int K, int S, int H,
                                         float sm_scale, int sliding_window, int kv_dtype, int out_dtype, lyra_stream_t stream) {
    return lyra::run_attention(q, k, v, k_scale, v_scale, sinks, position, position_stride, gate, out, workspace, workspace_bytes,
                               LYRA_E_WORKSPACE, false, v_unit, xsa_alpha, B, N, K, S, H, sm_scale, sliding_window, kv_dtype,
                               out_dtype, stream);
}

extern "C" int lyra_decode_attention_static(const void* q, const void* k, const void* v, const float* k_scale,
                                            const float* v_scale, const float* sinks, const int32_t* position,
                                            int position_stride, const void* gate, void* out, int B, int N, int K, int S, int H,
                                            float sm_scale, int sliding_window, int kv_dtype, int out_dtype,
                                            lyra_stream_t stream) {
    if (!q || !k || !v || !sinks || !position || !out) return LYRA_E_BADARG;
    void* ptr = lyra::static_scratch();
    if (!ptr) return LYRA_E_LAUNCH;
    // the arrival counters this call uses are cleared first: the buffer keeps whatever the last call on this GPU left
    return lyra::run_attention(q, k, v, k_scale, v_scale, sinks, position, position_stride, gate, out, ptr,
                               (size_t)LYRA_STATIC_SCRATCH_BYTES, LYRA_E_SCRATCH, true, nullptr, nullptr, B, N, K, S, H, sm_scale,
                               sliding_window, kv_dtype, out_dtype, stream);
}
