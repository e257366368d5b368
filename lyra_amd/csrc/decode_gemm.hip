// Decode grouped matmul for gfx950: out[r,:] = epilogue(lhs[r,:] @ rhs[expert(r)]) for a handful of
// rows per expert, weights BF16 or block-scaled FP8 (e4m3fn), optional bias and fused SwiGLU.
//
// Maths (lyra/kernels/gemm.py:1575-1617 as called from lyra/kernels/decode_gemm.py:390-399):
//   t = ragged_dot(lhs, W^, group_sizes) in float32;  t += bias[expert];  t = swiglu(t);  cast
// with W^ = f32(Wq) * scale[k/bk, n/bn].  The kernel streams every weight byte of a touched expert
// exactly once (experts with no rows are never read), multiplies raw FP8 values converted exactly
// to BF16 on the matrix cores and applies the block scales to the float32 accumulators.
//
// Mapping: the weight matrix is row-major [K,N] (N contiguous).  A wavefront owns 128 output columns
// (64 gate + 64 linear columns when SwiGLU is fused) and walks K in steps of 32 rows; the 4 wavefronts of a
// workgroup share the activations, staged in LDS 512 rows of K at a time.  Lane
// (x = lane & 15, kb = lane >> 4) reads 8 consecutive columns of the 8 rows 8*kb .. 8*kb+7; pairing two
// rows in the bf16 pack step yields the K-major B operand, so the transposition costs nothing.
//   D[16 rows, 16 cols] += X[16 rows x 32 k] . W[32 k x 16 cols]   for each of the 8 column phases.
//
// This file is compiled in several passes, selected by LYRA_GEMM_PART, and the objects are linked:
//   1  the C entry points, the planning, the finish and pack kernels and the launches of the bf16 and e4m3fn kernels
//   2  the K-split kernels for bf16 and e4m3fn weights, built with the compiler's option that keeps matrix-core
//      accumulators in ordinary vector registers: those kernels do one or two matrix instructions per accumulator and the
//      copies to and from the accumulator file were a sixth of their instructions (the option makes the expert kernel
//      spill registers, so the other passes are built without it)
//   3  the launches of pass 1 for e5m2 weights;  4  the kernels of pass 2 for e5m2 weights
// Without the macro the file is one complete translation unit.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "lyra_device.h"

#ifndef LYRA_GEMM_PART
#define LYRA_GEMM_PART 0
#endif
#if LYRA_GEMM_PART < 0 || LYRA_GEMM_PART > 4
#error "LYRA_GEMM_PART: 0 (everything) or one of the passes 1-4"
#endif
#define LYRA_GEMM_HAS_ENTRY (LYRA_GEMM_PART == 0 || LYRA_GEMM_PART == 1)
#define LYRA_GEMM_HAS_LAUNCH (LYRA_GEMM_PART == 0 || LYRA_GEMM_PART == 1 || LYRA_GEMM_PART == 3)
#define LYRA_GEMM_HAS_SPLITK (LYRA_GEMM_PART == 0 || LYRA_GEMM_PART == 2 || LYRA_GEMM_PART == 4)

namespace lyra {

// the weight formats of one byte per element (block-scaled)
static inline bool one_byte_format(int dtype) { return dtype == LYRA_DTYPE_E4M3FN || dtype == LYRA_DTYPE_E5M2; }

struct GemmParams {
    const uint16_t* lhs;
    const uint8_t* rhs;
    const float* scale;
    const int32_t* group_sizes;
    const float* bias;
    void* out;
    float* part;  // [ksplit, M, N] float32 partial products when ksplit > 1; grouped: two tile slots per workgroup
    int* arrivals;  // grouped: arrival counters of split units (zero between launches)
    int M, G, K, N;
    int bk, bn, KB, NB;
    int bn_shift;  // log2(bn): scale columns are power-of-two wide
    int bk_shift;  // log2(bk) when bk is a power of two, else -1
    int scale_mode;  // 0 none, 1 one scale per lane and k-block (bn % 8 == 0), 2 per column (bk == K)
    int out_f32, swiglu;
    float beta, limit;
    int ksplit, kpart;  // kpart: rows of K per split, multiple of 32 (and of bk when bk < K)
    int row_par;        // row blocks of a group that run as separate workgroups (grid.z = G * row_par)
    int wide;           // grouped kernel without SwiGLU: units of 256 columns (two wavefront pairs)
    int bias_post;      // one group, no SwiGLU: the bias is added to the bf16-rounded product, in bf16 (then scale / residual)
    int max_slices;     // grouped kernel: most K slices a left-over unit is cut into
    int snake;          // grouped kernel: odd rounds of units run over the workgroups in the opposite direction (-1: if >= 4 rounds)
    int touch_last;     // grouped kernel: touch the first weights of the last group's units before the unit list is known
    int even_spans;     // plain kernel: spans dealt out evenly over one workgroup per compute unit
    int row_block;      // K-split kernel: rows per workgroup (64 or 32)
    const int32_t* row_map;    // lhs row that feeds sorted row r (gather fused into the activation load), or null
    const uint16_t* residual;  // bf16 [M, NO] added after scaling, or null
    float out_scale;           // epilogue: out = bf16(residual + bf16(bf16(t) * out_scale)) when post_scale is set
    int post_scale;
    // span-major weights (lyra_gemm_pack): 0 = rhs is [G,K,N]; 1 = [G][pspans][K][128], span s = columns 128 s ...;
    // 2 = the same with span s = gate columns 64 s ... followed by their linear columns N/2 + 64 s ...
    int packed;
    int pspans;
    // Activations in tiles of 16 rows x 32 columns (1 KB each, tiles of a row block side by side): element (r, k) of an
    // array of C columns lies at (((r >> 4) * (C >> 5) + (k >> 5)) * 16 + (r & 15)) * 32 + (k & 31).  The 16 lanes that feed
    // one matrix instruction with 16 consecutive rows then read one contiguous KB instead of 16 pieces a row apart.
    // lhs_tiled: lhs comes in that layout (grouped kernel); out_tiled: the bf16 output is written in it (for the next matmul).
    int lhs_tiled, out_tiled;
    // Plain kernel, one group, float32 output, K not split: the maximum of every 128-column tile of every output row,
    // [M, tile_ld] float32 (tile t = columns 128 t ...; NaNs are skipped as fmaxf skips them), for a sampler that then
    // only looks into the few tiles that can hold a row's best values.  Null: not wanted.
    float* tile_max;
    int tile_ld;
};

// Element index of output (row, col .. col + 3) in an array of NO columns, row-major or tiled (GemmParams::out_tiled).
__device__ __forceinline__ size_t out_index(const GemmParams& p, int row, int col, int NO) {
    if (p.out_tiled) return ((((size_t)(row >> 4) * (NO >> 5) + (col >> 5)) * 16 + (row & 15)) << 5) + (col & 31);
    return (size_t)row * NO + col;
}

// Results go out with plain stores; only the float32 K slices that the next kernel sums are written through at agent
// scope (store_through): a K-split launch leaves 3-8 MB of them, and written back at the end of the kernel instead they
// cost the decode step 1.5 %.  (Writing every result through - expert outputs, logits - was measured too: 0.5 % slower than
// the slices alone.)
template <typename T> __device__ __forceinline__ void out_store(void* base, size_t off, T v) { *(T*)((char*)base + off) = v; }
__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// Index of the scale block (along K) that weight row k lies in.
__device__ __forceinline__ int scale_block_of(const GemmParams& p, int k) {
    k = min(k, p.K - 1);
    return p.bk_shift >= 0 ? k >> p.bk_shift : k / p.bk;
}

// Scale of one lane's 8 columns for one K step, fetched like the step's weights (a buffer load in the same in-order
// stream, so waiting for it never waits for younger loads; a plain pointer load here would drain everything in flight).
// lane_off: byte offset of the lane's scale column within the group's scale table, or kNoLoad.
__device__ __forceinline__ float load_step_scale(const GemmParams& p, const __amdgpu_buffer_rsrc_t& rsrc, bool live, int lane_off,
                                                 int k) {
    const int soff = __builtin_amdgcn_readfirstlane(live ? scale_block_of(p, k) * p.NB * 4 : 0);
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, live ? lane_off : kNoLoad, soff, 0));
}

// Residual epilogue of a projection (lyra/model.py:371-374, 631-636): the product is a bf16 array, it is scaled in
// bf16, then added to the bf16 residual stream.
__device__ __forceinline__ float residual_epilogue(const GemmParams& p, float t, size_t idx) {
    t = round_bf16(round_bf16(t) * p.out_scale);
    if (p.residual) t += bf16_bits_to_f32(p.residual[idx]);
    return t;
}

__device__ __forceinline__ float swiglu_one(float glu, float lin, float beta, float limit) {
    glu = fminf(glu, limit);
    lin = fminf(fmaxf(lin, -limit), limit);
    const float sig = __builtin_amdgcn_rcpf(1.0f + fast_exp2(-beta * kLog2e * glu));  // (1 ulp; the division sequence is 10 instructions)
    return (lin + 1.0f) * (glu * sig);
}

constexpr int kGemmWaves = 4;  // wavefronts per workgroup, each on its own 128-column span

// The template argument FP8 of everything below is the weight format: 0 bf16, 1 e4m3fn, 2 e5m2 (both 1-byte formats go the
// same way - codes converted exactly to bf16, block scales on the float32 accumulators - and differ in one instruction).
template <int FP8>
struct RawW {
    static constexpr int WW = FP8 ? 2 : 4;  // dwords per lane per weight row (8 columns)
    uint32_t w[8][WW];
};

// Two of the 8 weight rows of this lane (rows kk + 8*kb + 2*pair, +1), 8 columns each.  The lane part of the
// address is fixed (voff); the row part is uniform and travels in a scalar register.
template <int FP8>
__device__ __forceinline__ void load_w_pair(RawW<FP8>& t, int pair, __amdgpu_buffer_rsrc_t rsrc, int voff, int kk, int row_bytes) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int i = 2 * pair + h;
        const int soff = __builtin_amdgcn_readfirstlane((kk + i) * row_bytes);
        if constexpr (FP8) {
            const u32x2 d = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, soff, kStream);
            t.w[i][0] = d[0];
            t.w[i][1] = d[1];
        } else {
            const u32x4 d = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, kStream);
            t.w[i][0] = d[0];
            t.w[i][1] = d[1];
            t.w[i][2] = d[2];
            t.w[i][3] = d[3];
        }
    }
}

// Loads that may
// run past the end of the data are issued unconditionally with the lane offset kNoLoad instead of being branched around, so
// that the number of loads in flight is the same on every path and each wait covers exactly the loads it needs
// (a load inside a branch makes the compiler wait for every outstanding load at the next use).

template <int FP8>
__device__ __forceinline__ void load_w_pair_if(bool live, RawW<FP8>& t, int pair, __amdgpu_buffer_rsrc_t rsrc, int voff, int kk,
                                               int row_bytes) {
    load_w_pair<FP8>(t, pair, rsrc, live ? voff : kNoLoad, live ? kk : 0, live ? row_bytes : 0);
}

// Element `pair` of the K-major B operands of all 8 column phases: pairing two weight rows in the bf16 pack
// step transposes the row-major weights for free.
template <int FP8>
__device__ __forceinline__ void convert_pair(const RawW<FP8>& t, int pair, Pack8 (&bop)[8]) {
    const int i = 2 * pair;
#pragma unroll
    for (int c = 0; c < 8; c += 2) {
        if constexpr (FP8) {
            // the two rows' codes of columns c, c + 1 side by side (row i, row i + 1, row i, row i + 1), then one exact
            // conversion per pair: 3 instructions for 4 weights
            const uint32_t both = __builtin_amdgcn_perm(t.w[i + 1][c >> 2], t.w[i][c >> 2], (c & 2) ? 0x07030602u : 0x05010400u);
            bop[c].u[pair] = codes2_to_bf16x2<FP8>(both, false);
            bop[c + 1].u[pair] = codes2_to_bf16x2<FP8>(both, true);
        } else {
            const uint32_t a = t.w[i][c >> 1], b = t.w[i + 1][c >> 1];
            bop[c].u[pair] = __builtin_amdgcn_perm(b, a, 0x05040100u);
            bop[c + 1].u[pair] = __builtin_amdgcn_perm(b, a, 0x07060302u);
        }
    }
}

// The K-major B operands of column phases 2*cp and 2*cp + 1 from all 8 weight rows of this lane (what convert_pair does for
// one row pair and all phases, done for all row pairs and one pair of phases).
// SCALED: every value is multiplied by `scale` in float32 before it is rounded to bf16 - the dequantisation of the plain-JAX
// path, bit for bit: dequantize() forms f32(code) * scale and casts to the activation dtype (lyra/nn/quant.py:82-85).
template <int FP8, bool SCALED = false>
__device__ __forceinline__ void convert_colpair(const RawW<FP8>& t, int cp, Pack8& b0, Pack8& b1, float scale = 1.f) {
    const int c = 2 * cp;
#pragma unroll
    for (int pr = 0; pr < 4; ++pr) {
        const int i = 2 * pr;
        if constexpr (FP8) {
            // (the byte shuffle + single conversion of convert_pair - 3 instead of 4 instructions for 4 weights - was
            // measured here too: no faster, the lyra-max down projection 1.3 % slower; this loop hides its conversions
            // behind matrix instructions already)
            f32x2 fa = codes2_to_f32<FP8>(t.w[i][c >> 2], (c & 2) != 0);
            f32x2 fb = codes2_to_f32<FP8>(t.w[i + 1][c >> 2], (c & 2) != 0);
            if constexpr (SCALED) {
                fa[0] *= scale;
                fa[1] *= scale;
                fb[0] *= scale;
                fb[1] *= scale;
            }
            b0.u[pr] = pack_bf16(fa[0], fb[0]);
            b1.u[pr] = pack_bf16(fa[1], fb[1]);
        } else {
            const uint32_t a = t.w[i][c >> 1], b = t.w[i + 1][c >> 1];
            b0.u[pr] = __builtin_amdgcn_perm(b, a, 0x05040100u);
            b1.u[pr] = __builtin_amdgcn_perm(b, a, 0x07060302u);
        }
    }
}

// Writes 8 consecutive result columns of one row: fused epilogue (ksplit == 1) or float32 partials.
// Must be called by all lanes of the wavefront (SwiGLU exchanges gate and linear halves by shuffle);
// `store` says whether this lane's row exists.
__device__ __forceinline__ void finish_row(const GemmParams& p, float (&t)[8], const float (&bias8)[8], int row, int ncol, int out_col,
                                           int ks, bool store, bool is_lin_lane) {
    if (p.ksplit > 1) {
        if (store) {
            const size_t dst = (((size_t)ks * p.M + row) * p.N + ncol) * 4;
            store_through(p.part, dst, f32x4{t[0], t[1], t[2], t[3]});
            store_through(p.part, dst + 16, f32x4{t[4], t[5], t[6], t[7]});
        }
        return;
    }
    if (p.bias_post) {  // (the lane's 8 bias values were loaded once, by the caller)
#pragma unroll
        for (int c = 0; c < 8; ++c) t[c] = round_bf16(round_bf16(t[c]) + bias8[c]);
    } else if (p.bias) {
#pragma unroll
        for (int c = 0; c < 8; ++c) t[c] += bias8[c];
    }
    int NO = p.N;
    if (p.swiglu) {
        NO = p.N / 2;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float other = __shfl_xor(t[c], 8, kWave);  // gate lanes x<8 pair with linear lanes x+8
            t[c] = swiglu_one(t[c], other, p.beta, p.limit);
        }
        store = store && !is_lin_lane;
    }
    if (store) {
        if (p.post_scale) {
#pragma unroll
            for (int c = 0; c < 8; ++c) t[c] = residual_epilogue(p, t[c], (size_t)row * NO + out_col + c);
        }
        if (p.out_f32) {
            const size_t dst = ((size_t)row * NO + out_col) * 4;
            out_store(p.out, dst, f32x4{t[0], t[1], t[2], t[3]});
            out_store(p.out, dst + 16, f32x4{t[4], t[5], t[6], t[7]});
        } else {
            u32x4 d;
#pragma unroll
            for (int c = 0; c < 4; ++c) d[c] = pack_bf16(t[2 * c], t[2 * c + 1]);
            out_store(p.out, ((size_t)row * NO + out_col) * 2, d);
        }
    }
}

// GemmParams::tile_max: the 16 lanes that hold the 128 columns of one row of a span reduce their finished values (t as
// finish_row left it: bias added) and lane 0 of them (`writer`) stores the maximum.  Called by all lanes.
__device__ __forceinline__ void store_tile_max(const GemmParams& p, const float (&t)[8], int row, int span, bool lane_ok, bool writer) {
    float m = fmaxf(fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3])), fmaxf(fmaxf(t[4], t[5]), fmaxf(t[6], t[7])));
    m = row16_max(lane_ok ? m : -INFINITY);
    if (writer) p.tile_max[(size_t)row * p.tile_ld + span] = m;
}

constexpr int kTileMaxPitch = 20;  // floats per row of a wavefront's tile-maximum staging area (conflict-free for 4 rows x 16 lanes)

template <int FP8, int MT, bool TMAX = false>
__global__ __launch_bounds__(MT == 1 ? 768 : 512) __attribute__((amdgpu_waves_per_eu(MT == 1 ? 3 : 2)))
void decode_gemm_kernel(GemmParams p) {
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int KC = 512;          // rows of K whose activations are staged in LDS at a time
    constexpr int XPITCH = KC + 8;   // LDS pitch of a staged row in bf16 elements (keeps 16-lane reads conflict free)
    extern __shared__ uint16_t sm_x[];  // [16*MT rows][XPITCH] activations of the current K chunk, zero padded
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = lane & 15, kb = lane >> 4;
    const int g = blockIdx.z / p.row_par, rpar = blockIdx.z - g * p.row_par, ks = blockIdx.y;
    const int nwaves = blockDim.x >> 6;
    // which 128-column span this wavefront owns: 4 per workgroup, or (p.even_spans, one workgroup per compute unit)
    // workgroup i of n takes spans [i * total / n, (i + 1) * total / n), so that every compute unit has the same number
    // of spans to within one - 1600 spans as 400 workgroups of 4 leave 144 compute units with 8 spans and 112 with 4
    const int total_spans = p.swiglu ? ((p.N >> 1) + 63) / 64 : (p.N + 127) / 128;  // (the last span may be partly filled)
    const int first_span = p.even_spans ? (int)((long)blockIdx.x * total_spans / gridDim.x) : (int)blockIdx.x * kGemmWaves;
    const int end_span = p.even_spans ? (int)((long)(blockIdx.x + 1) * total_spans / gridDim.x) : total_spans;
    const int span = first_span + wave;
    // (TMAX: behind the activations, 16 * MT rows of kTileMaxPitch floats per wavefront)
    float* const sm_t = (float*)(sm_x + 16 * MT * XPITCH) + wave * (16 * MT * kTileMaxPitch);

    // rows of this group: [off, off + cnt)
    int part_sum = 0;
    for (int i = lane; i < g; i += 64) part_sum += p.group_sizes[i];
    part_sum = wave_sum(part_sum);
    const int off = min(part_sum, p.M);
    const int cnt = min(p.group_sizes[g], p.M - off);
    const int pad_from = (g == p.G - 1 && rpar == 0 && p.ksplit == 1 && ks == 0) ? off + cnt : p.M;  // rows past the last group
    if (cnt <= rpar * 16 * MT && pad_from >= p.M) return;  // no rows for this workgroup: its weights are never touched

    // columns of this lane (span_ok: they exist - N need not be a multiple of the span, only of 8 columns)
    int ncol, out_col;
    bool span_ok;
    const bool is_lin_lane = p.swiglu && x >= 8;
    if (p.swiglu) {
        const int half = p.N >> 1;
        out_col = span * 64 + 8 * (x & 7);
        span_ok = span < end_span && out_col + 8 <= half;
        ncol = is_lin_lane ? half + out_col : out_col;
    } else {
        ncol = out_col = span * 128 + 8 * x;
        span_ok = span < end_span && ncol + 8 <= p.N;
    }
    if (!span_ok) ncol = out_col = 0;  // idle wavefront of the last workgroup, lanes past the last column: keep pace, store nothing

    const int k0 = ks * p.kpart, k1 = min(p.K, k0 + p.kpart);
    // row-major weights: a row of the group's matrix is N elements; span-major (GemmParams::packed, layout 1): this
    // wavefront's span is K contiguous rows of 128 elements, and the spans of a group follow each other
    const int row_bytes = p.packed ? 128 * ES : p.N * ES;
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.rhs) + (size_t)g * (p.packed ? p.pspans * 128 : p.N) * p.K * ES, 0,
        (uint32_t)p.K * (uint32_t)((p.packed ? p.pspans * 128 : p.N) * ES), 0x00020000);
    const int wvoff = p.packed ? ((span < end_span ? span : 0) * p.K + 8 * kb) * row_bytes + 8 * x * ES : 8 * kb * row_bytes + ncol * ES;
    const float* sc_lane = nullptr;
    if (FP8 && p.scale_mode == 1) sc_lane = p.scale + (size_t)g * p.KB * p.NB + (ncol >> p.bn_shift);

    for (int rb = rpar * 16 * MT; rb < cnt; rb += p.row_par * 16 * MT) {
        const int rowbase = off + rb;
        const int rows_here = min(16 * MT, cnt - rb);
        const int n_mt = (rows_here + 15) >> 4;

        f32x4 acc[MT][8];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[mt][c] = f32x4{0.f, 0.f, 0.f, 0.f};

        // accumulators are kept in units of the current block scale; on a k-block boundary they are
        // re-expressed in the next block's unit, and the last unit is applied at the end
        float s_cur = 1.f, s_next = 1.f;
        const float* sc_ptr = sc_lane;  // scale of the k-block that starts at blk_kk
        int blk_kk = k0;
        if (FP8 && p.scale_mode == 1) {
            sc_ptr += (size_t)(k0 / p.bk) * p.NB;
            s_cur = *sc_ptr;
            s_next = s_cur;
        }

        // One register set of raw weights: a pair of rows is requested again (for the next step) as soon as it
        // has been converted, so weight loads are in flight during the whole step.
        RawW<FP8> w;
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) load_w_pair_if<FP8>(k0 < k1, w, pr, wrsrc, wvoff, k0, row_bytes);

        for (int kc = k0; kc < k1; kc += KC) {
            const int kc_end = min(kc + KC, k1);
            // The 4 wavefronts share the activations of this K chunk through LDS: lane = 16-byte piece of a row,
            // wavefront = row phase.  (The first weights of the chunk are already in flight.)
            __syncthreads();  // the previous chunk has been consumed by every wavefront
            const int pieces = (kc_end - kc) >> 3;  // <= 64
            if (lane < pieces) {
                for (int r = wave; r < 16 * n_mt; r += nwaves) {
                    u32x4 d = u32x4{0u, 0u, 0u, 0u};
                    if (r < rows_here) {
                        const int src = p.row_map ? p.row_map[rowbase + r] : rowbase + r;
                        d = *(const u32x4*)(p.lhs + (size_t)src * p.K + kc + lane * 8);
                    }
                    *(u32x4*)(sm_x + r * XPITCH + lane * 8) = d;
                }
            }
            __syncthreads();

            for (int kk = kc; kk < kc_end; kk += 32) {
                const bool more = kk + 32 < k1;
                if (FP8 && p.scale_mode == 1 && p.bk < p.K && kk == blk_kk) {
                    if (kk != k0) {
                        const float ratio = s_cur / s_next;
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            if (mt < n_mt)
#pragma unroll
                                for (int c = 0; c < 8; ++c) {
                                    acc[mt][c][0] *= ratio;
                                    acc[mt][c][1] *= ratio;
                                    acc[mt][c][2] *= ratio;
                                    acc[mt][c][3] *= ratio;
                                }
                        s_cur = s_next;
                    }
                    blk_kk += p.bk;  // prefetch the following block's scale
                    sc_ptr += p.NB;
                    if (blk_kk < k1) s_next = *sc_ptr;
                }
                Pack8 bop[8];
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) {
                    convert_pair<FP8>(w, pr, bop);
                    __builtin_amdgcn_sched_barrier(0);
                    load_w_pair_if<FP8>(more, w, pr, wrsrc, wvoff, kk + 32, row_bytes);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    if (mt < n_mt) {
                        const bf16x8 a = *(const bf16x8*)(sm_x + (mt * 16 + x) * XPITCH + (kk - kc) + 8 * kb);
#pragma unroll
                        for (int c = 0; c < 8; ++c) acc[mt][c] = mfma_16x16x32(a, bop[c].v, acc[mt][c]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        float colscale[8], bias8[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) bias8[c] = (p.bias && p.ksplit == 1) ? p.bias[(size_t)g * p.N + ncol + c] : 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) colscale[c] = s_cur;
        if (FP8 && p.scale_mode == 2) {
#pragma unroll
            for (int c = 0; c < 8; ++c) colscale[c] = p.scale[(size_t)g * p.NB + ((ncol + c) >> p.bn_shift)];
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt < n_mt) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int lr = mt * 16 + 4 * kb + r;
                    float t[8];
#pragma unroll
                    for (int c = 0; c < 8; ++c) t[c] = acc[mt][c][r] * colscale[c];
                    finish_row(p, t, bias8, rowbase + lr, ncol, out_col, ks, span_ok && lr < rows_here, is_lin_lane);
                    if (TMAX) {  // this lane's 8 columns of the row; the row's 16 lanes meet in LDS below
                        const float m = fmaxf(fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3])), fmaxf(fmaxf(t[4], t[5]), fmaxf(t[6], t[7])));
                        sm_t[lr * kTileMaxPitch + x] = span_ok ? m : -INFINITY;
                    }
                }
            }
        }
        if (TMAX) {
            // Lane l takes row l of the block: 16 partial maxima, one store.  Only this wavefront touches its staging area
            // and LDS serves a wavefront's requests in order, so no barrier - the fences keep the compiler from moving
            // the reads above the writes (or the next block's writes above these reads).
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (lane < 16 * MT) {
                const f32x4 a = *(const f32x4*)(sm_t + lane * kTileMaxPitch), b = *(const f32x4*)(sm_t + lane * kTileMaxPitch + 4);
                const f32x4 c = *(const f32x4*)(sm_t + lane * kTileMaxPitch + 8), d = *(const f32x4*)(sm_t + lane * kTileMaxPitch + 12);
                const float m = fmaxf(fmaxf(fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])), fmaxf(fmaxf(b[0], b[1]), fmaxf(b[2], b[3]))),
                                      fmaxf(fmaxf(fmaxf(c[0], c[1]), fmaxf(c[2], c[3])), fmaxf(fmaxf(d[0], d[1]), fmaxf(d[2], d[3]))));
                if (lane < rows_here && span < end_span) p.tile_max[(size_t)(rowbase + lane) * p.tile_ld + span] = m;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }

    // rows at or beyond sum(group_sizes): zero product, bias of the last group (lax.ragged_dot semantics)
    float pad_bias8[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) pad_bias8[c] = (p.bias && p.ksplit == 1 && pad_from < p.M) ? p.bias[(size_t)g * p.N + ncol + c] : 0.f;
    for (int row0 = pad_from; row0 < p.M; row0 += 4) {
        float t[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) t[c] = 0.f;
        finish_row(p, t, pad_bias8, row0 + kb, ncol, out_col, ks, span_ok && row0 + kb < p.M, is_lin_lane);
        if (TMAX) store_tile_max(p, t, row0 + kb, span, span_ok, span < end_span && row0 + kb < p.M && x == 0);
    }
}

#if LYRA_GEMM_HAS_ENTRY
// Second pass when K was split across workgroups: sum the partials, then bias / SwiGLU / cast.
// One thread per 4 output columns.
__global__ __launch_bounds__(256) void decode_gemm_finish_kernel(GemmParams p) {
    const int NO = p.swiglu ? p.N / 2 : p.N;
    // grid (column quads / 256, rows): no division to find the row (a 64-bit one cost this 5 us launch ~100 instructions)
    const int col = (int)(blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (col >= NO) return;
    for (int row = blockIdx.y; row < p.M; row += gridDim.y) {
    // The slices are requested before the row's group is looked up (that is a chain of loads of its own, and the row exists
    // whatever its group): 4 slices in flight, added in slice order.
    float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < p.ksplit; s0 += 4) {
        f32x4 va[4], vb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j < p.ksplit) {
                const float* src = p.part + ((size_t)(s0 + j) * p.M + row) * p.N;
                va[j] = *(const f32x4*)(src + col);
                if (p.swiglu) vb[j] = *(const f32x4*)(src + NO + col);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j < p.ksplit) {
#pragma unroll
                for (int c = 0; c < 4; ++c) a[c] += va[j][c];
                if (p.swiglu) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) b[c] += vb[j][c];
                }
            }
        }
    }
    int total = 0, g = p.G - 1;
    for (int i = 0; i < p.G; ++i) {
        const int nt = total + p.group_sizes[i];
        if (row >= total && row < nt) g = i;
        total = nt;
    }
    if (row >= total) {  // rows past the last group: zero product (lax.ragged_dot), bias of the last group
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c] = b[c] = 0.f;
    }
    if (p.bias) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float bv = p.bias[(size_t)g * p.N + col + c];
            a[c] = p.bias_post ? round_bf16(round_bf16(a[c]) + bv) : a[c] + bv;
            if (p.swiglu) b[c] += p.bias[(size_t)g * p.N + NO + col + c];
        }
    }
    if (p.swiglu) {
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c] = swiglu_one(a[c], b[c], p.beta, p.limit);
    }
    if (p.post_scale) {
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c] = residual_epilogue(p, a[c], (size_t)row * NO + col + c);
    }
    if (p.out_f32) {
        out_store(p.out, ((size_t)row * NO + col) * 4, f32x4{a[0], a[1], a[2], a[3]});
    } else {
        u32x2 d;
        d[0] = pack_bf16(a[0], a[1]);
        d[1] = pack_bf16(a[2], a[3]);
        out_store(p.out, out_index(p, row, col, NO) * 2, d);
    }
    }
}
#endif  // LYRA_GEMM_HAS_ENTRY

// ---- small weight sets: one group, a few MB of weights (the dense projections of a decode layer) -----------------
// Such a product is bound by latency, not bandwidth: what counts is how many weight rows are in flight.  A workgroup
// owns one 16-row x 128-column output tile; its 8 wavefronts interleave over K in steps of 32 rows, each keeping
// DEPTH steps of weights and activations in flight (activations come straight from global memory, they are L2
// resident), and their partial tiles are summed through LDS in a fixed order.  No split over workgroups, no second
// pass, no workspace.  Rows at or beyond group_sizes[0] multiply zeros (epilogue(0), lax.ragged_dot semantics).
constexpr int kSmallWaves = 8;

template <int FP8, int DEPTH, bool STEP_SCALES, bool ONE_ROUND>
__global__ __launch_bounds__(kSmallWaves * 64) void decode_gemm_small_kernel(GemmParams p) {
    constexpr int ES = FP8 ? 1 : 2;
    extern __shared__ float sm_part[];  // [kSmallWaves][16][128]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = lane & 15, kb = lane >> 4;
    const int span = blockIdx.x, row0 = blockIdx.y * 16;

    int ncol;
    const bool is_lin_lane = p.swiglu && x >= 8;
    if (p.swiglu) ncol = (is_lin_lane ? (p.N >> 1) : 0) + span * 64 + 8 * (x & 7);
    else ncol = span * 128 + 8 * x;

    const int row_bytes = p.N * ES;
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.rhs), 0, (uint32_t)p.K * (uint32_t)row_bytes, 0x00020000);
    const int wvoff = 8 * kb * row_bytes + ncol * ES;

    // Everything the kernel reads is requested before anything is waited for, in the order it is consumed
    // (loads return in order): activations, weights, then what the epilogue needs.
    // Activations of this lane: row row0 + x, 8 consecutive k of k-group kb.  Whether the row belongs to the group
    // is only known once group_sizes[0] has arrived; the values are zeroed then, the loads do not wait for it.
    const int arow = row0 + x;
    const int asrc = arow < p.M ? (p.row_map ? p.row_map[arow] : arow) : 0;
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.lhs), 0, 0x7FFFFFFFu, 0x00020000);
    const int avoff = arow < p.M ? (asrc * p.K + 8 * kb) * 2 : kNoLoad;

    const int steps = p.K >> 5;
    const int n_my = (steps - wave + kSmallWaves - 1) / kSmallWaves;  // steps wave, wave + 8, ...
    const float* sc_lane = (FP8 && p.scale_mode == 1) ? p.scale + (ncol >> p.bn_shift) : nullptr;

    RawW<FP8> w[DEPTH];
    u32x4 a[DEPTH];
    [[maybe_unused]] float step_sc[DEPTH];  // STEP_SCALES: the scale of each step in flight travels with its weights
    const __amdgpu_buffer_rsrc_t scrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(STEP_SCALES ? p.scale : nullptr), 0, STEP_SCALES ? (uint32_t)p.KB * (uint32_t)p.NB * 4u : 0u, 0x00020000);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const bool live = d < n_my;
        const int kk = (wave + kSmallWaves * d) << 5;
        a[d] = __builtin_amdgcn_raw_buffer_load_b128(arsrc, live ? avoff : kNoLoad, __builtin_amdgcn_readfirstlane(live ? kk * 2 : 0), 0);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const bool live = d < n_my;
        const int kk = (wave + kSmallWaves * d) << 5;
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) load_w_pair_if<FP8>(live, w[d], pr, wrsrc, wvoff, kk, row_bytes);
        if constexpr (STEP_SCALES) step_sc[d] = load_step_scale(p, scrsrc, live, (ncol >> p.bn_shift) * 4, kk);
    }
    __builtin_amdgcn_sched_barrier(0);

    // epilogue inputs: the scales of this lane's 8 columns; bias and residual of the 4 outputs thread t finishes
    // (row t / 32 of the tile; 4 columns, or 2 gate + 2 linear columns with SwiGLU)
    float colscale[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) colscale[c] = 1.f;
    if (FP8 && p.scale_mode == 1 && !STEP_SCALES) {
        const float sc = *sc_lane;
#pragma unroll
        for (int c = 0; c < 8; ++c) colscale[c] = sc;
    } else if (FP8 && p.scale_mode == 2) {
#pragma unroll
        for (int c = 0; c < 8; ++c) colscale[c] = p.scale[(ncol + c) >> p.bn_shift];
    }
    const int er = threadIdx.x >> 5, eq = threadIdx.x & 31;
    const int erow = row0 + er;
    const bool e_ok = erow < p.M;
    const int NO = p.swiglu ? p.N >> 1 : p.N;
    const int oc = p.swiglu ? span * 64 + 2 * eq : span * 128 + 4 * eq;
    const size_t oidx = (size_t)erow * NO + oc;
    float ebias[4] = {0.f, 0.f, 0.f, 0.f}, eres[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
        if (p.swiglu) {
            ebias[0] = p.bias[oc]; ebias[1] = p.bias[oc + 1]; ebias[2] = p.bias[NO + oc]; ebias[3] = p.bias[NO + oc + 1];
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) ebias[c] = p.bias[oc + c];
        }
    }
    if (p.residual && e_ok) {
        if (p.swiglu) {
            const uint32_t d = *(const uint32_t*)(p.residual + oidx);
            eres[0] = __uint_as_float(d << 16); eres[1] = __uint_as_float(d & 0xFFFF0000u);
        } else {
            const u32x2 d = *(const u32x2*)(p.residual + oidx);
            eres[0] = __uint_as_float(d[0] << 16); eres[1] = __uint_as_float(d[0] & 0xFFFF0000u);
            eres[2] = __uint_as_float(d[1] << 16); eres[3] = __uint_as_float(d[1] & 0xFFFF0000u);
        }
    }
    const int cnt = min(p.group_sizes[0], p.M);
    const bool a_ok = arow < cnt;
    __builtin_amdgcn_sched_barrier(0);

    f32x4 acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    // every pass issues the same loads (past the end they fetch nothing) and multiplies zeros there
    for (int base = 0; base < (ONE_ROUND ? 1 : n_my); base += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int idx = base + d;
            const int kk = (wave + kSmallWaves * idx) << 5;
            const int kk_next = kk + ((kSmallWaves * DEPTH) << 5);
            const bool more = idx + DEPTH < n_my;
            Pack8 bop[8], av;
#pragma unroll
            for (int i = 0; i < 4; ++i) av.u[i] = a_ok ? a[d][i] : 0u;
            [[maybe_unused]] float sc = 1.f;
            if constexpr (STEP_SCALES) sc = step_sc[d];
            if constexpr (!ONE_ROUND) {
                __builtin_amdgcn_sched_barrier(0);
                a[d] = __builtin_amdgcn_raw_buffer_load_b128(arsrc, more ? avoff : kNoLoad,
                                                             __builtin_amdgcn_readfirstlane(more ? kk_next * 2 : 0), 0);
            }
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {
                convert_pair<FP8>(w[d], pr, bop);
                if constexpr (!ONE_ROUND) {
                    __builtin_amdgcn_sched_barrier(0);
                    load_w_pair_if<FP8>(more, w[d], pr, wrsrc, wvoff, kk_next, row_bytes);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if constexpr (STEP_SCALES && !ONE_ROUND) step_sc[d] = load_step_scale(p, scrsrc, more, (ncol >> p.bn_shift) * 4, kk_next);
            if constexpr (STEP_SCALES) {
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const f32x4 t = mfma_16x16x32(av.v, bop[c].v, f32x4{0.f, 0.f, 0.f, 0.f});
                    acc[c][0] += t[0] * sc;
                    acc[c][1] += t[1] * sc;
                    acc[c][2] += t[2] * sc;
                    acc[c][3] += t[3] * sc;
                }
            } else {
#pragma unroll
                for (int c = 0; c < 8; ++c) acc[c] = mfma_16x16x32(av.v, bop[c].v, acc[c]);
            }
            if constexpr (ONE_ROUND) __builtin_amdgcn_sched_barrier(0);
        }
    }

    float* mine = sm_part + wave * (16 * 128);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float* dst = mine + (4 * kb + r) * 128 + 8 * x;
        *(f32x4*)dst = f32x4{acc[0][r] * colscale[0], acc[1][r] * colscale[1], acc[2][r] * colscale[2], acc[3][r] * colscale[3]};
        *(f32x4*)(dst + 4) = f32x4{acc[4][r] * colscale[4], acc[5][r] * colscale[5], acc[6][r] * colscale[6], acc[7][r] * colscale[7]};
    }
    __syncthreads();

    // thread t finishes row t / 32 of the tile: 4 columns (2 gate + 2 linear columns with SwiGLU)
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.swiglu) {
#pragma unroll
        for (int wv = 0; wv < kSmallWaves; ++wv) {
            const float* src = sm_part + wv * (16 * 128) + er * 128 + 2 * eq;
            const f32x2 g2 = *(const f32x2*)src, l2 = *(const f32x2*)(src + 64);
            v[0] += g2[0]; v[1] += g2[1]; v[2] += l2[0]; v[3] += l2[1];
        }
    } else {
#pragma unroll
        for (int wv = 0; wv < kSmallWaves; ++wv) {
            const f32x4 t = *(const f32x4*)(sm_part + wv * (16 * 128) + er * 128 + 4 * eq);
            v[0] += t[0]; v[1] += t[1]; v[2] += t[2]; v[3] += t[3];
        }
    }
    if (!e_ok) return;
#pragma unroll
    for (int c = 0; c < 4; ++c) v[c] = p.bias_post ? round_bf16(round_bf16(v[c]) + ebias[c]) : v[c] + ebias[c];
    if (p.swiglu) {
        float o[2] = {swiglu_one(v[0], v[2], p.beta, p.limit), swiglu_one(v[1], v[3], p.beta, p.limit)};
        if (p.post_scale) {
            o[0] = round_bf16(round_bf16(o[0]) * p.out_scale) + eres[0];
            o[1] = round_bf16(round_bf16(o[1]) * p.out_scale) + eres[1];
        }
        if (p.out_f32) out_store(p.out, oidx * 4, f32x2{o[0], o[1]});
        else out_store(p.out, oidx * 2, pack_bf16(o[0], o[1]));
    } else {
        if (p.post_scale) {
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = round_bf16(round_bf16(v[c]) * p.out_scale) + eres[c];
        }
        if (p.out_f32) {
            out_store(p.out, oidx * 4, f32x4{v[0], v[1], v[2], v[3]});
        } else {
            u32x2 d;
            d[0] = pack_bf16(v[0], v[1]);
            d[1] = pack_bf16(v[2], v[3]);
            out_store(p.out, oidx * 2, d);
        }
    }
}

// ---- one group, a few MB of weights, up to a few dozen rows: split over K across all compute units ----------------
// A compute unit ingests only ~30-50 GB/s, so a dense projection (4-13 MB of weights) must be spread over all of
// them with as few bytes per unit as possible.  A workgroup owns 64 rows x 128 columns x one K slice: it reads 1/ks of
// one column span of the weights once and the matching slice of the activations once (about equal byte counts at 64
// rows).  Its 4 wavefronts interleave over the slice in steps of 32 rows with everything requested up front; their
// partial tiles are summed through LDS in a fixed order and the float32 result goes to slice ks of the partial
// buffer [ks, M, N].  Bias / SwiGLU / residual are applied by whoever sums the slices (the finish kernel, or the
// next kernel of the decode step when the caller defers the sum to it).
constexpr int kSplitWaves = 4;
constexpr int kSplitPitch = 132;  // floats per row of a partial tile in LDS (128 + padding against bank conflicts)

// STEP_SCALES: 0 scales constant along K (applied to the finished tile); 1 scale blocks shorter than K, every wavefront's
// rows within one block (its scale applied to its finished tile); 2 one scale per 32-row step.  With 1 and 2 a wavefront
// takes DEPTH consecutive steps instead of every 4th.
// LOOP: slices longer than 4 * DEPTH steps (larger matrices, cut less finely so that one round of workgroups covers them):
// the DEPTH register sets are refilled as they are used, wavefronts interleave, STEP_SCALES is 0 or 2.
// MT: 16-row tiles the instantiation holds (1, 2 or 4 = row blocks of 16, 32, 64 rows): a launch with smaller blocks runs
// less code - these launches are bound by the instructions one wavefront per SIMD gets through, not by arithmetic.
template <int FP8, int DEPTH, int STEP_SCALES, bool LOOP, int MT = 4>
__global__ __launch_bounds__(kSplitWaves * 64) void decode_gemm_splitk_kernel(GemmParams p) {
    constexpr int ES = FP8 ? 1 : 2;
    extern __shared__ float sm_part[];  // [kSplitWaves][64][kSplitPitch]
    // (the wavefront's index as a scalar: the K rows of its steps, and with them the row part of every load address, are
    // then computed once in the scalar unit instead of per lane and read back - these launches are bound by the
    // instructions a wavefront gets through)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = lane & 15, kb = lane >> 4;
    const int span = blockIdx.x, ks = blockIdx.y, row0 = blockIdx.z * p.row_block;
    const bool cols = span * 128 + 8 * x < p.N;    // (N need not fill the last span: lanes past it load nothing, store nothing)
    const int ncol = cols ? span * 128 + 8 * x : 0;
    const int k0 = ks * p.kpart, k1 = min(p.K, k0 + p.kpart);
    const int steps = (k1 - k0) >> 5;
    // steps wave, wave + 4, ... of the slice (<= DEPTH), or steps wave * DEPTH ... when scales change along K
    const int n_my = (STEP_SCALES && !LOOP) ? max(0, min(DEPTH, steps - wave * DEPTH)) : (steps - wave + kSplitWaves - 1) / kSplitWaves;
    auto step_row = [&](int d) { return k0 + (((STEP_SCALES && !LOOP) ? wave * DEPTH + d : wave + kSplitWaves * d) << 5); };

    // (span-major weights: this workgroup's span is a contiguous run of K rows of 128 weights)
    const int row_bytes = p.packed ? 128 * ES : p.N * ES;
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.rhs) + (p.packed ? (size_t)span * p.K * row_bytes : (size_t)0), 0, (uint32_t)p.K * (uint32_t)row_bytes,
        0x00020000);
    const int wvoff = cols ? 8 * kb * row_bytes + (p.packed ? 8 * x : ncol) * ES : kNoLoad;
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.lhs), 0, 0x7FFFFFFFu, 0x00020000);
    int avoff[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int arow = row0 + mt * 16 + x;
        const bool mine = arow < p.M && mt * 16 < p.row_block;
        const int asrc = mine ? (p.row_map ? p.row_map[arow] : arow) : 0;
        avoff[mt] = !mine ? kNoLoad : (p.lhs_tiled ? (asrc >> 4) * (p.K >> 5) * 1024 + (asrc & 15) * 64 + kb * 16 : (asrc * p.K + 8 * kb) * 2);
    }
    const int a_step = p.lhs_tiled ? 32 : 2;  // (activations in tiles of 16 rows x 32 columns: GemmParams::lhs_tiled)
    const int n_mt = min(min(p.row_block >> 4, MT), (p.M - row0 + 15) >> 4);  // 16-row tiles of this block that exist

    // all operands are requested before anything is waited for, in the order they are consumed: the activations (from the
    // caches) first.  Weights first - so that memory starts earlier - was measured twice: the first step's only (+1.8 % on
    // the decode step: the other steps' weights then start behind the address arithmetic of the activations) and all of
    // them (+2.1 %: loads return in the order they were requested, so nothing can be multiplied before the last weight
    // is there).
    u32x4 a[DEPTH][MT];
    RawW<FP8> w[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const bool live = d < n_my;
        const int kk = step_row(d);
        const int soff = __builtin_amdgcn_readfirstlane(live ? kk * a_step : 0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {  // (row tiles the block does not have are not requested: a load that fetches nothing
            if (mt < n_mt) a[d][mt] = __builtin_amdgcn_raw_buffer_load_b128(arsrc, live ? avoff[mt] : kNoLoad, soff, 0);  // still takes its turn)
            else a[d][mt] = u32x4{0u, 0u, 0u, 0u};
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const bool live = d < n_my;
        const int kk = step_row(d);
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) load_w_pair_if<FP8>(live, w[d], pr, wrsrc, wvoff, kk, row_bytes);
    }
    __builtin_amdgcn_sched_barrier(0);
    float colscale[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) colscale[c] = 1.f;
    const float* sc_lane = (FP8 && p.scale_mode == 1) ? p.scale + (ncol >> p.bn_shift) : nullptr;
    [[maybe_unused]] float step_sc[DEPTH];
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t scrsrc2 = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(FP8 ? p.scale : nullptr), 0, FP8 ? (uint32_t)p.KB * (uint32_t)p.NB * 4u : 0u, 0x00020000);
    if (FP8 && p.scale_mode == 1 && STEP_SCALES != 2) {
        const float sc = sc_lane[(size_t)(STEP_SCALES ? scale_block_of(p, step_row(0)) : 0) * p.NB];
#pragma unroll
        for (int c = 0; c < 8; ++c) colscale[c] = sc;
    } else if (FP8 && STEP_SCALES == 2) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) step_sc[d] = load_step_scale(p, scrsrc2, d < n_my, (ncol >> p.bn_shift) * 4, step_row(d));
    } else if (FP8 && p.scale_mode == 2) {
        if (p.bn_shift == 0 && ((uintptr_t)p.scale & 15) == 0) {  // one scale per column: the lane's 8 in two loads
            const f32x4 s0 = *(const f32x4*)(p.scale + ncol), s1 = *(const f32x4*)(p.scale + ncol + 4);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                colscale[c] = s0[c];
                colscale[4 + c] = s1[c];
            }
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) colscale[c] = p.scale[(ncol + c) >> p.bn_shift];
        }
    }
    const int cnt = min(p.group_sizes[0], p.M);  // rows at or beyond it multiply zeros (lax.ragged_dot)
    __builtin_amdgcn_sched_barrier(0);

    f32x4 acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[mt][c] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int base = 0; base < (LOOP ? n_my : 1); base += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int idx = base + d;
            Pack8 bop[8], av[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                // (zeroing the finished rows where the slice is written instead - 32 to 64 fewer instructions in this
                // loop - was measured 0.6 % slower on the decode step)
                const bool a_ok = row0 + mt * 16 + x < cnt;
#pragma unroll
                for (int i = 0; i < 4; ++i) av[mt].u[i] = a_ok ? a[d][mt][i] : 0u;
            }
            float sc = 1.f;
            if constexpr (STEP_SCALES == 2) sc = step_sc[d];
            if constexpr (LOOP) {
                // refill this register set with the step DEPTH further on (past the end: nothing is fetched)
                const bool more = idx + DEPTH < n_my;
                const int kk_next = step_row(idx + DEPTH);
                __builtin_amdgcn_sched_barrier(0);
                const int soff = __builtin_amdgcn_readfirstlane(more ? kk_next * a_step : 0);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    if (mt < n_mt) a[d][mt] = __builtin_amdgcn_raw_buffer_load_b128(arsrc, more ? avoff[mt] : kNoLoad, soff, 0);
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) {
                    convert_pair<FP8>(w[d], pr, bop);
                    __builtin_amdgcn_sched_barrier(0);
                    load_w_pair_if<FP8>(more, w[d], pr, wrsrc, wvoff, kk_next, row_bytes);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (STEP_SCALES == 2) step_sc[d] = load_step_scale(p, scrsrc2, more, (ncol >> p.bn_shift) * 4, kk_next);
            } else {
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) convert_pair<FP8>(w[d], pr, bop);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (mt < n_mt) {
                    if constexpr (STEP_SCALES == 2) {
#pragma unroll
                        for (int c = 0; c < 8; ++c) {
                            const f32x4 t = mfma_16x16x32(av[mt].v, bop[c].v, f32x4{0.f, 0.f, 0.f, 0.f});
                            acc[mt][c][0] += t[0] * sc;
                            acc[mt][c][1] += t[1] * sc;
                            acc[mt][c][2] += t[2] * sc;
                            acc[mt][c][3] += t[3] * sc;
                        }
                    } else {
#pragma unroll
                        for (int c = 0; c < 8; ++c) acc[mt][c] = mfma_16x16x32(av[mt].v, bop[c].v, acc[mt][c]);
                    }
                }
            }
            if constexpr (!LOOP) __builtin_amdgcn_sched_barrier(0);
        }
    }

    float* mine = sm_part + wave * (64 * kSplitPitch);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt < n_mt) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float* dst = mine + (mt * 16 + 4 * kb + r) * kSplitPitch + 8 * x;
                *(f32x4*)dst = f32x4{acc[mt][0][r] * colscale[0], acc[mt][1][r] * colscale[1], acc[mt][2][r] * colscale[2],
                                     acc[mt][3][r] * colscale[3]};
                *(f32x4*)(dst + 4) = f32x4{acc[mt][4][r] * colscale[4], acc[mt][5][r] * colscale[5], acc[mt][6][r] * colscale[6],
                                           acc[mt][7][r] * colscale[7]};
            }
        }
    }
    __syncthreads();
    // thread t sums 4 columns of rows t / 32, t / 32 + 8, ... over the wavefronts and writes the slice's partial
    const int q = threadIdx.x & 31;
    for (int r = threadIdx.x >> 5; r < 16 * n_mt; r += 8) {
        const int row = row0 + r;
        if (row >= p.M) break;
        f32x4 v = *(const f32x4*)(sm_part + r * kSplitPitch + 4 * q);
#pragma unroll
        for (int wv = 1; wv < kSplitWaves; ++wv) {
            const f32x4 t = *(const f32x4*)(sm_part + wv * (64 * kSplitPitch) + r * kSplitPitch + 4 * q);
            v[0] += t[0]; v[1] += t[1]; v[2] += t[2]; v[3] += t[3];
        }
        if (span * 128 + 4 * q < p.N) store_through(p.part, (((size_t)ks * p.M + row) * p.N + span * 128 + 4 * q) * 4, v);
    }
}

// Finishes 4 consecutive output columns of one row: vg holds the accumulated columns (the gate columns with SwiGLU, vl
// then holds the matching linear columns): bias, SwiGLU, residual epilogue, cast, store.  oc = first output column.
__device__ __forceinline__ void group_epilogue(const GemmParams& p, float (&vg)[4], float (&vl)[4], int g, int row, int oc, int NO) {
    const size_t oidx = (size_t)row * NO + oc;      // (residual: always row-major)
    const size_t sidx = out_index(p, row, oc, NO);  // where the result goes
    float o[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float a = vg[c];
        if (p.bias) a += p.bias[(size_t)g * p.N + oc + c];
        if (p.swiglu) {
            float l = vl[c];
            if (p.bias) l += p.bias[(size_t)g * p.N + NO + oc + c];
            a = swiglu_one(a, l, p.beta, p.limit);
        }
        if (p.post_scale) a = residual_epilogue(p, a, oidx + c);
        o[c] = a;
    }
    if (p.out_f32) {
        out_store(p.out, sidx * 4, f32x4{o[0], o[1], o[2], o[3]});
    } else {
        u32x2 d;
        d[0] = pack_bf16(o[0], o[1]);
        d[1] = pack_bf16(o[2], o[3]);
        out_store(p.out, sidx * 2, d);
    }
}

__device__ __forceinline__ f32x4 load_f32x4(__amdgpu_buffer_rsrc_t rsrc, int voff) {
    const u32x4 d = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 0, 0);
    return f32x4{__uint_as_float(d[0]), __uint_as_float(d[1]), __uint_as_float(d[2]), __uint_as_float(d[3])};
}
// 4 consecutive bf16 values as float32
__device__ __forceinline__ f32x4 load_bf16x4(__amdgpu_buffer_rsrc_t rsrc, int voff) {
    const u32x2 d = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, 0, 0);
    return f32x4{__uint_as_float(d[0] << 16), __uint_as_float(d[0] & 0xFFFF0000u), __uint_as_float(d[1] << 16),
                 __uint_as_float(d[1] & 0xFFFF0000u)};
}

// Finishes 4 consecutive output columns of one row of a unit, all operands in registers: v the accumulated columns (gate
// columns with SwiGLU, then l the matching linear columns), their biases (zeros when there are none), res the 4 residual
// values.  The same arithmetic, in the same order, as group_epilogue.
__device__ __forceinline__ void finish4(const GemmParams& p, f32x4 v, f32x4 l, f32x4 bias_v, f32x4 bias_l, f32x4 res, size_t oidx) {
    float o[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float a = v[c] + bias_v[c];
        if (p.swiglu) a = swiglu_one(a, l[c] + bias_l[c], p.beta, p.limit);
        if (p.post_scale) a = round_bf16(round_bf16(a) * p.out_scale) + res[c];
        o[c] = a;
    }
    if (p.out_f32) {
        out_store(p.out, oidx * 4, f32x4{o[0], o[1], o[2], o[3]});
    } else {
        u32x2 d;
        d[0] = pack_bf16(o[0], o[1]);
        d[1] = pack_bf16(o[2], o[3]);
        out_store(p.out, oidx * 2, d);
    }
}

// ---- several groups (MoE experts), a handful of rows each: workgroups walk a list of (row block, column span) units -----
// A unit is up to 64 rows of one expert times one 128-column span over the whole K extent (256-1024 KB of weights).
// Every workgroup first builds the same unit list in LDS from group_sizes (experts without rows contribute nothing, so
// their weights are never read; the units with the most rows, which cost the most, come first) and then takes one unit
// of every round of gridDim.x units: at any time the workgroups stream neighbouring column spans of the same weight
// rows, which is what keeps the DRAM pages they touch open (handing every workgroup a run of consecutive units
// instead, so that shares could be cut to equal cost, was built and was 6-40 % slower for that reason).  The units left
// over after the last full round go to the workgroups that had the lightest units in the first.  Within a unit its 4 wavefronts interleave over K in steps of 32 rows with DEPTH steps of weights and
// activations in flight each; their partial tiles are summed through LDS in a fixed order and bias / SwiGLU / residual
// follow.  The first operands of the next unit are requested before the current unit's tile is summed and written, so a
// compute unit keeps streaming across unit boundaries.
// The units left over after the last full round of gridDim.x (all of them when there are fewer) would keep only some of
// the compute units busy - and a compute unit ingests ~30 GB/s whatever the others do - so each of them is cut into S
// slices along K, S as large as keeps tail * S <= gridDim.x, taken slice by slice in the same order.  A slice's tile goes to
// a float32 slot in the workspace (device-wide visible stores) and bumps the unit's arrival counter; the workgroup that
// arrives last adds the S slots in K order - so the result does not depend on who that is - and finishes the tile.
// Nobody waits for anybody, and results do not depend on timing.
// With SwiGLU a span is 128 gate columns (wavefronts 0, 1, interleaved over K) plus the matching 128 linear columns
// (wavefronts 2, 3), so every load covers whole 128-byte lines of a weight row; 64 + 64 columns per wavefront would fetch
// twice as many lines per byte.  ROUNDS passes over the DEPTH register sets are unrolled per trip of the K loop: in
// straight-line code every wait counts exactly the loads issued after the one it needs, whereas the wait at the head of a
// loop drains nearly everything in flight.
constexpr int kGroupTiles = 4;      // 16-row tiles a unit accumulates (64 rows)
constexpr int kMaxStreamGroups = 256;
constexpr int kMaxRowBlocks = 512;  // row blocks the LDS table holds
constexpr int kGroupMaxWgs = 256;   // shares (workgroups) of a launch; also the number of arrival counters in use
constexpr size_t kGemmCounterBytes = 65536;  // start of a matmul workspace: arrival counters, zero between launches

// Exclusive prefix sum of one int per thread over the 256 threads of a workgroup (sm4: 4 ints of LDS, free on entry).
__device__ __forceinline__ int wg_scan_exclusive(int v, int* sm4, int lane, int wave, int& total) {
    const int incl = wave_scan_inclusive(v);
    if (lane == 63) sm4[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int wv = 0; wv < wave; ++wv) base += sm4[wv];
    total = sm4[0] + sm4[1] + sm4[2] + sm4[3];
    return base + incl - v;
}

// The same over four 16-bit counts packed into 64 bits (no field may exceed 65535 in total).
__device__ __forceinline__ unsigned long long wg_scan_exclusive4(unsigned long long v, unsigned long long* sm4, int lane, int wave,
                                                                 unsigned long long& total) {
    // (no field of the low or of the high word overflows into the other word, so the two words are summed on their own)
    const unsigned long long incl = (unsigned long long)(unsigned)wave_scan_inclusive((int)(unsigned)v) |
                                    ((unsigned long long)(unsigned)wave_scan_inclusive((int)(unsigned)(v >> 32)) << 32);
    if (lane == 63) sm4[wave] = incl;
    __syncthreads();
    unsigned long long base = 0;
    for (int wv = 0; wv < wave; ++wv) base += sm4[wv];
    total = sm4[0] + sm4[1] + sm4[2] + sm4[3];
    return base + incl - v;
}

// WIDE_DYN: an instantiation for launches without SwiGLU that may have enough units for the wider ones (decided below,
// once the unit list is known; the other instantiations know their layout from the start).
// PACKED: the weights are span-major (GemmParams::packed): every unit streams one or two contiguous runs of K rows of 128
// weights.  With SwiGLU a span then holds 64 gate columns and their 64 linear columns, so a unit of one span is half as
// wide as without the copy and a launch has twice the units to deal out; whether wavefront pairs take two spans (as many
// rounds as before) or all four wavefronts one span (short lists: finer shares) is decided once the unit list is known.
template <int FP8, bool STEP_SCALES, int ROUNDS, bool SLICED, bool WIDE_DYN = false, bool PACKED = false>
__global__ __launch_bounds__(kSplitWaves * 64) void decode_gemm_group_kernel(GemmParams p) {
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int DEPTH = FP8 ? 4 : 2;
    constexpr int MTM = kGroupTiles;
    constexpr int TRIP = ROUNDS * DEPTH;  // steps of one wavefront per trip
    extern __shared__ float sm_part[];  // [kSplitWaves][16 * MTM][kSplitPitch]
    __shared__ int sm_blk[kMaxRowBlocks][3];  // (group, first row, rows) of every row block, heavy groups first
    __shared__ int sm_scan[8];
    __shared__ unsigned long long sm_scan4[4];
    __shared__ int sm_last;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = lane & 15, kb = lane >> 4;

    // wide: a unit is two sets of 128 columns, each taken by a pair of wavefronts that interleave over K (gate and linear
    // columns with SwiGLU, else two adjacent spans: 256 contiguous bytes of every weight row per workgroup instead of 128,
    // which streams ~14 % faster); otherwise one set of 128 columns and all 4 wavefronts interleave.
    const int NO = p.swiglu ? p.N >> 1 : p.N;
    const int q = threadIdx.x & 31;
    const int row_bytes = PACKED ? 128 * ES : p.N * ES;
    const int steps = p.K >> 5;
    const int half_stride = p.swiglu ? (p.N >> 1) : 128;
    const int a_step = p.lhs_tiled ? 32 : 2;  // bytes from the activations of K row k to those of k + 1 ... (a step is 32 rows of K)
    bool wide;
    int spans, kw, wslot, half, span_cols, tile_cols, n_my, trips;
    auto set_layout = [&](bool w) {
        wide = w;
        if constexpr (PACKED) spans = w ? (p.pspans + 1) >> 1 : p.pspans;
        else spans = p.swiglu ? ((p.N >> 1) + 127) / 128 : (w ? p.N / 256 : (p.N + 127) / 128);  // (the last span may be partly filled)
        kw = w ? 2 : kSplitWaves;
        wslot = w ? (wave & 1) : wave, half = w ? (wave >> 1) : 0;
        span_cols = PACKED ? (p.swiglu ? (w ? 128 : 64) : (w ? 256 : 128)) : (p.swiglu || !w ? 128 : 256);  // output columns of a unit
        tile_cols = w ? 256 : 128;                                  // floats per row of a workspace slot
        n_my = (steps - wslot + kw - 1) / kw;                       // steps of this wavefront in a whole unit
        trips = ((steps + kw - 1) / kw + TRIP - 1) / TRIP;          // trips of a whole unit (same for every wavefront)
    };
    if constexpr (!WIDE_DYN) set_layout(PACKED ? false : (p.swiglu || p.wide));

    // ---- unit list: thread t looks at group G-1-t ----
    const int t = threadIdx.x;
    [[maybe_unused]] uint32_t touched[2] = {0u, 0u};  // (what the touch below reads: looked at once, at the very end)
    int my_cnt = 0, my_before = 0;  // rows of "my" group and rows of all groups before it (in lhs order)
    int total_rows;
    {
        const int v = t < p.G ? p.group_sizes[t] : 0;
        // The list starts with the row blocks of the last group, which is where a model keeps its shared expert: every
        // token has a row there, so the units with the most rows - the ones that decide how long the launch lasts - are
        // known before the group sizes are.  The workgroups that own them if that holds touch the lines of their first
        // DEPTH steps now (one lane per 128-byte line, behind the request for the group sizes so that nothing waits for
        // them): the real requests, two round trips later, then meet them in L2.  Where it does not hold, a few
        // workgroups have fetched 64 KB each for nothing.
        if constexpr (!WIDE_DYN && !PACKED) {
            const int blk0 = (int)blockIdx.x / spans, span0 = (int)blockIdx.x - blk0 * spans;
            const bool guess = p.touch_last && blk0 * (16 * MTM) < p.M;
            const __amdgpu_buffer_rsrc_t trsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint8_t*>(p.rhs) + (size_t)(p.G - 1) * p.K * row_bytes, 0, (uint32_t)p.K * (uint32_t)row_bytes, 0x00020000);
            const int col0 = (half * half_stride + span0 * span_cols) * ES;  // first byte of this wavefront's columns in a row
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int line = lane + 64 * j;                  // 128 lines: DEPTH steps x 32 rows x ES lines
                const int rowi = line / ES, sub = line - rowi * ES;
                const int idx = rowi >> 5, r = rowi & 31;
                const int off = ((wslot + kw * idx) * 32 + r) * row_bytes + col0 + 128 * sub;
                touched[j] = __builtin_amdgcn_raw_buffer_load_b32(trsrc, guess && idx < n_my ? off : kNoLoad, 0, 0);
            }
        }
        const int before = wg_scan_exclusive(v, sm_scan, lane, wave, total_rows);
        // hand (before, size) of natural group t to the thread that owns it in heavy-first order: thread G-1-t
        int* tmp = (int*)sm_part;  // scratch before the tiles are used
        if (t < p.G) {
            tmp[2 * (p.G - 1 - t)] = min(before, p.M);
            tmp[2 * (p.G - 1 - t) + 1] = max(0, min(v, p.M - min(before, p.M)));
        }
        __syncthreads();
        if (t < p.G) {
            my_before = tmp[2 * t];
            my_cnt = tmp[2 * t + 1];
        }
    }
    const int my_blocks = (my_cnt + 16 * MTM - 1) / (16 * MTM);
    int n_blocks_all;
    const int blk_base = wg_scan_exclusive(my_blocks, sm_scan + 4, lane, wave, n_blocks_all);
    const int n_blocks = min(kMaxRowBlocks, n_blocks_all);  // (the host keeps n_blocks_all <= kMaxRowBlocks)
    for (int i = 0; i < my_blocks; ++i) {
        const int j = blk_base + i;
        if (j < kMaxRowBlocks) {
            sm_blk[j][0] = p.G - 1 - t;
            sm_blk[j][1] = my_before + i * 16 * MTM;
            sm_blk[j][2] = min(16 * MTM, my_cnt - i * 16 * MTM);
        }
    }
    if (n_blocks_all * (PACKED ? p.pspans : (p.N >> 8)) > (int)gridDim.x) {
        // More than one round of units: the list is put in the order of cost, in four classes by the number of 16-row
        // tiles a block fills - all blocks of 49-64 rows (in group order from the last group down), then those of 33-48,
        // 17-32 and 1-16 rows - so that, whatever the order of the groups, the units at the end of the list are the light
        // ones.  One prefix sum over the four counts, packed into 64 bits, places every block.  (A single round gains
        // nothing from the order, and the second prefix sum would cost it 0.8 us.)
        const int my_full = my_cnt / (16 * MTM), my_rem = my_cnt - my_full * (16 * MTM);
        const int my_class = my_rem > 0 ? MTM - ((my_rem + 15) >> 4) : 0;  // class of the partly filled block
        unsigned long long all4;
        const unsigned long long before4 = wg_scan_exclusive4(
            (unsigned long long)my_full + (my_rem > 0 ? 1ull << (16 * my_class) : 0ull), sm_scan4, lane, wave, all4);
        int class_base = 0;  // blocks of the classes before my_class
        for (int c = 0; c < my_class; ++c) class_base += (int)((all4 >> (16 * c)) & 0xFFFF);
        const int full_base = (int)(before4 & 0xFFFF);
        const int rem_at = class_base + (int)((before4 >> (16 * my_class)) & 0xFFFF) + (my_class == 0 ? my_full : 0);
        for (int i = 0; i < my_blocks; ++i) {  // (after the barrier in the prefix sum: every block is written again, elsewhere)
            const int j = i < my_full ? full_base + i : rem_at;
            if (j < kMaxRowBlocks) {
                sm_blk[j][0] = p.G - 1 - t;
                sm_blk[j][1] = my_before + i * 16 * MTM;
                sm_blk[j][2] = min(16 * MTM, my_cnt - i * 16 * MTM);
            }
        }
    }
    __syncthreads();
    const int nwg = gridDim.x;
    // Without SwiGLU the wider units are taken when they still fill 1.75 rounds of workgroups (lyra-max down projection at
    // batch 128: -8 %); with fewer, their coarser rounds cost more than the access pattern gains.
    if constexpr (WIDE_DYN) {
        if constexpr (PACKED) set_layout(p.wide || 4 * n_blocks * ((p.pspans + 1) >> 1) >= 7 * nwg);
        else set_layout(p.swiglu || p.wide || 4 * n_blocks * (p.N / 256) >= 7 * nwg);
    }
    const int n_units = __builtin_amdgcn_readfirstlane(n_blocks * spans);  // (same in every lane: tell the compiler)
    // whole units in full rounds of nwg; when there is not even one full round, the units are cut into `slices` K slices each
    // (a power of two that divides trips).  After a full round slicing the rest was measured to cost as much as it saves:
    // the few workgroups of a last partial round stream faster, having the memory system to themselves.
    const int n_whole = n_units / nwg * nwg, tail = n_units - n_whole;
    int slices = 1;
    while (SLICED && tail > 0 && n_whole == 0 && 2 * slices * tail <= nwg && trips % (2 * slices) == 0 && 2 * slices <= p.max_slices) slices *= 2;
    const int trips_per_slice = trips / slices;
    const int n_work = n_whole + tail * slices;  // work items: unit v for v < n_whole, else slice (v - n_whole) / tail of a tail unit
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.lhs), 0, 0x7FFFFFFFu, 0x00020000);

    // state of the work item whose operands are in flight / being consumed
    int v = blockIdx.x, round = 0;  // (v = round * nwg + blockIdx.x)
    bool seg_valid = false;
    int seg_u = 0, seg_r0 = 0, seg_r1 = 0;  // its unit and trips [r0, r1) of it
    int g = 0, row0 = 0, rows = 0, span = 0, ncol = 0, wvoff = kNoLoad, avoff[MTM];
    bool seg_cols = false;  // the lane's columns exist (scales of absent columns are not read)
    __amdgpu_buffer_rsrc_t wrsrc;
    constexpr int ADEPTH = 2;  // activation steps in flight (they come from the caches; the weights, from memory, need DEPTH)
    u32x4 a[ADEPTH][MTM];
    RawW<FP8> w[DEPTH];
    [[maybe_unused]] float step_sc[DEPTH];  // STEP_SCALES: the scale of each step in flight travels with its weights
    [[maybe_unused]] int sc_voff = kNoLoad;
    const __amdgpu_buffer_rsrc_t scrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(FP8 ? p.scale : nullptr), 0, FP8 ? (uint32_t)p.G * (uint32_t)p.KB * (uint32_t)p.NB * 4u : 0u, 0x00020000);

    // Looks work item vv up and requests its first DEPTH steps (an item past the end requests nothing).
    // After full rounds, the left-over units go to the workgroups at the far end: the heavy units come first in the list, so
    // the workgroups at the near end have had the most to do in the first round (lyra-medium expert matmuls at 64 tokens:
    // -10 %).  With four or more full rounds, odd rounds also run over the workgroups in the opposite direction, which evens
    // out what is left of that slope (lyra-max up projection at 128 tokens: -5 %; with two rounds it costs 4 %).
    const bool snake = p.snake < 0 ? n_whole >= 4 * (int)nwg : p.snake != 0;
    auto open_segment = [&](int vv) {
        bool valid = vv < n_work;
        if (n_whole > 0 && vv >= n_whole) {
            const int rev = (int)nwg - 1 - (vv - n_whole);
            valid = rev >= 0 && rev < tail;
            vv = n_whole + rev;
        } else if (snake && vv < n_whole && (round & 1)) {
            vv = vv - (int)blockIdx.x + ((int)nwg - 1 - (int)blockIdx.x);  // odd rounds run the other way
        }
        seg_valid = valid;
        if constexpr (SLICED) {
            const int ti = vv - n_whole;  // >= 0: slice ti / tail of tail unit ti % tail
            const int sl = (valid && ti >= 0) ? ti / tail : 0;
            seg_u = __builtin_amdgcn_readfirstlane(!valid ? 0 : (ti >= 0 ? n_whole + (ti - sl * tail) : vv));
            seg_r0 = __builtin_amdgcn_readfirstlane((valid && ti >= 0) ? sl * trips_per_slice : 0);
            seg_r1 = __builtin_amdgcn_readfirstlane(!valid ? 0 : (ti >= 0 ? seg_r0 + trips_per_slice : trips));
        } else {
            seg_u = valid ? vv : 0;
            seg_r0 = 0;
            seg_r1 = valid ? trips : 0;
        }
        const int blk = seg_u / spans;
        span = seg_u - blk * spans;
        g = __builtin_amdgcn_readfirstlane(valid ? sm_blk[blk][0] : 0);
        row0 = __builtin_amdgcn_readfirstlane(valid ? sm_blk[blk][1] : 0);
        rows = __builtin_amdgcn_readfirstlane(valid ? sm_blk[blk][2] : 0);
        bool cols;
        if constexpr (PACKED) {
            // this wavefront's span of the packed copy: K rows of 128 weights, contiguous.  ncol is the column (of the
            // reference's array) that the lane's first weight belongs to: scales and biases keep that order.
            const int ps = wide ? 2 * span + half : span;
            const bool ps_ok = ps < p.pspans;
            if (p.swiglu) {
                ncol = (x < 8 ? 0 : (p.N >> 1)) + 64 * ps + 8 * (x & 7);
                cols = ps_ok && 64 * ps + 8 * (x & 7) < NO;
            } else {
                ncol = 128 * ps + 8 * x;
                cols = ps_ok && ncol < NO;
            }
            wrsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint8_t*>(p.rhs) + ((size_t)g * p.pspans + (ps_ok ? ps : 0)) * p.K * row_bytes, 0,
                (uint32_t)p.K * (uint32_t)row_bytes, 0x00020000);
            wvoff = valid && ps_ok ? 8 * kb * row_bytes + 8 * x * ES : kNoLoad;  // (columns N does not have hold zeros)
        } else {
            ncol = half * half_stride + span * span_cols + 8 * x;
            // (N need not fill the last span: lanes past the last column - of the gate or linear half with SwiGLU - load
            // nothing, accumulate zeros and are left out of the epilogue)
            cols = span * span_cols + (wide && !p.swiglu ? 128 * half : 0) + 8 * x < NO;
            wrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.rhs) + (size_t)g * p.K * row_bytes, 0,
                                                      (uint32_t)p.K * (uint32_t)row_bytes, 0x00020000);
            wvoff = valid && cols ? 8 * kb * row_bytes + ncol * ES : kNoLoad;
        }
        seg_cols = cols;
        if constexpr (STEP_SCALES) sc_voff = valid && cols ? (g * p.KB * p.NB + (ncol >> p.bn_shift)) * 4 : kNoLoad;
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt) {
            const int r = mt * 16 + x;
            int src = row0 + min(r, max(rows - 1, 0));
            if (p.row_map) src = p.row_map[src];
            avoff[mt] = r >= rows ? kNoLoad
                                  : (p.lhs_tiled ? (src >> 4) * (p.K >> 5) * 1024 + (src & 15) * 64 + kb * 16 : (src * p.K + 8 * kb) * 2);
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int idx = seg_r0 * TRIP + d;
            const bool live = valid && idx < n_my;
            const int kk = (wslot + kw * idx) << 5;
            const int soff = __builtin_amdgcn_readfirstlane(live ? kk * a_step : 0);
            if (d < ADEPTH) {
#pragma unroll
                for (int mt = 0; mt < MTM; ++mt)
                    if (mt * 16 < rows) a[d % ADEPTH][mt] = __builtin_amdgcn_raw_buffer_load_b128(arsrc, live ? avoff[mt] : kNoLoad, soff, 0);
            }
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) load_w_pair_if<FP8>(live, w[d], pr, wrsrc, wvoff, kk, row_bytes);
            if constexpr (STEP_SCALES) step_sc[d] = load_step_scale(p, scrsrc, live, sc_voff, kk);
        }
    };

    // bias [G, N] float32 and residual [M, NO] bf16 through descriptors, so that an absent operand reads as zeros
    const __amdgpu_buffer_rsrc_t bias_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(p.bias), 0, p.bias ? (uint32_t)p.G * (uint32_t)p.N * 4u : 0u, 0x00020000);
    const __amdgpu_buffer_rsrc_t res_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.residual), 0, p.residual ? (uint32_t)p.M * (uint32_t)NO * 2u : 0u, 0x00020000);
    // workspace slots: [tail unit][K slice][64 rows][tile_cols] float32, at most kGroupMaxWgs of them
    const __amdgpu_buffer_rsrc_t slot_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        p.part, 0, (uint32_t)(kGroupMaxWgs * 16 * MTM) * (uint32_t)tile_cols * 4u, 0x00020000);

    open_segment(v);
    while (seg_valid) {
        const int cur_u = seg_u, r0 = seg_r0, r1 = seg_r1;
        const int cur_g = g, cur_row0 = row0, cur_rows = rows, cur_span = span, cur_ncol = ncol;
        const bool cur_cols = seg_cols;
        const int n_mt = (cur_rows + 15) >> 4;
        const __amdgpu_buffer_rsrc_t cur_wrsrc = wrsrc;
        const int cur_wvoff = wvoff;
        [[maybe_unused]] const int cur_sc_voff = sc_voff;
        int cur_avoff[MTM];
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt) cur_avoff[mt] = avoff[mt];
        f32x4 acc[MTM][8];
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt)
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[mt][c] = f32x4{0.f, 0.f, 0.f, 0.f};

        // every pass issues the same loads (past the end of the segment they fetch nothing) and multiplies zeros there
        const int idx_end = min(n_my, r1 * TRIP);
        // The steps of a wavefront form a software pipeline: while the matrix cores multiply step s, the vector ALU turns the
        // raw weights of step s+1 into operands, two column phases at a time - the 2 * NMT matrix instructions that consume
        // the current operands of phases 2cp, 2cp+1 are interleaved with the 16 conversions that produce their successors,
        // which then take their place.  A unit of many rows (32 matrix instructions per step) thus hides its conversions
        // behind them instead of doing one after the other.  The loop is instantiated per number of 16-row tiles so that a
        // step is straight-line code the scheduler can interleave.
        Pack8 bop[8];
        auto k_loop = [&](auto nmt_c) {
            constexpr int NMT = decltype(nmt_c)::value;
            {  // operands of the item's first step; its register set is then refilled with step DEPTH
                const int idx0 = r0 * TRIP;
                const bool more = idx0 + DEPTH < idx_end;
                const int kk_next = (wslot + kw * (idx0 + DEPTH)) << 5;
#pragma unroll
                for (int cp = 0; cp < 4; ++cp) {
                    if constexpr (STEP_SCALES) convert_colpair<FP8, true>(w[0], cp, bop[2 * cp], bop[2 * cp + 1], step_sc[0]);
                    else convert_colpair<FP8>(w[0], cp, bop[2 * cp], bop[2 * cp + 1]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) load_w_pair_if<FP8>(more, w[0], pr, cur_wrsrc, cur_wvoff, kk_next, row_bytes);
                if constexpr (STEP_SCALES) step_sc[0] = load_step_scale(p, scrsrc, more, cur_sc_voff, kk_next);
                __builtin_amdgcn_sched_barrier(0);
            }
            for (int trip = r0; trip < r1; ++trip) {
#pragma unroll
                for (int ur = 0; ur < ROUNDS; ++ur) {
#pragma unroll
                    for (int d = 0; d < DEPTH; ++d) {
                        const int dn = (d + 1) % DEPTH;
                        const int idx = (trip * ROUNDS + ur) * DEPTH + d;
                        const int kk = (wslot + kw * idx) << 5;
                        const int kk_w = kk + ((kw * (DEPTH + 1)) << 5);      // the next step of the following weight register set
                        const int kk_act = kk + ((kw * ADEPTH) << 5);         // the next step of this step's activation registers
                        const int ad = (ur * DEPTH + d) % ADEPTH;
                        const bool more_w = idx + 1 + DEPTH < idx_end, more_act = idx + ADEPTH < idx_end;
                        bf16x8 av[NMT];
#pragma unroll
                        for (int mt = 0; mt < NMT; ++mt) av[mt] = __builtin_bit_cast(bf16x8, a[ad][mt]);
#pragma unroll
                        for (int cp = 0; cp < 4; ++cp) {
                            __builtin_amdgcn_sched_barrier(0);
                            Pack8 n0, n1;
                            if constexpr (STEP_SCALES) convert_colpair<FP8, true>(w[dn], cp, n0, n1, step_sc[dn]);
                            else convert_colpair<FP8>(w[dn], cp, n0, n1);
#pragma unroll
                            for (int mt = 0; mt < NMT; ++mt) {
                                acc[mt][2 * cp] = mfma_16x16x32(av[mt], bop[2 * cp].v, acc[mt][2 * cp]);
                                acc[mt][2 * cp + 1] = mfma_16x16x32(av[mt], bop[2 * cp + 1].v, acc[mt][2 * cp + 1]);
                            }
                            // 2 * NMT matrix instructions, 16 (FP8) or 8 (bf16) vector instructions: spread evenly
                            constexpr int kVecOps = FP8 ? (STEP_SCALES ? 32 : 16) : 8, kPer = (kVecOps + 2 * NMT - 1) / (2 * NMT);
#pragma unroll
                            for (int j = 0; j < 2 * NMT; ++j) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                                __builtin_amdgcn_sched_group_barrier(0x002, kPer, 0);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                            bop[2 * cp] = n0;
                            bop[2 * cp + 1] = n1;
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        // the registers just consumed are requested again: the activations for step idx + ADEPTH, the converted
                        // weight rows for step idx + 1 + DEPTH
                        const int soff_act = __builtin_amdgcn_readfirstlane(more_act ? kk_act * a_step : 0);
#pragma unroll
                        for (int mt = 0; mt < NMT; ++mt)  // (only the row tiles the unit has)
                            a[ad][mt] = __builtin_amdgcn_raw_buffer_load_b128(arsrc, more_act ? cur_avoff[mt] : kNoLoad, soff_act, 0);
#pragma unroll
                        for (int pr = 0; pr < 4; ++pr) load_w_pair_if<FP8>(more_w, w[dn], pr, cur_wrsrc, cur_wvoff, kk_w, row_bytes);
                        if constexpr (STEP_SCALES) step_sc[dn] = load_step_scale(p, scrsrc, more_w, cur_sc_voff, kk_w);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };
        switch (n_mt) {
            case 1: k_loop(std::integral_constant<int, 1>{}); break;
            case 2: k_loop(std::integral_constant<int, 2>{}); break;
            case 3: k_loop(std::integral_constant<int, 3>{}); break;
            default: k_loop(std::integral_constant<int, 4>{}); break;
        }

        // Scales that are constant along K are applied to the finished tile.  They are requested here, ahead of the next
        // item's operands (loads return in order), and arrive while those are being requested.
        float colscale[8];
        if (FP8 && p.scale_mode == 2 && p.bn_shift == 0) {  // one scale per column: the lane's 8 in two requests
            const int off = (!PACKED || cur_cols) ? (cur_g * p.NB + cur_ncol) * 4 : kNoLoad;
            const u32x4 s0 = __builtin_amdgcn_raw_buffer_load_b128(scrsrc, off, 0, 0);
            const u32x4 s1 = __builtin_amdgcn_raw_buffer_load_b128(scrsrc, off, 16, 0);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                colscale[c] = __uint_as_float(s0[c]);
                colscale[4 + c] = __uint_as_float(s1[c]);
            }
        } else
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            colscale[c] = 1.f;  // (scale blocks along K were applied to the weights)
            if (FP8 && p.scale_mode == 1 && !STEP_SCALES) {
                const int off = (!PACKED || cur_cols) ? (cur_g * p.KB * p.NB + (cur_ncol >> p.bn_shift)) * 4 : kNoLoad;
                if (c == 0) colscale[0] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(scrsrc, off, 0, 0));
                else colscale[c] = colscale[0];
            } else if (FP8 && p.scale_mode == 2) {
                const int off = (!PACKED || cur_cols) ? (cur_g * p.NB + ((cur_ncol + c) >> p.bn_shift)) * 4 : kNoLoad;
                colscale[c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(scrsrc, off, 0, 0));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // the next item's first operands fly while this tile is summed and written
        v += nwg;
        ++round;
        open_segment(v);

        float* mine = sm_part + wave * (16 * MTM * kSplitPitch);
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt) {
            if (mt < n_mt) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float* dst = mine + (mt * 16 + 4 * kb + r) * kSplitPitch + 8 * x;
                    *(f32x4*)dst = f32x4{acc[mt][0][r] * colscale[0], acc[mt][1][r] * colscale[1], acc[mt][2][r] * colscale[2],
                                         acc[mt][3][r] * colscale[3]};
                    *(f32x4*)(dst + 4) = f32x4{acc[mt][4][r] * colscale[4], acc[mt][5][r] * colscale[5],
                                               acc[mt][6][r] * colscale[6], acc[mt][7][r] * colscale[7]};
                }
            }
        }
        lds_barrier();  // (the next item's operands stay in flight)
        constexpr int TS = 16 * MTM * kSplitPitch;  // floats per wavefront tile
        // Sum of the wavefront tiles for 4 columns of row r: vg (and vl, the second set of 128 columns of a wide unit).
        auto tile_row = [&](int r, float (&vg)[4], float (&vl)[4]) {
            const float* src = sm_part + r * kSplitPitch + 4 * q;
            const f32x4 t0 = *(const f32x4*)src, t1 = *(const f32x4*)(src + TS), t2 = *(const f32x4*)(src + 2 * TS),
                        t3 = *(const f32x4*)(src + 3 * TS);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (wide) {
                    vg[c] = t0[c] + t1[c];
                    vl[c] = t2[c] + t3[c];
                } else {
                    vg[c] = ((t0[c] + t1[c]) + t2[c]) + t3[c];
                    vl[c] = 0.f;
                }
            }
        };
        bool finish = !SLICED || (r0 == 0 && r1 == trips);  // the whole unit was summed here
        if (SLICED && !finish) {
            // a K slice of a unit: publish the tile, count the arrival; whoever arrives last adds all slices in K order
            const int ui = cur_u - n_whole;                          // tail unit
            const int my_slot = ui * slices + r0 / trips_per_slice;  // slots of a unit are consecutive, in K order
            for (int r = threadIdx.x >> 5; r < cur_rows; r += 8) {
                float vg[4], vl[4];
                tile_row(r, vg, vl);
                const int off = ((my_slot * (16 * MTM) + r) * tile_cols + 4 * q) * 4;
                store_agent_b128(slot_rsrc, off, f32x4{vg[0], vg[1], vg[2], vg[3]});
                if (wide) store_agent_b128(slot_rsrc, off + 512, f32x4{vl[0], vl[1], vl[2], vl[3]});
            }
            wait_all_memory();  // this lane's part has reached device-wide visibility
            __syncthreads();    // ... and so has everybody else's in this workgroup, before the arrival is counted
            if (threadIdx.x == 0) {
                const int seen = add_agent(&p.arrivals[ui], 1);
                sm_last = seen == slices - 1;
                if (sm_last) store_agent(&p.arrivals[ui], 0);  // leave the counter ready for the next launch
            }
            __syncthreads();
            finish = sm_last;
            if (finish) {
                // the sums replace this thread's part of the wavefront tiles (tile 0, and tile 2 for the second set of
                // columns; the others become zero), so that one epilogue serves both cases
                f32x4 vg[8], vl[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) vg[j] = vl[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                for (int c = 0; c < slices; ++c) {
                    const int base = (ui * slices + c) * (16 * MTM);
                    f32x4 tg[8], tl[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int r = (threadIdx.x >> 5) + 8 * j;
                        const int off = r < cur_rows ? ((base + r) * tile_cols + 4 * q) * 4 : kNoLoad;
                        tg[j] = load_agent_b128(slot_rsrc, off);
                        tl[j] = load_agent_b128(slot_rsrc, wide ? off + 512 : kNoLoad);
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        vg[j] += tg[j];
                        vl[j] += tl[j];
                    }
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int r = (threadIdx.x >> 5) + 8 * j;
                    if (r < cur_rows) {
                        float* dst = sm_part + r * kSplitPitch + 4 * q;
                        *(f32x4*)dst = vg[j];
                        *(f32x4*)(dst + TS) = f32x4{0.f, 0.f, 0.f, 0.f};
                        *(f32x4*)(dst + 2 * TS) = vl[j];
                        *(f32x4*)(dst + 3 * TS) = f32x4{0.f, 0.f, 0.f, 0.f};
                    }
                }
                // The epilogue of a span-major SwiGLU unit below reads the tile by another thread mapping than the one that
                // just wrote the sums (every other epilogue reads what the same thread wrote): the writes must have landed.
                // (`finish` is the same in every thread of the workgroup, so all of them arrive here.)
                if (PACKED && p.swiglu) lds_barrier();
            }
        }
        if (finish && PACKED && p.swiglu) {
            // A span's tile holds 64 gate columns followed by their 64 linear columns.  Thread (eq = q & 15) finishes 4 output
            // columns of one row for each span of the unit; the 32 threads that share threadIdx.x >> 5 take two rows.
            const int eq = q & 15;
            const int oc_a = cur_span * span_cols + 4 * eq, oc_b = oc_a + 64;  // first output column in the unit's first / second span
            const bool a_live = oc_a < NO, b_live = wide && oc_b < NO;
            const f32x4 bias_ga = load_f32x4(bias_rsrc, (p.bias && a_live) ? (cur_g * p.N + oc_a) * 4 : kNoLoad);
            const f32x4 bias_la = load_f32x4(bias_rsrc, (p.bias && a_live) ? (cur_g * p.N + NO + oc_a) * 4 : kNoLoad);
            const f32x4 bias_gb = load_f32x4(bias_rsrc, (p.bias && b_live) ? (cur_g * p.N + oc_b) * 4 : kNoLoad);
            const f32x4 bias_lb = load_f32x4(bias_rsrc, (p.bias && b_live) ? (cur_g * p.N + NO + oc_b) * 4 : kNoLoad);
            const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int r = 2 * (int)(threadIdx.x >> 5) + (q >> 4); r < cur_rows; r += 16) {
                const float* src = sm_part + r * kSplitPitch + 4 * eq;
                const f32x4 g0 = *(const f32x4*)src, g1 = *(const f32x4*)(src + TS), g2 = *(const f32x4*)(src + 2 * TS),
                            g3 = *(const f32x4*)(src + 3 * TS);
                const f32x4 l0 = *(const f32x4*)(src + 64), l1 = *(const f32x4*)(src + 64 + TS),
                            l2 = *(const f32x4*)(src + 64 + 2 * TS), l3 = *(const f32x4*)(src + 64 + 3 * TS);
                f32x4 ga, la, gb = zero4, lb = zero4;
                if (wide) {
                    ga = g0 + g1;
                    la = l0 + l1;
                    gb = g2 + g3;
                    lb = l2 + l3;
                } else {
                    ga = ((g0 + g1) + g2) + g3;
                    la = ((l0 + l1) + l2) + l3;
                }
                const size_t oa = (size_t)(cur_row0 + r) * NO + oc_a;
                f32x4 res_a = zero4, res_b = zero4;
                if (p.residual) {
                    res_a = load_bf16x4(res_rsrc, a_live ? (int)(oa * 2) : kNoLoad);
                    res_b = load_bf16x4(res_rsrc, b_live ? (int)((oa + 64) * 2) : kNoLoad);
                }
                if (a_live) finish4(p, ga, la, bias_ga, bias_la, res_a, out_index(p, cur_row0 + r, oc_a, NO));
                if (b_live) finish4(p, gb, lb, bias_gb, bias_lb, res_b, out_index(p, cur_row0 + r, oc_b, NO));
            }
        } else if (finish) {
            // biases of this thread's columns once per unit; residual values per row; every load unconditional (a null
            // operand is read with an offset outside its descriptor and yields zeros), rows two at a time
            const int oc = cur_span * span_cols + 4 * q;
            const int oc2 = p.swiglu ? NO + oc : oc + 128;  // second set of columns of a wide unit: linear columns, or the next span
            const bool oc_live = oc < NO, oc2_live = oc + 128 < NO;  // (a last span that N does not fill: nothing is stored past N)
            const f32x4 bias_v = load_f32x4(bias_rsrc, p.bias ? (cur_g * p.N + oc) * 4 : kNoLoad);
            const f32x4 bias_l = load_f32x4(bias_rsrc, (p.bias && wide) ? (cur_g * p.N + oc2) * 4 : kNoLoad);
            const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
            // Two copies of the row loop: without a residual there is no load in it, so nothing in it waits for memory -
            // a load in the loop makes every pass wait for the stores of the pass before (stores and loads share the
            // counter the compiler waits on), which cost ~1 us per pass.
            auto run_rows = [&](auto with_residual) {
                constexpr bool kRes = decltype(with_residual)::value;
                for (int r = threadIdx.x >> 5; r < cur_rows; r += 16) {
                    const int rb = min(r + 8, 16 * MTM - 1);  // second row of the pair (clamped: read, not written, when past the end)
                    const bool two = r + 8 < cur_rows;
                    float ag[4], al[4], bg[4], bl[4];
                    tile_row(r, ag, al);
                    tile_row(rb, bg, bl);
                    const size_t oa = (size_t)(cur_row0 + r) * NO + oc, ob = (size_t)(cur_row0 + rb) * NO + oc;
                    f32x4 ra = zero4, rb4 = zero4, ra2 = zero4, rb2 = zero4;
                    if constexpr (kRes) {
                        ra = load_bf16x4(res_rsrc, (int)(oa * 2));
                        rb4 = load_bf16x4(res_rsrc, two ? (int)(ob * 2) : kNoLoad);
                        if (wide && !p.swiglu) {
                            ra2 = load_bf16x4(res_rsrc, (int)((oa + 128) * 2));
                            rb2 = load_bf16x4(res_rsrc, two ? (int)((ob + 128) * 2) : kNoLoad);
                        }
                    }
                    if (wide && !p.swiglu) {  // two plain spans: finish them one after the other
                        if (oc_live) finish4(p, f32x4{ag[0], ag[1], ag[2], ag[3]}, zero4, bias_v, zero4, ra, out_index(p, cur_row0 + r, oc, NO));
                        if (oc2_live) finish4(p, f32x4{al[0], al[1], al[2], al[3]}, zero4, bias_l, zero4, ra2, out_index(p, cur_row0 + r, oc + 128, NO));
                        if (two) {
                            if (oc_live) finish4(p, f32x4{bg[0], bg[1], bg[2], bg[3]}, zero4, bias_v, zero4, rb4, out_index(p, cur_row0 + rb, oc, NO));
                            if (oc2_live) finish4(p, f32x4{bl[0], bl[1], bl[2], bl[3]}, zero4, bias_l, zero4, rb2, out_index(p, cur_row0 + rb, oc + 128, NO));
                        }
                    } else if (oc_live) {
                        finish4(p, f32x4{ag[0], ag[1], ag[2], ag[3]}, f32x4{al[0], al[1], al[2], al[3]}, bias_v, bias_l, ra, out_index(p, cur_row0 + r, oc, NO));
                        if (two) finish4(p, f32x4{bg[0], bg[1], bg[2], bg[3]}, f32x4{bl[0], bl[1], bl[2], bl[3]}, bias_v, bias_l, rb4, out_index(p, cur_row0 + rb, oc, NO));
                    }
                }
            };
            if (p.residual) run_rows(std::true_type{});
            else run_rows(std::false_type{});
        }
        lds_barrier();  // the tiles are free for the next unit
    }
    wait_all_memory();  // (requests of an item past the end return nothing, but must not outlive the wavefront's registers)
    if constexpr (!WIDE_DYN && !PACKED) asm volatile("" ::"v"(touched[0]), "v"(touched[1]));  // (the touch above is a real request)

    // rows at or beyond sum(group_sizes): zero product, bias of the last group (lax.ragged_dot semantics)
    const int total = total_rows;
    const int pad_rows = p.M - min(total, p.M);
    const int pad_spans = (NO + 127) / 128;
    for (int i = blockIdx.x; i < pad_rows * pad_spans; i += gridDim.x) {
        const int sp = i % pad_spans;
        if (threadIdx.x < 32 && sp * 128 + 4 * q < NO) {
            const int row = min(total, p.M) + i / pad_spans;
            float vg[4] = {0.f, 0.f, 0.f, 0.f}, vl[4] = {0.f, 0.f, 0.f, 0.f};
            group_epilogue(p, vg, vl, p.G - 1, row, sp * 128 + 4 * q, NO);
        }
    }
}

// ---- span-major copy of a weight array (done once, when the weights are loaded) ---------------------------------------
// One thread moves 8 consecutive elements of a packed row: they come from 8 consecutive columns of the reference's array
// (widths are multiples of 8, or 16 with gate and linear halves) or are zeros where the span runs past the last column.
#if LYRA_GEMM_HAS_ENTRY
struct PackParams {
    const uint8_t* src;
    uint8_t* dst;
    int G, K, N, es, glu, pspans;
};
__global__ __launch_bounds__(256) void gemm_pack_kernel(PackParams p) {
    const size_t total = (size_t)p.G * p.pspans * p.K * 16;  // pieces of 8 elements
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int piece = (int)(i & 15);
        const size_t row = i >> 4;  // (g * pspans + s) * K + k
        const int k = (int)(row % p.K);
        const size_t gs = row / p.K;
        const int s = (int)(gs % p.pspans), g = (int)(gs / p.pspans);
        int col;  // first source column of the piece, or -1
        if (p.glu) {
            const int half = p.N >> 1, c = 64 * s + 8 * (piece & 7);
            col = c < half ? (piece < 8 ? c : half + c) : -1;
        } else {
            const int c = 128 * s + 8 * piece;
            col = c < p.N ? c : -1;
        }
        const size_t dst = i * 8 * p.es;
        if (p.es == 1) {
            u32x2 v = u32x2{0u, 0u};
            if (col >= 0) v = *(const u32x2*)(p.src + ((size_t)g * p.K + k) * p.N + col);
            *(u32x2*)(p.dst + dst) = v;
        } else {
            u32x4 v = u32x4{0u, 0u, 0u, 0u};
            if (col >= 0) v = *(const u32x4*)(p.src + (((size_t)g * p.K + k) * p.N + col) * 2);
            *(u32x4*)(p.dst + dst) = v;
        }
    }
}
#endif  // LYRA_GEMM_HAS_ENTRY

static int packed_spans(int N, int layout) { return layout == 2 ? (N / 2 + 63) / 64 : (N + 127) / 128; }

struct GemmPlan {
    int mt;       // 16-row tiles held in registers per pass
    int row_par;  // row blocks of one group spread over this many workgroups
    int row_block = 64;  // K-split kernel: rows per block
    int spans;    // 128-column spans (64+64 with SwiGLU)
    int ksplit, kpart;
    bool one_pass;  // single group with a few MB of weights, swiglu tile layout: decode_gemm_small_kernel
    bool split_k;   // single group with a few MB of weights: decode_gemm_splitk_kernel + a sum over the K slices
    bool grouped;   // several groups: decode_gemm_group_kernel, one pass
    bool wide = false;  // ... with units of 256 plain columns
};

// Shape-only plan (group sizes live on the device).  Large weight sets are streamed once: wide row blocks, K
// split only as far as needed to fill 256 compute units.  Small ones (a few MB: the dense projections) are
// latency bound, so they are cut into as many independent 16-row x 128-column x K-slice pieces as the
// float32 partials allow, even though row tiles of one group then read the same weights through L2.
static GemmPlan plan_gemm(int M, int G, int K, int N, int bk, int fused_swiglu, bool allow_split_k = true) {
    static const long target_env = [] {
        const char* e = getenv("LYRA_GEMM_TARGET_WGS");  // tuning override, read once
        return e ? atol(e) : 0L;
    }();
    GemmPlan pl;
    const int touched = std::max(1, std::min(G, M));
    const double weight_bytes = (double)touched * K * N;
    static const bool no_one_pass = getenv("LYRA_GEMM_NO_ONE_PASS") != nullptr;  // tuning overrides
    static const bool no_split_k = getenv("LYRA_GEMM_NO_SPLIT_K") != nullptr;
    pl.one_pass = false;
    static const bool no_grouped = getenv("LYRA_GEMM_NO_GROUPED") != nullptr;
    // the kernels built on whole 128-column spans; any other width (a multiple of 8) goes to the general kernel
    const bool whole_spans = N % 128 == 0 && (!fused_swiglu || N % 256 == 0);
    pl.grouped = G > 1 && G <= kMaxStreamGroups && G + M / (16 * kGroupTiles) <= kMaxRowBlocks && !no_grouped;  // (any width)
    if (pl.grouped) {
        pl.mt = 4;
        pl.row_par = 1;
        static const bool want_wide = getenv("LYRA_GEMM_WIDE") != nullptr;  // tuning override: 256-column units whatever their number
        pl.wide = !fused_swiglu && N % 256 == 0 && want_wide;
        pl.spans = fused_swiglu ? (N / 2 + 127) / 128 : (pl.wide ? N / 256 : (N + 127) / 128);
        pl.ksplit = 1;
        pl.kpart = K;
        pl.split_k = false;
        return pl;
    }
    // (a K that is not a multiple of 128 leaves the last slice's wavefronts unequal shares, which is fine; scale blocks
    // along K are only lined up with the slices for K % 128 == 0)
    pl.split_k = allow_split_k && G == 1 && weight_bytes <= 160e6 && M <= 256 && (K % 128 == 0 || bk <= 0 || bk >= K) && !no_split_k;
    if (pl.split_k) {
        // ~256 workgroups; a slice is a multiple of 128 rows (4 wavefronts x 32) and of the scale block, at most 512 rows
        pl.mt = 4;
        pl.spans = (N + 127) / 128;
        // Row blocks of 64, 32 or 16 rows: as many blocks as still leave K slices of 512 rows for ~256 workgroups.  These
        // launches are bound by what one workgroup has to pull in and by the float32 slices their consumer sums, not by their
        // bytes: smaller blocks shrink a workgroup's activation slice and partial tile, and more row blocks mean fewer K
        // slices (2048-wide variant at 64 rows: q/k/v 8 -> 4 slices with 32-row blocks, output projection 8 -> 4 with 16-row
        // blocks; decode step -3 %).  Matrices with enough spans and slices to fill the device keep 64-row blocks: smaller
        // ones would read the weights again for nothing (4096-wide variant: +4 % when forced).
        static const int row_block_env = [] {
            const char* e = getenv("LYRA_GEMM_ROW_BLOCK");  // tuning override, read once: 16, 32 or 64 for every K-split launch
            return e ? atoi(e) : 0;
        }();
        const long blocks_wanted = std::max(1L, 256L / ((long)pl.spans * ((K + 511) / 512)));
        pl.row_block = 64;
        while (pl.row_block > 16 && (M + pl.row_block / 2 - 1) / (pl.row_block / 2) <= blocks_wanted) pl.row_block /= 2;
        if (row_block_env == 16 || row_block_env == 32 || row_block_env == 64) pl.row_block = row_block_env;
        pl.row_par = (M + pl.row_block - 1) / pl.row_block;
        // slices of at least 256 rows: 128-row slices fill more compute units but double the float32 slices the consumer
        // has to sum (2048 x 2048 out projection: 16 -> 8 slices shortened the decode step by 1.2 %)
        int unit = (K % 256 == 0 && K >= 512) ? 256 : 128;
        if (bk > 0 && bk < K) unit = std::max(unit, (bk + 127) / 128 * 128);
        const long want = std::max(1L, 256L / ((long)pl.spans * pl.row_par));
        int kpart = (int)((K + want - 1) / want);
        // up to 512 rows per slice everything is requested at once; longer slices (larger matrices) refill 4 register sets
        kpart = std::min(2048, (kpart + unit - 1) / unit * unit);
        if (unit > 512 || (bk > 0 && bk < K && kpart % bk)) pl.split_k = false;  // scale blocks that do not tile a slice
        pl.kpart = kpart;
        pl.ksplit = (K + kpart - 1) / kpart;
        if (pl.split_k) return pl;
    }
    pl.one_pass = G == 1 && weight_bytes <= 48e6 && whole_spans && !no_one_pass;
    if (pl.one_pass) {
        pl.mt = 1;
        pl.row_par = (M + 15) / 16;
        pl.spans = fused_swiglu ? (N / 2 + 63) / 64 : (N + 127) / 128;
        pl.ksplit = 1;
        pl.kpart = K;
        return pl;
    }
    const bool small = weight_bytes <= 48e6 && M > 16;
    pl.mt = M <= 16 ? 1 : (small ? 1 : (M <= 32 ? 2 : 4));
    pl.row_par = small ? std::min(8, (M / std::max(1, touched) + 15) / 16) : 1;
    pl.row_par = std::max(1, pl.row_par);
    pl.spans = fused_swiglu ? (N / 2 + 63) / 64 : (N + 127) / 128;
    const long wgs_noksplit = (long)((pl.spans + kGemmWaves - 1) / kGemmWaves) * touched * pl.row_par;
    const long target = target_env > 0 ? target_env : 512;
    int unit = 32;
    if (bk > 0 && bk < K) unit = std::max(unit, bk);  // splits start on a scale-block boundary
    const int max_split = std::max(1, K / std::max(unit, 256));
    int ksplit = (int)std::min((long)max_split, std::max(1L, target / std::max(1L, wgs_noksplit)));
    int kpart = (K + ksplit - 1) / ksplit;
    kpart = (kpart + unit - 1) / unit * unit;
    pl.ksplit = (K + kpart - 1) / kpart;
    pl.kpart = kpart;
    return pl;
}

// Launches the K-split kernel of a plan with split_k set for weights of format WT (0 bf16, 1 e4m3fn, 2 e5m2); p.part
// receives [ksplit, M, N] float32 slices.
template <int WT>
int launch_split_k_fmt(const GemmParams& p, const GemmPlan& pl, hipStream_t st);
// Sums the K slices in p.part and applies the epilogue (the finish kernel lives in the pass with the entry points).
int launch_finish(const GemmParams& p, hipStream_t st);

#if LYRA_GEMM_HAS_SPLITK
template <int WT>
int launch_split_k_fmt(const GemmParams& p, const GemmPlan& pl, hipStream_t st) {
    const dim3 grid(pl.spans, pl.ksplit, pl.row_par), block(kSplitWaves * 64);
    const size_t lds = (size_t)kSplitWaves * 64 * kSplitPitch * sizeof(float);
    const int depth = (pl.kpart / 32 + kSplitWaves - 1) / kSplitWaves;  // 1..4 steps per wavefront, or more: the looping variant
    const bool loop = depth > 4;
    // scales that change along K: free when every wavefront's rows (32 * depth) lie within one scale block
    const int step_scales =
        !(WT != 0 && p.scale_mode == 1 && p.bk < p.K) ? 0 : ((!loop && p.bk % (32 * std::max(1, std::min(depth, 4))) == 0) ? 1 : 2);
#define LYRA_SPLITK_M(D, S, M_)                                                                                        \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)decode_gemm_splitk_kernel<WT, D, S, false, M_>, \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);     \
        if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                                 \
        hipLaunchKernelGGL((decode_gemm_splitk_kernel<WT, D, S, false, M_>), grid, block, lds, st, p);                \
    } while (0)
#define LYRA_SPLITK(D, S)                              \
    do {                                               \
        if (pl.row_block <= 16) LYRA_SPLITK_M(D, S, 1); \
        else if (pl.row_block <= 32) LYRA_SPLITK_M(D, S, 2); \
        else LYRA_SPLITK_M(D, S, 4);                   \
    } while (0)
#define LYRA_SPLITK_LOOP(S)                                                                                            \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)decode_gemm_splitk_kernel<WT, (WT ? 4 : 2), S, true>, \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);     \
        if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                                 \
        hipLaunchKernelGGL((decode_gemm_splitk_kernel<WT, (WT ? 4 : 2), S, true>), grid, block, lds, st, p);           \
    } while (0)
#define LYRA_SPLITK_D(S)                   \
    do {                                   \
        if (depth <= 1) LYRA_SPLITK(1, S); \
        else if (depth == 2) LYRA_SPLITK(2, S); \
        else if (depth == 3) LYRA_SPLITK(3, S); \
        else LYRA_SPLITK(4, S);            \
    } while (0)
    if constexpr (WT != 0) {
        if (loop) {
            if (step_scales == 2) LYRA_SPLITK_LOOP(2);
            else LYRA_SPLITK_LOOP(0);
        } else if (step_scales == 1) LYRA_SPLITK_D(1);
        else if (step_scales == 2) LYRA_SPLITK_D(2);
        else LYRA_SPLITK_D(0);
    } else {
        if (loop) LYRA_SPLITK_LOOP(0);
        else LYRA_SPLITK_D(0);
    }
#undef LYRA_SPLITK_D
#undef LYRA_SPLITK_LOOP
#undef LYRA_SPLITK
#undef LYRA_SPLITK_M
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}
#if LYRA_GEMM_PART == 2
template int launch_split_k_fmt<0>(const GemmParams&, const GemmPlan&, hipStream_t);
template int launch_split_k_fmt<1>(const GemmParams&, const GemmPlan&, hipStream_t);
#elif LYRA_GEMM_PART == 4
template int launch_split_k_fmt<2>(const GemmParams&, const GemmPlan&, hipStream_t);
#endif
#endif  // LYRA_GEMM_HAS_SPLITK


}  // namespace lyra

namespace lyra {
// Launches the kernels of a plan for weights of format WT (0 bf16, 1 e4m3fn, 2 e5m2); p is complete except even_spans.
template <int WT>
int launch_planned(GemmParams p, const GemmPlan& pl, int layout, int fused_swiglu, float* tile_max, hipStream_t st);

#if LYRA_GEMM_HAS_LAUNCH
template <int WT>
int launch_planned(GemmParams p, const GemmPlan& pl, int layout, int fused_swiglu, float* tile_max, hipStream_t st) {
    constexpr bool fp8 = WT != 0;
    const int M = p.M, G = p.G, K = p.K, N = p.N;
    if (pl.grouped) {
        // one workgroup per compute unit (more would only queue behind the LDS tiles), fewer when there is less work
        const long most_blocks = std::min((long)G + M / (16 * kGroupTiles), (long)std::max(1, M));
        // (packed: units of one span unless the list is long enough for units of two - the kernel's own rule, on the most
        // row blocks the shapes allow)
        const bool packed_wide = layout && 4 * most_blocks * ((p.pspans + 1) / 2) >= 7 * (long)kGroupMaxWgs;
        const long most_units = (layout ? (long)p.pspans : (long)pl.spans) * most_blocks;
        const int gkw = layout ? (packed_wide ? 2 : kSplitWaves) : ((fused_swiglu || pl.wide) ? 2 : kSplitWaves);
        const long trips_least = std::max(1, ((K / 32 + gkw - 1) / gkw + 7) / 8);  // trips per unit (at least)
        const dim3 ggrid((unsigned)std::max(1L, std::min((long)kGroupMaxWgs, most_units * trips_least))), gblock(kSplitWaves * 64);
        const size_t glds = (size_t)kSplitWaves * 16 * kGroupTiles * kSplitPitch * sizeof(float);
        const bool step_scales = fp8 && p.scale_mode == 1 && p.bk < p.K;
#define LYRA_GROUP_RS(F, S, R, C)                                                                                     \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)decode_gemm_group_kernel<F, S, R, C>,        \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)glds);    \
        if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                                 \
        hipLaunchKernelGGL((decode_gemm_group_kernel<F, S, R, C>), ggrid, gblock, glds, st, p);                       \
    } while (0)
    // fewer units than workgroups whatever the group sizes: the variant that cuts units into K slices
    // without SwiGLU, when the shapes allow 1.75 rounds of 256-column units: the variant that decides on them on the device
    static const bool no_wide_dyn = getenv("LYRA_GEMM_NO_WIDE_IF_MANY") != nullptr;  // tuning override
    const bool wide_dyn = !no_wide_dyn && !fused_swiglu && !pl.wide && N % 256 == 0 &&
                          4 * std::min((long)G + M / (16 * kGroupTiles), (long)std::max(1, M)) * (N / 256) >= 7 * (long)kGroupMaxWgs;
#define LYRA_GROUP_RSW(F, S, R)                                                                                       \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)decode_gemm_group_kernel<F, S, R, false, true>, \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)glds);    \
        if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                                 \
        hipLaunchKernelGGL((decode_gemm_group_kernel<F, S, R, false, true>), ggrid, gblock, glds, st, p);             \
    } while (0)
#define LYRA_GROUP_P(F, S, R, C, W)                                                                                   \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)decode_gemm_group_kernel<F, S, R, C, W, true>, \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)glds);    \
        if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                                 \
        hipLaunchKernelGGL((decode_gemm_group_kernel<F, S, R, C, W, true>), ggrid, gblock, glds, st, p);              \
    } while (0)
#define LYRA_GROUP_R(F, S, R)                                               \
    do {                                                                    \
        if (layout) {                                                       \
            if (most_units < (long)kGroupMaxWgs && p.max_slices > 1) LYRA_GROUP_P(F, S, R, true, false); \
            else LYRA_GROUP_P(F, S, R, false, true);                        \
        } else if (most_units < (long)kGroupMaxWgs && p.max_slices > 1) LYRA_GROUP_RS(F, S, R, true); \
        else if (wide_dyn) LYRA_GROUP_RSW(F, S, R);                         \
        else LYRA_GROUP_RS(F, S, R, false);                                 \
    } while (0)
#define LYRA_GROUP(F, S, DEPTH_)                                                          \
    do {                                                                                  \
        const int kw = gkw;                                                               \
        const int per_wave = (K / 32 + kw - 1) / kw;                                      \
        const int rounds = (per_wave + (DEPTH_) - 1) / (DEPTH_);                          \
        if (K % (kw * 32) == 0 && rounds % 2 == 0) LYRA_GROUP_R(F, S, 2);                 \
        else LYRA_GROUP_R(F, S, 1);                                                       \
    } while (0)
        if constexpr (WT != 0) {
            if (step_scales) LYRA_GROUP(WT, true, 4);
            else LYRA_GROUP(WT, false, 4);
        } else {
            LYRA_GROUP(0, false, 2);
        }
#undef LYRA_GROUP
#undef LYRA_GROUP_R
#undef LYRA_GROUP_P
#undef LYRA_GROUP_RSW
#undef LYRA_GROUP_RS
        return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
    }
    if (pl.split_k) {
        const int rc = launch_split_k_fmt<WT>(p, pl, st);
        if (rc != LYRA_OK) return rc;
        return launch_finish(p, st);
    }
    if (pl.one_pass) {
        const dim3 sgrid(pl.spans, pl.row_par), sblock(kSmallWaves * 64);
        const size_t slds = (size_t)kSmallWaves * 16 * 128 * sizeof(float);
        const int per_wave = (K / 32 + kSmallWaves - 1) / kSmallWaves;  // steps of 32 rows each wavefront walks
        const bool step_scales = fp8 && p.scale_mode == 1 && p.bk < p.K;
#define LYRA_SMALL(F, D, S, O) hipLaunchKernelGGL((decode_gemm_small_kernel<F, D, S, O>), sgrid, sblock, slds, st, p)
        if constexpr (WT != 0) {
            if (step_scales) {
                if (per_wave <= 4) LYRA_SMALL(WT, 4, true, true);
                else LYRA_SMALL(WT, 4, true, false);
            } else {
                if (per_wave <= 2) LYRA_SMALL(WT, 2, false, true);
                else if (per_wave <= 4) LYRA_SMALL(WT, 4, false, true);
                else if (per_wave <= 6) LYRA_SMALL(WT, 6, false, true);
                else if (per_wave <= 8) LYRA_SMALL(WT, 8, false, true);
                else LYRA_SMALL(WT, 6, false, false);
            }
        } else {
            if (per_wave <= 2) LYRA_SMALL(0, 2, false, true);
            else if (per_wave <= 4) LYRA_SMALL(0, 4, false, true);
            else LYRA_SMALL(0, 4, false, false);
        }
#undef LYRA_SMALL
        return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
    }
    dim3 grid((pl.spans + kGemmWaves - 1) / kGemmWaves, pl.ksplit, G * pl.row_par), block(kGemmWaves * 64);
    // a very wide single projection (the LM head): one workgroup per compute unit with as many wavefronts as its share of spans
    static const bool no_even = getenv("LYRA_GEMM_NO_EVEN_SPANS") != nullptr;  // tuning override
    const int per_cu = (pl.spans + kGroupMaxWgs - 1) / kGroupMaxWgs;
    if (!no_even && G == 1 && pl.ksplit == 1 && pl.row_par == 1 && pl.spans >= 4 * kGroupMaxWgs && per_cu <= (pl.mt == 1 ? 12 : 8)) {
        p.even_spans = 1;
        grid = dim3(kGroupMaxWgs, 1, 1);
        block = dim3(per_cu * 64);
    }
    const size_t lds = (size_t)16 * pl.mt * (512 + 8) * sizeof(uint16_t) +
                       (tile_max ? (size_t)(block.x / 64) * 16 * pl.mt * kTileMaxPitch * sizeof(float) : 0);
#define LYRA_LAUNCH_GEMM(F, T)                                                                                         \
    do {                                                                                                               \
        if (tile_max) {                                                                                                \
            static const hipError_t attr = hipFuncSetAttribute((const void*)decode_gemm_kernel<F, T, true>,            \
                                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (attr != hipSuccess) return LYRA_E_LAUNCH;                                                              \
            hipLaunchKernelGGL((decode_gemm_kernel<F, T, true>), grid, block, lds, st, p);                             \
        } else {                                                                                                       \
            hipLaunchKernelGGL((decode_gemm_kernel<F, T>), grid, block, lds, st, p);                                   \
        }                                                                                                              \
    } while (0)
    if (pl.mt == 1) LYRA_LAUNCH_GEMM(WT, 1);
    else if (pl.mt == 2) LYRA_LAUNCH_GEMM(WT, 2);
    else LYRA_LAUNCH_GEMM(WT, 4);
#undef LYRA_LAUNCH_GEMM
    if (hipGetLastError() != hipSuccess) return LYRA_E_LAUNCH;
    if (pl.ksplit > 1) return launch_finish(p, st);
    return LYRA_OK;
}
#if LYRA_GEMM_PART == 1
extern template int launch_planned<2>(GemmParams, const GemmPlan&, int, int, float*, hipStream_t);  // (pass 3 has it)
template int launch_planned<0>(GemmParams, const GemmPlan&, int, int, float*, hipStream_t);
template int launch_planned<1>(GemmParams, const GemmPlan&, int, int, float*, hipStream_t);
#elif LYRA_GEMM_PART == 3
template int launch_planned<2>(GemmParams, const GemmPlan&, int, int, float*, hipStream_t);
#endif
#endif  // LYRA_GEMM_HAS_LAUNCH
}  // namespace lyra

#if LYRA_GEMM_HAS_ENTRY

namespace lyra {
int launch_finish(const GemmParams& p, hipStream_t st) {
    const int NO = p.swiglu ? p.N / 2 : p.N;
    hipLaunchKernelGGL(decode_gemm_finish_kernel, dim3((unsigned)((NO / 4 + 255) / 256), (unsigned)std::min(p.M, 65535)), dim3(256), 0, st, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

// Bytes of float32 partials (behind the counters) that the launch of `pl` writes.
static size_t gemm_partial_bytes(const GemmPlan& pl, int M, int N) {
    if (pl.grouped)  // one tile slot of 64 rows x 256 columns per workgroup
        return (size_t)kGroupMaxWgs * 16 * kGroupTiles * 256 * sizeof(float);
    if (pl.ksplit == 1 && !pl.split_k) return 0;
    return ((size_t)pl.ksplit * M * N * sizeof(float) + 255) / 256 * 256;
}
}  // namespace lyra

extern "C" size_t lyra_gemm_packed_bytes(int G, int K, int N, int rhs_dtype, int layout) {
    if (G <= 0 || K <= 0 || N <= 0 || (layout != 1 && layout != 2)) return 0;
    if (rhs_dtype != LYRA_DTYPE_BF16 && !lyra::one_byte_format(rhs_dtype)) return 0;
    if (N % 8 || (layout == 2 && N % 16)) return 0;
    return (size_t)G * lyra::packed_spans(N, layout) * K * 128 * (lyra::one_byte_format(rhs_dtype) ? 1 : 2);
}

extern "C" int lyra_gemm_pack(const void* rhs, void* packed, int G, int K, int N, int rhs_dtype, int layout, lyra_stream_t stream) {
    using namespace lyra;
    if (!rhs || !packed || G <= 0 || K <= 0 || N <= 0 || (layout != 1 && layout != 2)) return LYRA_E_BADARG;
    if (rhs_dtype != LYRA_DTYPE_BF16 && !lyra::one_byte_format(rhs_dtype)) return LYRA_E_UNSUPPORTED;
    if (N % 8 || (layout == 2 && N % 16)) return LYRA_E_UNSUPPORTED;
    if (((uintptr_t)rhs | (uintptr_t)packed) % 16) return LYRA_E_BADARG;
    PackParams p{(const uint8_t*)rhs, (uint8_t*)packed, G, K, N, lyra::one_byte_format(rhs_dtype) ? 1 : 2, layout == 2, packed_spans(N, layout)};
    const size_t pieces = (size_t)G * p.pspans * K * 16;
    const unsigned blocks = (unsigned)std::min<size_t>((pieces + 255) / 256, 65536);
    hipLaunchKernelGGL(gemm_pack_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}

extern "C" size_t lyra_decode_gemm_workspace(int M, int G, int K, int N, int fused_swiglu) {
    if (M <= 0 || G <= 0 || K <= 0 || N <= 0) return 0;
    // The scale block is not known here and decides both which kernel runs (a block that does not tile a K slice sends a
    // small projection to the general kernel) and how many K slices it writes; a coarser block only ever lowers the slice
    // count of either kernel, so the larger of the two plans without a block covers every block.
    const lyra::GemmPlan with_split = lyra::plan_gemm(M, G, K, N, 0, fused_swiglu, true);
    const lyra::GemmPlan general = lyra::plan_gemm(M, G, K, N, 0, fused_swiglu, false);
    return lyra::kGemmCounterBytes + std::max(lyra::gemm_partial_bytes(with_split, M, N), lyra::gemm_partial_bytes(general, M, N));
}

extern "C" size_t lyra_decode_gemm_workspace_for(int M, int G, int K, int N, int bk, int fused_swiglu) {
    if (M <= 0 || G <= 0 || K <= 0 || N <= 0 || bk < 0) return 0;
    const lyra::GemmPlan pl = lyra::plan_gemm(M, G, K, N, bk, fused_swiglu);
    return lyra::kGemmCounterBytes + lyra::gemm_partial_bytes(pl, M, N);
}

extern "C" int lyra_decode_gemm(const void* lhs, const void* rhs, const float* rhs_scale, int bk, int bn,
                                const int32_t* group_sizes, const float* bias, void* out, void* workspace,
                                size_t workspace_bytes, int M, int G, int K, int N, int rhs_dtype, int out_dtype,
                                int fused_swiglu, float swiglu_beta, float swiglu_limit, lyra_stream_t stream) {
    return lyra_decode_gemm_ex(lhs, nullptr, rhs, rhs_scale, bk, bn, group_sizes, bias, nullptr, 1.0f, 0, out, workspace,
                               workspace_bytes, M, G, K, N, rhs_dtype, out_dtype, fused_swiglu, swiglu_beta, swiglu_limit, stream);
}

namespace lyra {
static int run_decode_gemm(const void* lhs, const int32_t* lhs_row_map, const void* rhs, const float* rhs_scale, int bk, int bn,
                           const int32_t* group_sizes, const float* bias, const void* residual, float out_scale, int post_scale,
                           void* out, float* tile_max, void* workspace, size_t workspace_bytes, int M, int G, int K, int N,
                           int rhs_dtype, int out_dtype, int fused_swiglu, float swiglu_beta, float swiglu_limit,
                           lyra_stream_t stream);
}

extern "C" int lyra_decode_gemm_ex(const void* lhs, const int32_t* lhs_row_map, const void* rhs, const float* rhs_scale, int bk,
                                   int bn, const int32_t* group_sizes, const float* bias, const void* residual, float out_scale,
                                   int post_scale, void* out, void* workspace, size_t workspace_bytes, int M, int G, int K, int N,
                                   int rhs_dtype, int out_dtype, int fused_swiglu, float swiglu_beta, float swiglu_limit,
                                   lyra_stream_t stream) {
    return lyra::run_decode_gemm(lhs, lhs_row_map, rhs, rhs_scale, bk, bn, group_sizes, bias, residual, out_scale, post_scale, out,
                                 nullptr, workspace, workspace_bytes, M, G, K, N, rhs_dtype, out_dtype, fused_swiglu, swiglu_beta,
                                 swiglu_limit, stream);
}

extern "C" int lyra_decode_gemm_tile_max(const void* lhs, const int32_t* lhs_row_map, const void* rhs, const float* rhs_scale, int bk,
                                         int bn, const int32_t* group_sizes, const float* bias, void* out, float* tile_max,
                                         void* workspace, size_t workspace_bytes, int M, int G, int K, int N, int rhs_dtype,
                                         int out_dtype, lyra_stream_t stream) {
    if (!tile_max) return LYRA_E_BADARG;
    return lyra::run_decode_gemm(lhs, lhs_row_map, rhs, rhs_scale, bk, bn, group_sizes, bias, nullptr, 1.0f, 0, out, tile_max,
                                 workspace, workspace_bytes, M, G, K, N, rhs_dtype, out_dtype, 0, 0.f, 0.f, stream);
}

namespace lyra {
static int run_decode_gemm(const void* lhs, const int32_t* lhs_row_map, const void* rhs, const float* rhs_scale, int bk, int bn,
                           const int32_t* group_sizes, const float* bias, const void* residual, float out_scale, int post_scale,
                           void* out, float* tile_max, void* workspace, size_t workspace_bytes, int M, int G, int K, int N,
                           int rhs_dtype, int out_dtype, int fused_swiglu, float swiglu_beta, float swiglu_limit,
                           lyra_stream_t stream) {
    const bool bias_post = (post_scale & 2) != 0;  // post_scale: bit 0 the scale / residual epilogue, bit 1 the bias after the cast
    post_scale &= 1;
    const bool lhs_tiled = (rhs_dtype & LYRA_LHS_TILED16) != 0, out_tiled = (rhs_dtype & LYRA_OUT_TILED16) != 0;
    // span-major weights (lyra_gemm_pack): the layout travels in the upper bits of rhs_dtype
    const int layout = (rhs_dtype & LYRA_RHS_SPAN_MAJOR) ? 1 : ((rhs_dtype & LYRA_RHS_SPAN_MAJOR_GLU) ? 2 : 0);
    if ((rhs_dtype & LYRA_RHS_SPAN_MAJOR) && (rhs_dtype & LYRA_RHS_SPAN_MAJOR_GLU)) return LYRA_E_BADARG;
    rhs_dtype &= ~(LYRA_RHS_SPAN_MAJOR | LYRA_RHS_SPAN_MAJOR_GLU | LYRA_LHS_TILED16 | LYRA_OUT_TILED16);
    if (residual && (!post_scale || out_dtype != LYRA_DTYPE_BF16)) return LYRA_E_BADARG;
    if (bias_post && (!bias || out_dtype != LYRA_DTYPE_BF16)) return LYRA_E_BADARG;
    if (bias_post && (G != 1 || fused_swiglu)) return LYRA_E_UNSUPPORTED;
    if (!lhs || !rhs || !group_sizes || !out) return LYRA_E_BADARG;
    if (M <= 0 || G <= 0 || K <= 0 || N <= 0) return LYRA_E_BADARG;
    if (rhs_dtype != LYRA_DTYPE_BF16 && !lyra::one_byte_format(rhs_dtype)) return LYRA_E_UNSUPPORTED;
    if (out_dtype != LYRA_DTYPE_BF16 && out_dtype != LYRA_DTYPE_F32) return LYRA_E_UNSUPPORTED;
    const bool fp8 = one_byte_format(rhs_dtype);
    if (fp8 != (rhs_scale != nullptr)) return LYRA_E_BADARG;
    if (K % 32 || N % 8 || (fused_swiglu && N % 16) || G > 8191) return LYRA_E_UNSUPPORTED;  // (a lane holds 8 columns)
    if ((size_t)M * N * 4 >= (1ull << 31)) return LYRA_E_UNSUPPORTED;  // results are stored through 31-bit buffer offsets

    GemmParams p;
    p.scale_mode = 0;
    p.bk = p.bn = 1;
    p.KB = p.NB = 1;
    p.bn_shift = 0;
    p.bk_shift = 0;
    if (fp8) {
        if (bk <= 0 || bn <= 0 || K % bk || N % bn) return LYRA_E_BADARG;
        if (bn & (bn - 1)) return LYRA_E_UNSUPPORTED;  // scale columns must be a power of two wide
        p.bk = bk; p.bn = bn; p.KB = K / bk; p.NB = N / bn;
        p.bn_shift = __builtin_ctz((unsigned)bn);
        p.bk_shift = (bk & (bk - 1)) ? -1 : __builtin_ctz((unsigned)bk);
        if (bn % 8 == 0 && (bk % 32 == 0 || bk == K)) p.scale_mode = 1;
        else if (bk == K) p.scale_mode = 2;
        else return LYRA_E_UNSUPPORTED;
    }
    const GemmPlan pl = plan_gemm(M, G, K, N, fp8 ? bk : 0, fused_swiglu);
    // the packed copy exists for the kernels that stream whole spans: several groups (layout 2 with SwiGLU, else 1), the
    // K-split projections of one group (layout 1) and the general kernel without SwiGLU (layout 1; offsets below 2 GB)
    if (layout && !((pl.grouped && layout == (fused_swiglu ? 2 : 1)) || (!pl.grouped && pl.split_k && layout == 1) ||
                    (!pl.grouped && !pl.split_k && !pl.one_pass && layout == 1 && !fused_swiglu && (size_t)G * packed_spans(N, 1) * K * 256 < (1ull << 31)))) return LYRA_E_UNSUPPORTED;
    if (layout && ((uintptr_t)rhs % 128)) return LYRA_E_BADARG;
    p.packed = layout;
    p.pspans = layout ? packed_spans(N, layout) : 0;
    // tiled activations: the grouped kernel and the K-split kernel (whose finish step writes the output); a tiled output is
    // bf16, a whole number of 32-column tiles, no residual
    if ((lhs_tiled || out_tiled) && !pl.grouped && !pl.split_k) return LYRA_E_UNSUPPORTED;
    if (out_tiled && (out_dtype != LYRA_DTYPE_BF16 || residual || (fused_swiglu ? N / 2 : N) % 32)) return LYRA_E_UNSUPPORTED;
    p.lhs_tiled = lhs_tiled;
    p.out_tiled = out_tiled;
    // tile maxima: what the plain kernel's epilogue can give - every (row, span) finished by one wavefront, in float32
    if (tile_max && (G != 1 || pl.grouped || pl.split_k || pl.one_pass || pl.ksplit > 1 || fused_swiglu ||
                     out_dtype != LYRA_DTYPE_F32 || post_scale || bias_post))
        return LYRA_E_UNSUPPORTED;
    p.tile_max = tile_max;
    p.tile_ld = (N + 127) / 128;
    p.lhs = (const uint16_t*)lhs;
    p.rhs = (const uint8_t*)rhs;
    p.scale = rhs_scale;
    p.group_sizes = group_sizes;
    p.bias = bias;
    p.out = out;
    p.part = nullptr;
    p.M = M; p.G = G; p.K = K; p.N = N;
    p.out_f32 = out_dtype == LYRA_DTYPE_F32;
    p.swiglu = fused_swiglu != 0;
    p.beta = swiglu_beta;
    p.limit = swiglu_limit;
    p.ksplit = pl.ksplit;
    p.row_par = pl.row_par;
    p.row_block = pl.row_block;
    p.kpart = pl.kpart;
    p.row_map = lhs_row_map;
    p.wide = pl.wide;
    static const int max_slices_env = [] {
        const char* e = getenv("LYRA_GEMM_MAX_SLICES");  // tuning override, read once
        return e ? atoi(e) : 64;
    }();
    p.max_slices = max_slices_env;
    static const int snake_env = [] {
        const char* e = getenv("LYRA_GEMM_SNAKE");  // tuning override, read once: 0 never, 1 always
        return e ? atoi(e) : -1;
    }();
    p.snake = snake_env;
    static const bool no_touch = getenv("LYRA_GEMM_NO_TOUCH") != nullptr;  // tuning override
    p.touch_last = no_touch ? 0 : 1;
    p.even_spans = 0;
    p.residual = (const uint16_t*)residual;
    p.out_scale = out_scale;
    p.post_scale = post_scale != 0;
    p.bias_post = bias_post ? 1 : 0;
    p.arrivals = nullptr;
    if (pl.ksplit > 1 || pl.split_k || pl.grouped) {
        // the first kGemmCounterBytes belong to the grouped kernel's arrival counters, whichever kernel runs
        // (checked against the plan that is launched: never more than lyra_decode_gemm_workspace answers for the shape)
        const size_t need = kGemmCounterBytes + gemm_partial_bytes(pl, M, N);
        if (need >= (1ull << 31)) return LYRA_E_UNSUPPORTED;
        if (!workspace || workspace_bytes < need || ((uintptr_t)workspace % 256)) return LYRA_E_WORKSPACE;
        p.arrivals = (int*)workspace;
        p.part = (float*)((char*)workspace + kGemmCounterBytes);
    }

    hipStream_t st = (hipStream_t)stream;
    if (rhs_dtype == LYRA_DTYPE_E5M2) return launch_planned<2>(p, pl, layout, fused_swiglu, tile_max, st);
    if (fp8) return launch_planned<1>(p, pl, layout, fused_swiglu, tile_max, st);
    return launch_planned<0>(p, pl, layout, fused_swiglu, tile_max, st);
}
}  // namespace lyra

extern "C" int lyra_decode_gemm_splits(int M, int K, int N, int bk) {
    if (M <= 0 || K <= 0 || N <= 0 || K % 32 || N % 8) return 0;  // (a last span that N does not fill is fine)
    const lyra::GemmPlan pl = lyra::plan_gemm(M, 1, K, N, bk, 0);
    return pl.split_k ? pl.ksplit : 0;
}

extern "C" int lyra_decode_gemm_partials(const void* lhs, const void* rhs, const float* rhs_scale, int bk, int bn,
                                         const int32_t* group_sizes, float* partials, size_t partials_bytes, int M, int K, int N,
                                         int rhs_dtype, lyra_stream_t stream) {
    using namespace lyra;
    if (!lhs || !rhs || !group_sizes || !partials || M <= 0 || K <= 0 || N <= 0) return LYRA_E_BADARG;
    if (rhs_dtype & LYRA_RHS_SPAN_MAJOR_GLU) return LYRA_E_UNSUPPORTED;
    const int layout = (rhs_dtype & LYRA_RHS_SPAN_MAJOR) ? 1 : 0;
    const bool lhs_tiled = (rhs_dtype & LYRA_LHS_TILED16) != 0;
    if (rhs_dtype & LYRA_OUT_TILED16) return LYRA_E_UNSUPPORTED;  // (the slices are float32, row-major)
    rhs_dtype &= ~(LYRA_RHS_SPAN_MAJOR | LYRA_LHS_TILED16);
    if (layout && ((uintptr_t)rhs % 128)) return LYRA_E_BADARG;
    if (rhs_dtype != LYRA_DTYPE_BF16 && !lyra::one_byte_format(rhs_dtype)) return LYRA_E_UNSUPPORTED;
    const bool fp8 = one_byte_format(rhs_dtype);
    if (fp8 != (rhs_scale != nullptr)) return LYRA_E_BADARG;
    if (K % 32 || N % 8) return LYRA_E_UNSUPPORTED;
    GemmParams p = {};
    p.bk = p.bn = p.KB = p.NB = 1;
    if (fp8) {
        if (bk <= 0 || bn <= 0 || K % bk || N % bn) return LYRA_E_BADARG;
        if (bn & (bn - 1)) return LYRA_E_UNSUPPORTED;
        p.bk = bk; p.bn = bn; p.KB = K / bk; p.NB = N / bn;
        p.bn_shift = __builtin_ctz((unsigned)bn);
        p.bk_shift = (bk & (bk - 1)) ? -1 : __builtin_ctz((unsigned)bk);
        if (bn % 8 == 0 && (bk % 32 == 0 || bk == K)) p.scale_mode = 1;
        else if (bk == K) p.scale_mode = 2;
        else return LYRA_E_UNSUPPORTED;
    }
    const GemmPlan pl = plan_gemm(M, 1, K, N, fp8 ? bk : 0, 0);
    if (!pl.split_k) return LYRA_E_UNSUPPORTED;
    if ((size_t)pl.ksplit * M * N * sizeof(float) >= (1ull << 31)) return LYRA_E_UNSUPPORTED;
    if (partials_bytes < (size_t)pl.ksplit * M * N * sizeof(float) || ((uintptr_t)partials % 16)) return LYRA_E_WORKSPACE;
    p.lhs = (const uint16_t*)lhs;
    p.rhs = (const uint8_t*)rhs;
    p.scale = rhs_scale;
    p.group_sizes = group_sizes;
    p.part = partials;
    p.M = M; p.G = 1; p.K = K; p.N = N;
    p.ksplit = pl.ksplit;
    p.kpart = pl.kpart;
    p.row_par = pl.row_par;
    p.row_block = pl.row_block;
    p.packed = layout;
    p.pspans = layout ? packed_spans(N, layout) : 0;
    p.lhs_tiled = lhs_tiled;
    if (rhs_dtype == LYRA_DTYPE_E5M2) return launch_split_k_fmt<2>(p, pl, (hipStream_t)stream);
    return fp8 ? launch_split_k_fmt<1>(p, pl, (hipStream_t)stream) : launch_split_k_fmt<0>(p, pl, (hipStream_t)stream);
}
#endif  // LYRA_GEMM_HAS_ENTRY
