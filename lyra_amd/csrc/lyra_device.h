// Device-side helpers shared by the gfx950 decode kernels: vector types, FP8/BF16 conversions,
// the 16x16x32 BF16 matrix-core tile and wavefront (64-lane) reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lyra_hip.h"

namespace lyra {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// A buffer-load lane offset beyond any buffer descriptor used here (all are shorter than 2 GiB; the constant
// offsets added to it stay far below 4 GiB): such a load returns zeros without touching memory.
constexpr int kNoLoad = (int)0x80000000u;
// Cache policy of buffer loads that stream data read once per launch (KV cache, weights): non-temporal.  A plain linear
// read of 277 MB runs at 7.1 TB/s with it and at 6.3 TB/s without.
constexpr int kStream = 2;

// D(16x16,f32) += A(16x32,bf16) * B(32x16,bf16).  Lane l supplies row (l & 15) of A and column
// (l & 15) of B, each as the 8 consecutive k-slots of k-group (l >> 4); both operands use the same
// slot -> k mapping, so only "same k in the same slot" matters.  Lane l receives D[4*(l>>4)+r][l&15]
// in element r of the result.
__device__ __forceinline__ f32x4 mfma_16x16x32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

union Pack8 {
    bf16x8 v;
    uint32_t u[4];
    bf16x2 h[4];
};

// two e4m3fn codes (low or high half of a dword) -> two float32, exact
__device__ __forceinline__ f32x2 fp8x2_to_f32(uint32_t w, bool hi) {
    return hi ? __builtin_amdgcn_cvt_pk_f32_fp8(w, true) : __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
}

// two float32 -> packed bf16x2 (round to nearest even), one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    bf16x2 r;
    r[0] = (__bf16)lo;
    r[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, r);
}

// two e4m3fn codes -> packed bf16x2 in one instruction (the conversion is exact; scale 1)
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t w, bool hi) {
    bf16x2 r = hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)
                  : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
    return __builtin_bit_cast(uint32_t, r);
}

// The same for the two 1-byte formats the kernels read, picked at compile time.  FMT 1: e4m3fn; FMT 2: e5m2 (OCP FP8 E5M2:
// 5 exponent bits, 2 mantissa bits, max 57344; its infinities and NaNs never occur in quantised data, which is clipped).
template <int FMT>
__device__ __forceinline__ uint32_t codes2_to_bf16x2(uint32_t w, bool hi) {
    static_assert(FMT == 1 || FMT == 2, "1-byte formats: 1 = e4m3fn, 2 = e5m2");
    if constexpr (FMT == 2) {
        bf16x2 r = hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(w, 1.0f, true)
                      : __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(w, 1.0f, false);
        return __builtin_bit_cast(uint32_t, r);
    } else {
        return fp8x2_to_bf16x2(w, hi);
    }
}
template <int FMT>
__device__ __forceinline__ f32x2 codes2_to_f32(uint32_t w, bool hi) {
    static_assert(FMT == 1 || FMT == 2, "1-byte formats: 1 = e4m3fn, 2 = e5m2");
    if constexpr (FMT == 2) return hi ? __builtin_amdgcn_cvt_pk_f32_bf8(w, true) : __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
    else return fp8x2_to_f32(w, hi);
}

// 8 consecutive 1-byte codes (two dwords) -> bf16x8 in the same order
template <int FMT = 1>
__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(uint32_t w0, uint32_t w1) {
    Pack8 p;
    p.u[0] = codes2_to_bf16x2<FMT>(w0, false);
    p.u[1] = codes2_to_bf16x2<FMT>(w0, true);
    p.u[2] = codes2_to_bf16x2<FMT>(w1, false);
    p.u[3] = codes2_to_bf16x2<FMT>(w1, true);
    return p.v;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    __bf16 h = (__bf16)f;
    return __builtin_bit_cast(uint16_t, h);
}

// a float32 value rounded to bf16 and back (where the JAX code holds a bf16 array)
__device__ __forceinline__ float bf16r(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// float32 -> e4m3fn code, round to nearest even; |v| <= 448 by construction
__device__ __forceinline__ uint8_t f32_to_e4m3fn(float v) {
    const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(v, 0.f, 0, false);
    return (uint8_t)(packed & 0xFF);
}

// float32 -> e5m2 code, round to nearest even; |v| <= 57344 by construction
__device__ __forceinline__ uint8_t f32_to_e5m2(float v) {
    const int packed = __builtin_amdgcn_cvt_pk_bf8_f32(v, 0.f, 0, false);
    return (uint8_t)(packed & 0xFF);
}

// Largest finite value of a 1-byte format (jnp.finfo(dtype).max in lyra/nn/quant.py:68) and the quantiser for it.
__device__ __forceinline__ float fp8_format_max(bool e5m2) { return e5m2 ? 57344.f : 448.f; }
__device__ __forceinline__ uint8_t f32_to_fp8_code(float v, bool e5m2) { return e5m2 ? f32_to_e5m2(v) : f32_to_e4m3fn(v); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Exchange between the four 16-lane rows of a wavefront without going through LDS.
// v_permlane32_swap swaps the upper 32 lanes of its first operand with the lower 32 of its second;
// fed the same value twice it returns {x[l & 31], x[l | 32]}: both halves' values in every lane.
// v_permlane16_swap does the same for odd/even rows of 16: {x[l & ~16], x[l | 16]}.
__device__ __forceinline__ void both_halves32(float x, float& a, float& b) {
    const uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void both_rows16(float x, float& a, float& b) {
    const uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
}
// reductions over lanes l, l^16, l^32, l^48 (the four rows that share l & 15)
__device__ __forceinline__ float group4_max(float x) {
    float a, b;
    both_halves32(x, a, b);
    x = fmaxf(a, b);
    both_rows16(x, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float group4_sum(float x) {
    float a, b;
    both_halves32(x, a, b);
    x = a + b;
    both_rows16(x, a, b);
    return a + b;
}

// Device-wide visible stores and loads (write-through / cache-bypassing at agent scope).  Producers publish
// with store_agent + wait_all_memory, then bump an arrival counter with add_agent; a consumer that saw the
// final count reads with load_agent.  No cache-wide write-back or invalidate is involved.
__device__ __forceinline__ void store_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int add_agent(int* p, int v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(int* p, int v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Stores of results that a later kernel reads.  Every XCD has its own L2, so what a kernel leaves dirty there is written
// back when the kernel ends, and the next kernel waits for that; a store at agent scope is written through as it is
// issued, while the kernel still has work to do.
__device__ __forceinline__ void store_through(uint16_t* p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_through(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_through(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_through(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_through(u32x2* p, u32x2 v) {
    __hip_atomic_store((unsigned long long*)p, (unsigned long long)v[0] | ((unsigned long long)v[1] << 32), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_through(u32x4* p, u32x4 v) {
    store_through((u32x2*)p, u32x2{v[0], v[1]});
    store_through((u32x2*)p + 1, u32x2{v[2], v[3]});
}
__device__ __forceinline__ void store_through(f32x2* p, f32x2 v) { store_through((u32x2*)p, u32x2{__float_as_uint(v[0]), __float_as_uint(v[1])}); }
__device__ __forceinline__ void store_through(f32x4* p, f32x4 v) {
    store_through((u32x4*)p, u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])});
}
// ... and through a buffer descriptor on a wave-uniform base pointer (offsets in bytes, below 2 GB): 4, 8 and 16 bytes.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t through_rsrc(void* base) {
    return __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7FFFFFFFu, 0x00020000);
}
__device__ __forceinline__ void store_through(void* base, size_t off, uint32_t v) {
    __builtin_amdgcn_raw_buffer_store_b32(v, through_rsrc(base), (int)off, 0, 16);
}
__device__ __forceinline__ void store_through(void* base, size_t off, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, through_rsrc(base), (int)off, 0, 16);
}
__device__ __forceinline__ void store_through(void* base, size_t off, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, through_rsrc(base), (int)off, 0, 16);
}
__device__ __forceinline__ void store_through(void* base, size_t off, f32x2 v) {
    store_through(base, off, u32x2{__float_as_uint(v[0]), __float_as_uint(v[1])});
}
__device__ __forceinline__ void store_through(void* base, size_t off, f32x4 v) {
    store_through(base, off, u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])});
}
__device__ __forceinline__ void wait_all_memory() { __builtin_amdgcn_s_waitcnt(0); }
// 16-byte forms of store_agent / load_agent through a buffer descriptor (cache-policy bit 4 = sc1: agent scope on gfx950).
__device__ __forceinline__ void store_agent_b128(__amdgpu_buffer_rsrc_t rsrc, int voff, f32x4 v) {
    u32x4 d;
#pragma unroll
    for (int i = 0; i < 4; ++i) d[i] = __float_as_uint(v[i]);
    __builtin_amdgcn_raw_buffer_store_b128(d, rsrc, voff, 0, 16);
}
__device__ __forceinline__ f32x4 load_agent_b128(__amdgpu_buffer_rsrc_t rsrc, int voff) {
    const u32x4 d = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 0, 16);
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(d[i]);
    return v;
}

// Workgroup barrier for data exchanged through LDS: waits for this wavefront's LDS operations only.  __syncthreads() also
// waits for every global load the wavefront has in flight, which empties the prefetch queue of a streaming kernel.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Reductions over the 64 lanes of a wavefront, result in every lane: within a row of 16 lanes by DPP (lane pairs, quads,
// mirrored halves of 8, mirrored row), then across the four rows by the lane swaps above.  A dozen ALU instructions; the
// same butterfly through __shfl_xor goes through LDS six times (~0.3 us each time a small kernel reduces a row).
template <int CTRL> __device__ __forceinline__ int dpp_row(int x) { return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xF, 0xF, true); }
template <int CTRL> __device__ __forceinline__ float dpp_row(float x) { return __uint_as_float((uint32_t)dpp_row<CTRL>((int)__float_as_uint(x))); }
__device__ __forceinline__ float row16_max(float x) {  // over the 16 lanes of a row, result in each of them
    x = fmaxf(x, dpp_row<0xB1>(x));   // quad_perm [1, 0, 3, 2]
    x = fmaxf(x, dpp_row<0x4E>(x));   // quad_perm [2, 3, 0, 1]
    x = fmaxf(x, dpp_row<0x141>(x));  // row_half_mirror
    return fmaxf(x, dpp_row<0x140>(x));  // row_mirror
}
__device__ __forceinline__ float wave_max(float x) { return group4_max(row16_max(x)); }
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_row<0xB1>(x);
    x += dpp_row<0x4E>(x);
    x += dpp_row<0x141>(x);
    x += dpp_row<0x140>(x);
    return group4_sum(x);
}
__device__ __forceinline__ int wave_sum(int x) {
    x += dpp_row<0xB1>(x);
    x += dpp_row<0x4E>(x);
    x += dpp_row<0x141>(x);
    x += dpp_row<0x140>(x);
    const uint32_t u = (uint32_t)x;
    auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const uint32_t t = h[0] + h[1];
    auto r = __builtin_amdgcn_permlane16_swap(t, t, false, false);
    return (int)(r[0] + r[1]);
}
// The same butterfly for a (value, index) pair with a caller's rule: take(v, i, ov, oi) replaces (v, i) by (ov, oi) where
// the other pair wins.  The rule must not depend on the order in which pairs meet (a total order with ties broken by index).
// `lanes`: how many neighbouring lanes (a power of two, aligned) form one group; 64 = the whole wavefront.
template <typename Take>
__device__ __forceinline__ void wave_best(float& v, int& i, Take take, int lanes = 64) {
    if (lanes > 1) take(v, i, dpp_row<0xB1>(v), dpp_row<0xB1>(i));
    if (lanes > 2) take(v, i, dpp_row<0x4E>(v), dpp_row<0x4E>(i));
    if (lanes > 4) take(v, i, dpp_row<0x141>(v), dpp_row<0x141>(i));
    if (lanes > 8) take(v, i, dpp_row<0x140>(v), dpp_row<0x140>(i));
    if (lanes > 16) {
        auto rv = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        auto ri = __builtin_amdgcn_permlane16_swap((uint32_t)i, (uint32_t)i, false, false);
        v = __uint_as_float(rv[0]), i = (int)ri[0];
        take(v, i, __uint_as_float(rv[1]), (int)ri[1]);
    }
    if (lanes > 32) {
        auto hv = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        auto hi = __builtin_amdgcn_permlane32_swap((uint32_t)i, (uint32_t)i, false, false);
        v = __uint_as_float(hv[0]), i = (int)hi[0];
        take(v, i, __uint_as_float(hv[1]), (int)hi[1]);
    }
}
// Inclusive prefix sum over the lanes of a wavefront: within rows of 16 by shifted DPP reads, then the last lane of a row
// (of the first half) is added to the rows behind it.
__device__ __forceinline__ int wave_scan_inclusive(int x) {
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false);  // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false);  // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false);  // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false);  // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
    return x;
}

// QK norm (when `norm`) and rotary embedding of one head row held as two halves per lane (a: element `lane`, c: element
// `lane + H/2`), rounded to bf16 wherever the JAX code holds a bf16 array (lyra/model.py:183-191, 315-323).  Every lane of
// the wavefront calls it (idle lanes with zeros).  One definition, with the contraction of products and sums into fused
// multiply-adds switched off, so that every kernel that uses it rounds identically.
__device__ __forceinline__ void head_norm_rope(float& a, float& c, bool norm, float ns_a, float ns_c, float cs, float sn,
                                               float eps, int H) {
#pragma clang fp contract(off)
    if (norm) {
        const float ss = wave_sum(a * a + c * c);
        const float inv = rsqrtf(ss / (float)H + eps);
        a = bf16r(a * inv * ns_a);
        c = bf16r(c * inv * ns_c);
    }
    const float ra = bf16r(a * cs - c * sn), rc = bf16r(c * cs + a * sn);
    a = ra;
    c = rc;
}

}  // namespace lyra
