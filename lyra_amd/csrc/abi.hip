// ABI housekeeping and a device self-check of the hardware behaviours the kernels assume.
#include "lyra_device.h"

namespace lyra {

// e4m3fn code -> float by the format's definition (s.eeee.mmm, bias 7, no infinities)
__device__ float e4m3fn_by_definition(int code) {
    const float sign = (code & 0x80) ? -1.f : 1.f;
    const int e = (code >> 3) & 0xF, m = code & 7;
    if (e == 0xF && m == 7) return __builtin_nanf("");
    if (e == 0) return sign * ldexpf((float)m / 8.f, -6);
    return sign * ldexpf(1.f + (float)m / 8.f, e - 7);
}

// e5m2 code -> float by the format's definition (s.eeeee.mm, bias 15, exponent 31 = infinity / NaN)
__device__ float e5m2_by_definition(int code) {
    const float sign = (code & 0x80) ? -1.f : 1.f;
    const int e = (code >> 2) & 0x1F, m = code & 3;
    if (e == 0x1F) return m ? __builtin_nanf("") : sign * __builtin_inff();
    if (e == 0) return sign * ldexpf((float)m / 4.f, -14);
    return sign * ldexpf(1.f + (float)m / 4.f, e - 15);
}

__global__ __launch_bounds__(64) void selftest_kernel(int32_t* report) {
    const int lane = threadIdx.x;
    const int x = lane & 15, kb = lane >> 4;
    int bad_mfma = 0, bad_cvt = 0, bad_cvt_bf16 = 0, bad_pack = 0, bad_perm = 0, bad_denorm = 0;

    // [0] accumulator layout of the 16x16x32 bf16 tile: A[i][k] = (i+1) if k == 0 else 0,
    //     B[k][j] = (j+1) if k == 0 else 0  ->  D[i][j] = (i+1)(j+1); slot 0 of k-group 0 plays k == 0.
    {
        Pack8 a, b;
        for (int i = 0; i < 4; ++i) a.u[i] = b.u[i] = 0u;
        if (kb == 0) {
            a.u[0] = pack_bf16((float)(x + 1), 0.f);
            b.u[0] = pack_bf16((float)(x + 1), 0.f);
        }
        f32x4 d = mfma_16x16x32(a.v, b.v, f32x4{0.f, 0.f, 0.f, 0.f});
        for (int r = 0; r < 4; ++r) bad_mfma += d[r] != (float)((4 * kb + r + 1) * (x + 1));
    }
    // [1] every k slot contributes once, with the same slot pairing in A and B:
    //     A[i][slot] = 1, B[slot][j] = w(slot) distinct powers of two -> D = sum of all w
    {
        Pack8 a, b;
        float want = 0.f;
        for (int g = 0; g < 4; ++g)
            for (int i = 0; i < 8; ++i) want += ldexpf(1.f, (8 * g + i) % 8 - 3) * (float)(g + 1);
        for (int i = 0; i < 4; ++i) {
            a.u[i] = pack_bf16(1.f, 1.f);
            b.u[i] = pack_bf16(ldexpf(1.f, (2 * i) % 8 - 3) * (float)(kb + 1), ldexpf(1.f, (2 * i + 1) % 8 - 3) * (float)(kb + 1));
        }
        f32x4 d = mfma_16x16x32(a.v, b.v, f32x4{0.f, 0.f, 0.f, 0.f});
        for (int r = 0; r < 4; ++r) bad_mfma += d[r] != want;
    }
    // [2] FP8 conversions over all 256 codes (4 per lane), both halves of the dword
    for (int q = 0; q < 4; ++q) {
        const int c0 = lane * 4 + q;
        const uint32_t w = (uint32_t)c0 | ((uint32_t)(255 - c0) << 8) | ((uint32_t)c0 << 16) | ((uint32_t)(255 - c0) << 24);
        const float e0 = e4m3fn_by_definition(c0), e1 = e4m3fn_by_definition(255 - c0);
        const f32x2 lo = fp8x2_to_f32(w, false), hi = fp8x2_to_f32(w, true);
        auto same = [](float a, float b) { return (a != a && b != b) || __float_as_uint(a) == __float_as_uint(b); };
        bad_cvt += !same(lo[0], e0) + !same(lo[1], e1) + !same(hi[0], e0) + !same(hi[1], e1);
        const uint32_t blo = fp8x2_to_bf16x2(w, false), bhi = fp8x2_to_bf16x2(w, true);
        auto bf = [](uint32_t v, int h) { return __uint_as_float((h ? (v >> 16) : (v & 0xFFFFu)) << 16); };
        bad_cvt_bf16 += !same(bf(blo, 0), e0) + !same(bf(blo, 1), e1) + !same(bf(bhi, 0), e0) + !same(bf(bhi, 1), e1);
        // the same for e5m2 (the finite codes: quantised data holds no others)
        const float f0 = e5m2_by_definition(c0), f1 = e5m2_by_definition(255 - c0);
        const bool fin0 = ((c0 >> 2) & 0x1F) != 0x1F, fin1 = (((255 - c0) >> 2) & 0x1F) != 0x1F;
        const f32x2 lo5 = codes2_to_f32<2>(w, false), hi5 = codes2_to_f32<2>(w, true);
        bad_cvt += (fin0 && (!same(lo5[0], f0) || !same(hi5[0], f0))) + (fin1 && (!same(lo5[1], f1) || !same(hi5[1], f1)));
        const uint32_t blo5 = codes2_to_bf16x2<2>(w, false), bhi5 = codes2_to_bf16x2<2>(w, true);
        bad_cvt_bf16 += (fin0 && (!same(bf(blo5, 0), f0) || !same(bf(bhi5, 0), f0))) + (fin1 && (!same(bf(blo5, 1), f1) || !same(bf(bhi5, 1), f1)));
        // and the float32 -> code direction on every finite code's own value (exact round trip)
        bad_cvt += (fin0 && f32_to_e5m2(f0) != (uint8_t)c0 && f0 != 0.f) + (c0 != 0x7F && c0 != 0xFF && e0 != 0.f && f32_to_e4m3fn(e0) != (uint8_t)c0);
    }
    // [3] float32 -> bf16 packing rounds to nearest even
    {
        const float v[4] = {1.00390625f, 1.01171875f, -3.0e-3f * (lane + 1), 65504.f + lane};
        for (int i = 0; i < 4; ++i) {
            uint32_t u = __float_as_uint(v[i]);
            const uint32_t want = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
            bad_pack += (pack_bf16(v[i], 0.f) & 0xFFFFu) != want;
            bad_pack += (pack_bf16(0.f, v[i]) >> 16) != want;
        }
    }
    // [4] half-word interleave used for bf16 operands
    {
        const uint32_t a = 0x11002200u + lane, b = 0x33004400u + lane;
        bad_perm += __builtin_amdgcn_perm(b, a, 0x05040100u) != ((b << 16) | (a & 0xFFFFu));
        bad_perm += __builtin_amdgcn_perm(b, a, 0x07060302u) != ((b & 0xFFFF0000u) | (a >> 16));
    }
    // [5] the smallest FP8 subnormal (2^-9, exact in bf16) survives the matrix core unflushed
    {
        Pack8 a, b;
        for (int i = 0; i < 4; ++i) a.u[i] = b.u[i] = 0u;
        if (kb == 0) {
            a.u[0] = fp8x2_to_bf16x2(0x01u, false);
            b.u[0] = pack_bf16(1.f, 0.f);
        }
        f32x4 d = mfma_16x16x32(a.v, b.v, f32x4{0.f, 0.f, 0.f, 0.f});
        for (int r = 0; r < 4; ++r) bad_denorm += d[r] != ldexpf(1.f, -9);
    }

    // [6] row exchanges: reductions over lanes {l, l^16, l^32, l^48}
    int bad_rows = 0;
    {
        const float v = (float)((lane * 37) % 101);
        float wmax = -1.f, wsum = 0.f;
        for (int g = 0; g < 4; ++g) {
            const float o = (float)(((16 * g + x) * 37) % 101);
            wmax = fmaxf(wmax, o);
            wsum += o;
        }
        bad_rows += group4_max(v) != wmax;
        bad_rows += group4_sum(v) != wsum;
    }

    int vals[7] = {bad_mfma, bad_cvt, bad_cvt_bf16, bad_pack, bad_perm, bad_denorm, bad_rows};
    for (int i = 0; i < 7; ++i) {
        const int v = wave_sum(vals[i]);
        if (lane == 0) report[i] = v;
    }
    if (lane == 0) report[7] = LYRA_ABI_VERSION;
}

}  // namespace lyra

extern "C" int lyra_abi_version(void) { return LYRA_ABI_VERSION; }

extern "C" const char* lyra_strerror(int code) {
    switch (code) {
        case LYRA_OK: return "ok";
        case LYRA_E_BADARG: return "bad argument (null pointer, non-positive size, inconsistent dtype/scale)";
        case LYRA_E_UNSUPPORTED: return "shape or dtype not supported by the gfx950 kernels";
        case LYRA_E_WORKSPACE: return "workspace missing, misaligned or too small";
        case LYRA_E_LAUNCH: return "HIP runtime refused the kernel launch";
        case LYRA_E_SCRATCH: return "the call needs more than the static scratch buffer (4 MiB): use the entry point that takes a workspace";
        default: return "unknown lyra error code";
    }
}

extern "C" int lyra_selftest(int32_t* report, lyra_stream_t stream) {
    if (!report) return LYRA_E_BADARG;
    hipLaunchKernelGGL(lyra::selftest_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, report);
    return hipGetLastError() == hipSuccess ? LYRA_OK : LYRA_E_LAUNCH;
}
