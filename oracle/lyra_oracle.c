/*
 * CPU oracle for Lyra's decode hot path, plain C (float32 arithmetic).
 *
 * TEST INFRASTRUCTURE ONLY: used by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py as the checker / timed CPU baseline.  The
 * shipped library never links or loads it.
 *
 * It restates the op sequence of the reference's plain-JAX decode path:
 *   attention  lyra/kernels/decode_attention.py:311-361 (+ :263-308 slab path,
 *              :392-395 "dequantise the whole cache first")
 *   gemm       lyra/kernels/decode_gemm.py:368-401 -> lyra/kernels/gemm.py:1575-1617
 *              ("dequantise every expert, ragged dot, bias, SwiGLU")
 *   formats    lyra/nn/quant.py:48-86
 * bf16 arrays cross this ABI as uint16 bit patterns, fp8 arrays as uint8 codes.
 * Pinning: tests check every function here against oracle/lyra_oracle.py, which in
 * turn is pinned against torch library routines and closed forms.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define LYRA_DECODE_BLOCK 128 /* decode_attention.py:29 */

/* ---- number formats ------------------------------------------------------------- */
/* Two 1-byte formats (lyra/nn/quant.py:10): index 1 = e4m3fn (s.eeee.mmm, bias 7, no infinities, S.1111.111 = NaN, max
 * 448), index 2 = e5m2 (s.eeeee.mm, bias 15, IEEE-like: exponent 31 = inf / NaN, max 57344).  Wherever this file takes a
 * flag "fp8" for an array, 0 means bf16 and 1 / 2 name the format of its codes. */
static float fp8_tables[3][256];
static int fp8_table_ready = 0;
#define fp8_table fp8_tables[1]

static void fp8_init(void) {
    if (fp8_table_ready) return;
    for (int code = 0; code < 256; ++code) {
        float sign = (code & 0x80) ? -1.0f : 1.0f;
        int e = (code >> 3) & 0xF, m = code & 7;
        float v;
        if (e == 0xF && m == 7) v = NAN;
        else if (e == 0) v = sign * ldexpf((float)m / 8.0f, -6);
        else v = sign * ldexpf(1.0f + (float)m / 8.0f, e - 7);
        fp8_tables[1][code] = v;
        int e5 = (code >> 2) & 0x1F, m5 = code & 3;
        if (e5 == 0x1F) v = m5 ? NAN : sign * INFINITY;
        else if (e5 == 0) v = sign * ldexpf((float)m5 / 4.0f, -14);
        else v = sign * ldexpf(1.0f + (float)m5 / 4.0f, e5 - 15);
        fp8_tables[2][code] = v;
    }
    fp8_table_ready = 1;
}

static inline float fp8_format_max(int fmt) { return fmt == 2 ? 57344.0f : 448.0f; }

float lyra_oracle_fp8_e5m2_to_f32(uint8_t code) {
    fp8_init();
    return fp8_tables[2][code];
}

/* float32 -> e5m2, round to nearest even; magnitudes that round above 57344 -> inf (0x7c), NaN -> 0x7f. */
uint8_t lyra_oracle_f32_to_fp8_e5m2(float x) {
    uint8_t sign = signbit(x) ? 0x80 : 0;
    if (isnan(x)) return sign | 0x7F;
    double a = fabs((double)x);
    if (a == 0.0) return sign;
    if (isinf(a)) return sign | 0x7C;
    int e;
    frexp(a, &e);
    e -= 1;
    if (e < -14) e = -14;
    if (e > 15) e = 15;
    double ulp = ldexp(1.0, e - 2);
    double val = nearbyint(a / ulp) * ulp; /* ties to even */
    if (val > 57344.0) return sign | 0x7C;
    if (val < ldexp(1.0, -14)) return sign | (uint8_t)nearbyint(val / ldexp(1.0, -16));
    int e2;
    frexp(val, &e2);
    e2 -= 1;
    int mant = (int)nearbyint((val / ldexp(1.0, e2) - 1.0) * 4.0);
    return sign | (uint8_t)(((e2 + 15) << 2) | mant);
}

float lyra_oracle_fp8_e4m3fn_to_f32(uint8_t code) {
    fp8_init();
    return fp8_table[code];
}

/* float32 -> e4m3fn, round to nearest even; |x| rounding above 448 or NaN -> 0x7f. */
uint8_t lyra_oracle_f32_to_fp8_e4m3fn(float x) {
    uint8_t sign = signbit(x) ? 0x80 : 0;
    if (isnan(x)) return sign | 0x7F;
    double a = fabs((double)x);
    if (a == 0.0) return sign;
    int e;
    frexp(a, &e); /* a = f * 2^e, f in [0.5,1) -> binade exponent e-1 */
    e -= 1;
    if (e < -6) e = -6;
    if (e > 8) e = 8;
    double ulp = ldexp(1.0, e - 3);
    double r = nearbyint(a / ulp); /* default rounding mode: ties to even */
    double val = r * ulp;
    if (val > 448.0) return sign | 0x7F;
    if (val < ldexp(1.0, -6)) return sign | (uint8_t)nearbyint(val / ldexp(1.0, -9));
    int e2;
    frexp(val, &e2);
    e2 -= 1;
    int mant = (int)nearbyint((val / ldexp(1.0, e2) - 1.0) * 8.0);
    return sign | (uint8_t)(((e2 + 7) << 3) | mant);
}

uint8_t lyra_oracle_f32_to_fp8_e4m3fn(float x);
static inline uint8_t f32_to_fp8(float x, int fmt) { return fmt == 2 ? lyra_oracle_f32_to_fp8_e5m2(x) : lyra_oracle_f32_to_fp8_e4m3fn(x); }

static inline float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if (isnan(f)) return (uint16_t)((u >> 16) | 0x40);
    uint32_t lsb = (u >> 16) & 1;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float bf16_round(float f) { return bf16_to_f32(f32_to_bf16(f)); }

uint16_t lyra_oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* ---- quantise one block-row (KV cache block (1,H)): quant.py:68-72 ------------------ */
void lyra_oracle_quantize_rows_fmt(const float* x, int64_t rows, int H, uint8_t* qval, float* scale, int fmt) {
    fp8_init();
    const float fmax = fp8_format_max(fmt);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* xr = x + r * H;
        float amax = 0.0f;
        for (int h = 0; h < H; ++h) amax = fmaxf(amax, fabsf(xr[h]));
        float s = amax > 0.0f ? amax / fmax : 1.0f;
        float inv = 1.0f / s;
        scale[r] = s;
        for (int h = 0; h < H; ++h) {
            float t = xr[h] * inv;
            t = fminf(fmaxf(t, -fmax), fmax);
            qval[r * H + h] = f32_to_fp8(t, fmt);
        }
    }
}

void lyra_oracle_quantize_rows(const float* x, int64_t rows, int H, uint8_t* qval, float* scale) {
    lyra_oracle_quantize_rows_fmt(x, rows, H, qval, scale, 1);
}

/* ---- quantise [G,K,N] weights with block (bk,bn): quant.py:48-75; scale is [G,K/bk,N/bn] ------- */
int lyra_oracle_quantize_blocks_fmt(const float* x, int G, int K, int N, int bk, int bn, uint8_t* qval, float* scale, int fmt) {
    if (G <= 0 || K <= 0 || N <= 0 || bk <= 0 || bn <= 0 || K % bk || N % bn) return -1;
    fp8_init();
    const float fmax = fp8_format_max(fmt);
    const int KB = K / bk, NB = N / bn;
#pragma omp parallel for collapse(3) schedule(static)
    for (int g = 0; g < G; ++g) {
        for (int kb = 0; kb < KB; ++kb) {
            for (int nb = 0; nb < NB; ++nb) {
                const size_t base = ((size_t)g * K + (size_t)kb * bk) * N + (size_t)nb * bn;
                float amax = 0.0f;
                for (int i = 0; i < bk; ++i)
                    for (int j = 0; j < bn; ++j) amax = fmaxf(amax, fabsf(x[base + (size_t)i * N + j]));
                const float s = amax > 0.0f ? amax / fmax : 1.0f;
                const float inv = 1.0f / s;
                scale[((size_t)g * KB + kb) * NB + nb] = s;
                for (int i = 0; i < bk; ++i)
                    for (int j = 0; j < bn; ++j) {
                        float t = x[base + (size_t)i * N + j] * inv;
                        t = fminf(fmaxf(t, -fmax), fmax);
                        qval[base + (size_t)i * N + j] = f32_to_fp8(t, fmt);
                    }
            }
        }
    }
    return 0;
}

int lyra_oracle_quantize_blocks(const float* x, int G, int K, int N, int bk, int bn, uint8_t* qval, float* scale) {
    return lyra_oracle_quantize_blocks_fmt(x, G, K, N, bk, bn, qval, scale, 1);
}

/* ---- window arithmetic: decode_attention.py:63-69, :277-280 -------------------------- */
int lyra_oracle_decode_window(int sliding_window) {
    int n_blocks = (sliding_window + LYRA_DECODE_BLOCK - 1 + LYRA_DECODE_BLOCK - 1) / LYRA_DECODE_BLOCK;
    return n_blocks * LYRA_DECODE_BLOCK;
}

int lyra_oracle_is_sw(int sliding_window, int kv_len) {
    return sliding_window > 0 && lyra_oracle_decode_window(sliding_window) < kv_len;
}

static int floordiv(int a, int b) { /* floor division as in XLA / Python */
    int q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
    return q;
}

int lyra_oracle_sliding_start(int position, int sliding_window, int kv_len) {
    int wlen = lyra_oracle_decode_window(sliding_window);
    int vis = position - sliding_window + 1;
    int start = floordiv(vis, LYRA_DECODE_BLOCK) * LYRA_DECODE_BLOCK;
    if (start < 0) start = 0;
    if (start > kv_len - wlen) start = kv_len - wlen;
    return start;
}

/*
 * Decode attention, reference op order.  kv_fp8 != 0: k,v are uint8 [B,K,S,H] with
 * f32 scales [B,K,S]; else uint16 bf16 [B,K,S,H].  ref_rounding != 0 rounds where the
 * JAX code holds bf16 (dequantised cache, qk logits, output); 0 = pure float32.
 * position has B entries.  gate (nullable) is float32 [B,N].  out is float32 [B,N,H].
 * Returns 0, or -1 on bad arguments.
 */
int lyra_oracle_decode_attention(const uint16_t* q, const void* k, const void* v, const float* k_scale,
                                 const float* v_scale, const float* sinks, const int32_t* position,
                                 const float* gate, float* out, int B, int N, int K, int S, int H, float sm_scale,
                                 int sliding_window, int kv_fp8, int ref_rounding) {
    if (B <= 0 || N <= 0 || K <= 0 || S <= 0 || H <= 0 || N % K) return -1;
    fp8_init();
    const int G = N / K;
    const int slab = lyra_oracle_is_sw(sliding_window, S);
    const int wlen = slab ? lyra_oracle_decode_window(sliding_window) : S;
    int status = 0;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b) {
        for (int kh = 0; kh < K; ++kh) {
            const int pos = position[b];
            const int start = slab ? lyra_oracle_sliding_start(pos, sliding_window, S) : 0;
            float* kd = (float*)malloc((size_t)wlen * H * sizeof(float));
            float* vd = (float*)malloc((size_t)wlen * H * sizeof(float));
            float* qk = (float*)malloc((size_t)wlen * sizeof(float));
            if (!kd || !vd || !qk) {
                status = -1;
                free(kd); free(vd); free(qk);
                continue;
            }
            /* step 1: materialise the (slab of the) cache as bf16 - decode_attention.py:327-330 */
            const size_t base = ((size_t)b * K + kh) * S;
            for (int j = 0; j < wlen; ++j) {
                const size_t row = base + start + j;
                for (int h = 0; h < H; ++h) {
                    float kv_, vv_;
                    if (kv_fp8) {
                        kv_ = fp8_tables[kv_fp8 == 2 ? 2 : 1][((const uint8_t*)k)[row * H + h]] * k_scale[row];
                        vv_ = fp8_tables[kv_fp8 == 2 ? 2 : 1][((const uint8_t*)v)[row * H + h]] * v_scale[row];
                        if (ref_rounding) { kv_ = bf16_round(kv_); vv_ = bf16_round(vv_); }
                    } else {
                        kv_ = bf16_to_f32(((const uint16_t*)k)[row * H + h]);
                        vv_ = bf16_to_f32(((const uint16_t*)v)[row * H + h]);
                    }
                    kd[(size_t)j * H + h] = kv_;
                    vd[(size_t)j * H + h] = vv_;
                }
            }
            for (int g = 0; g < G; ++g) {
                const int n = kh * G + g;
                const uint16_t* qn = q + ((size_t)b * N + n) * H;
                const float sink = sinks[n];
                /* step 2: logits + mask - :343-346 / :290-293 */
                float vmax = sink;
                for (int j = 0; j < wlen; ++j) {
                    const int key = start + j;
                    int vis = key <= pos;
                    if (sliding_window > 0) vis = vis && (key > pos - sliding_window);
                    float s;
                    if (vis) {
                        float acc = 0.0f;
                        for (int h = 0; h < H; ++h) acc += bf16_to_f32(qn[h]) * kd[(size_t)j * H + h];
                        s = ref_rounding ? bf16_round(bf16_round(acc) * sm_scale) : acc * sm_scale;
                    } else {
                        s = -INFINITY;
                    }
                    qk[j] = s;
                    vmax = fmaxf(vmax, s);
                }
                /* step 3: sink softmax - :348-355 */
                float denom = expf(sink - vmax);
                for (int j = 0; j < wlen; ++j) {
                    qk[j] = expf(qk[j] - vmax);
                    denom += qk[j];
                }
                const float norm = 1.0f / denom;
                /* step 4: weighted values - :357-359 */
                float* on = out + ((size_t)b * N + n) * H;
                for (int h = 0; h < H; ++h) on[h] = 0.0f;
                for (int j = 0; j < wlen; ++j) {
                    const float a = qk[j] * norm;
                    if (a == 0.0f) continue;
                    for (int h = 0; h < H; ++h) on[h] += a * vd[(size_t)j * H + h];
                }
                for (int h = 0; h < H; ++h) {
                    float o = ref_rounding ? bf16_round(on[h]) : on[h];
                    if (gate) {
                        o *= gate[(size_t)b * N + n];
                        if (ref_rounding) o = bf16_round(o);
                    }
                    on[h] = o;
                }
            }
            free(kd); free(vd); free(qk);
        }
    }
    return status;
}

/*
 * Decode GEMM, reference op order.  rhs_fp8 != 0: rhs uint8 [G,K,N] with f32 scales
 * [G,K/bk,N/bn]; else uint16 bf16 [G,K,N].  lhs uint16 bf16 [M,K]; bias (nullable) f32 [G,N];
 * out float32 [M, fused_swiglu ? N/2 : N].  Every expert is dequantised (decode_gemm.py:431)
 * whether or not it has rows; "scratch" must hold G*K*N floats (caller-provided so the
 * timed region can exclude the allocation).  Returns 0 or -1.
 */
int lyra_oracle_decode_gemm(const uint16_t* lhs, const void* rhs, const float* rhs_scale, int bk, int bn,
                            const int32_t* group_sizes, const float* bias, float* out, float* scratch, int M, int G,
                            int K, int N, int rhs_fp8, int fused_swiglu, float beta, float limit, int ref_rounding) {
    if (M < 0 || G <= 0 || K <= 0 || N <= 0) return -1;
    if (rhs_fp8 && (bk <= 0 || bn <= 0 || K % bk || N % bn)) return -1;
    if (fused_swiglu && (N % 2)) return -1;
    fp8_init();
    const int KB = rhs_fp8 ? K / bk : 0, NB = rhs_fp8 ? N / bn : 0;
    /* ref_rounding: 0 = float32 throughout, 1 = dequantised weights and outputs rounded to bf16 as the JAX code holds them,
       2 = only the dequantised weights rounded (quant.py:85), product and epilogue in float32 */
    const int round_out = ref_rounding == 1;
    /* step 1: dequantise ALL experts to lhs.dtype */
#pragma omp parallel for collapse(2) schedule(static)
    for (int g = 0; g < G; ++g) {
        for (int kk = 0; kk < K; ++kk) {
            const size_t row = ((size_t)g * K + kk) * N;
            for (int n = 0; n < N; ++n) {
                float w;
                if (rhs_fp8) {
                    w = fp8_tables[rhs_fp8 == 2 ? 2 : 1][((const uint8_t*)rhs)[row + n]] * rhs_scale[((size_t)g * KB + kk / bk) * NB + n / bn];
                    if (ref_rounding) w = bf16_round(w);
                } else {
                    w = bf16_to_f32(((const uint16_t*)rhs)[row + n]);
                }
                scratch[row + n] = w;
            }
        }
    }
    /* expert id per row: gemm.py:450-456 (rows at or beyond sum(group_sizes) get id G-1) */
    int* ids = (int*)malloc(sizeof(int) * (size_t)(M > 0 ? M : 1));
    if (!ids) return -1;
    int total = 0;
    for (int g = 0; g < G; ++g)
        for (int i = 0; i < group_sizes[g] && total < M; ++i) ids[total++] = g;
    const int valid = total;
    for (int r = valid; r < M; ++r) ids[r] = G - 1;
    const int NO = fused_swiglu ? N / 2 : N;
#pragma omp parallel
    {
        float* t = (float*)malloc(sizeof(float) * (size_t)N);
#pragma omp for schedule(dynamic)
        for (int r = 0; r < M; ++r) {
            const int g = ids[r];
            for (int n = 0; n < N; ++n) t[n] = 0.0f;
            if (r < valid) { /* step 2: ragged dot, f32 accumulate - gemm.py:1606-1607 */
                const float* w = scratch + (size_t)g * K * N;
                for (int kk = 0; kk < K; ++kk) {
                    const float x = bf16_to_f32(lhs[(size_t)r * K + kk]);
                    const float* wr = w + (size_t)kk * N;
                    for (int n = 0; n < N; ++n) t[n] += x * wr[n];
                }
            }
            if (bias) /* step 3: :1608-1612 */
                for (int n = 0; n < N; ++n) t[n] += bias[(size_t)g * N + n];
            float* o = out + (size_t)r * NO;
            if (fused_swiglu) { /* step 4: common.py:98-114 */
                for (int n = 0; n < NO; ++n) {
                    float glu = fminf(t[n], limit);
                    float lin = fminf(fmaxf(t[NO + n], -limit), limit);
                    float y = (lin + 1.0f) * (glu * (1.0f / (1.0f + expf(-beta * glu))));
                    o[n] = round_out ? bf16_round(y) : y;
                }
            } else {
                for (int n = 0; n < NO; ++n) o[n] = round_out ? bf16_round(t[n]) : t[n];
            }
        }
        free(t);
    }
    free(ids);
    return 0;
}

int lyra_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
