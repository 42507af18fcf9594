/*
 * CPU oracle for the tensor programs of the Heron hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It restates, in plain C, the mathematics
 * that the reference defines for its operators, so that the HIP kernels can be
 * checked against it.  It is used only by the test-suite, by the smoke check
 * and by the `cpu_baseline` leg of the benchmark; the product path never
 * calls it.
 *
 * What each function follows in the reference (paths relative to the
 * reference checkout):
 *   orc_gemm_u8s8s32_scalar   ops/x86/dense.py:6-32       C[i,j] = sum_k i32(A[i,k]) * i32(B[j,k])
 *   orc_gemm_u8s8s32_dlboost  ops/x86/dense.py:21-26 + schedule/sched_op/cpu_operator.py:84-117,17-27
 *                             (16 output lanes x 4 k per `vpdpbusd`, parallel fused outer tiles)
 *   orc_bmm_u8s8s32_scalar    ops/x86/batch_matmul.py:6-34
 *   orc_gemm_f32              ops/cuda/dense.py:4-54       C[i,j] = sum_k A[i,k] * B[j,k]   (B stored (N,K))
 *   orc_bmm_f32               ops/cuda/batch_matmul.py:5-56
 *   orc_conv2d_nhwc_u8s8s32   ops/x86/conv2d_int8.py:31-109  (filter KRSC, output (N,HO,WO,CO))
 *   orc_conv2d_nhwc_u8s8s32_blocked  the same operator with the reference's own operand shapes: filter
 *                             (CO/b, KH, KW, CI/4, b, 4), output (N,HO,WO,CO/b,b)   (conv2d_int8.py:50-93)
 *   orc_conv2d_nhwc_f32       ops/cuda/conv2d.py:137-232   (filter taken as KRSC = (CO,KH,KW,CI); the
 *                             reference stores HWIO (KH,KW,CI,CO) - same sum, different weight order)
 *
 * The arithmetic of the reference itself lives in TVM-generated code (TVM is
 * not part of the reference checkout and cannot be built here), and the
 * reference holds no golden output for any of these operators, so the
 * functions are pinned by independent checks in tests/test_oracle.py: brute
 * force Python loops on tiny inputs, numpy int64 matmul, the hardware
 * `vpdpbusd` path against the scalar path, torch's CPU conv2d, extreme-value
 * closed forms, linearity/identity invariants.
 *
 * Floating point references take fp32 arrays (the fp16 inputs widened
 * exactly) and accumulate in double, then round once to fp32.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__x86_64__)
#include <immintrin.h>
#endif

#define ORC_API __attribute__((visibility("default")))

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ops/x86/dense.py:13-18 - plain triple loop, int32 accumulate. */
ORC_API void orc_gemm_u8s8s32_scalar(const uint8_t* A, const int8_t* B, int32_t* C,
                                     int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            int32_t acc = 0;
            for (int64_t k = 0; k < K; ++k)
                acc += (int32_t)A[i * K + k] * (int32_t)B[j * K + k];
            C[i * N + j] = acc;
        }
}

/* ops/x86/batch_matmul.py:14-19 */
ORC_API void orc_bmm_u8s8s32_scalar(const uint8_t* A, const int8_t* B, int32_t* C,
                                    int64_t batch, int64_t M, int64_t N, int64_t K) {
    for (int64_t b = 0; b < batch; ++b)
        orc_gemm_u8s8s32_scalar(A + b * M * K, B + b * N * K, C + b * M * N, M, N, K);
}

/* 1 when the running CPU executes AVX512-VNNI (`vpdpbusd zmm`). */
ORC_API int orc_has_vnni(void) {
#if defined(__x86_64__)
    __builtin_cpu_init();
    return __builtin_cpu_supports("avx512vnni") && __builtin_cpu_supports("avx512bw");
#else
    return 0;
#endif
}

#if defined(__x86_64__)
/*
 * The DL Boost structure: the spatial axis j is split by 16 and the reduce
 * axis k by 4 (cpu_operator.py:84-117), and the innermost 16x4 block is one
 * `vpdpbusd`: out[0:16] += sum_{t<4} u8 a[t] * s8 w[j][t]  (dense.py:25,
 * intrinsic dot_16x1x16_uint8_int8_int32_cascadelake, non saturating).
 * The 16x4 weight block must be contiguous for the 64-byte load, so B (N,K)
 * is re-packed to [N/16][K/4][16][4] first.
 */
__attribute__((target("avx512f,avx512bw,avx512vnni")))
static void pack_b_16x4(const int8_t* B, int8_t* P, int64_t N, int64_t K) {
    const int64_t nb = N / 16, kb = K / 4;
#pragma omp parallel for schedule(static)
    for (int64_t jb = 0; jb < nb; ++jb)
        for (int64_t k4 = 0; k4 < kb; ++k4) {
            int8_t* dst = P + (jb * kb + k4) * 64;
            for (int j = 0; j < 16; ++j)
                memcpy(dst + j * 4, B + (jb * 16 + j) * K + k4 * 4, 4);
        }
}

#define ORC_MR 8
__attribute__((target("avx512f,avx512bw,avx512vnni")))
static void micro_8x32(const uint8_t* A, int64_t lda, const int8_t* P0, const int8_t* P1,
                       int64_t kb, int32_t* C, int64_t ldc, int rows) {
    __m512i acc0[ORC_MR], acc1[ORC_MR];
    for (int r = 0; r < ORC_MR; ++r) { acc0[r] = _mm512_setzero_si512(); acc1[r] = _mm512_setzero_si512(); }
    for (int64_t k4 = 0; k4 < kb; ++k4) {
        const __m512i w0 = _mm512_loadu_si512((const void*)(P0 + k4 * 64));
        const __m512i w1 = _mm512_loadu_si512((const void*)(P1 + k4 * 64));
        for (int r = 0; r < ORC_MR; ++r) {
            int32_t a4;
            memcpy(&a4, A + (r < rows ? r : 0) * lda + k4 * 4, 4);
            const __m512i a = _mm512_set1_epi32(a4);
            acc0[r] = _mm512_dpbusd_epi32(acc0[r], a, w0);
            acc1[r] = _mm512_dpbusd_epi32(acc1[r], a, w1);
        }
    }
    for (int r = 0; r < rows; ++r) {
        _mm512_storeu_si512((void*)(C + r * ldc), acc0[r]);
        _mm512_storeu_si512((void*)(C + r * ldc + 16), acc1[r]);
    }
}

__attribute__((target("avx512f,avx512bw,avx512vnni")))
static void gemm_vnni_packed(const uint8_t* A, const int8_t* P, int32_t* C,
                             int64_t M, int64_t N, int64_t K) {
    const int64_t kb = K / 4, nb32 = N / 32, mb = (M + ORC_MR - 1) / ORC_MR;
    /* fused outer tiles run in parallel (cpu_operator.py:17-27) */
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t jb = 0; jb < nb32; ++jb)
        for (int64_t ib = 0; ib < mb; ++ib) {
            const int64_t i0 = ib * ORC_MR;
            const int rows = (int)((M - i0) < ORC_MR ? (M - i0) : ORC_MR);
            micro_8x32(A + i0 * K, K, P + (2 * jb) * kb * 64, P + (2 * jb + 1) * kb * 64, kb,
                       C + i0 * N + jb * 32, N, rows);
        }
}
#endif

/*
 * Persistent packed-weight handle so that a benchmark can time the multiply
 * without the one-off re-pack (as a weight reorder would be in deployment).
 */
typedef struct { int8_t* P; int64_t N, K; } orc_packed_b;

ORC_API void* orc_pack_b(const int8_t* B, int64_t N, int64_t K) {
#if defined(__x86_64__)
    if (!orc_has_vnni() || N % 32 || K % 4) return NULL;
    orc_packed_b* h = (orc_packed_b*)malloc(sizeof(orc_packed_b));
    if (!h) return NULL;
    h->P = (int8_t*)aligned_alloc(64, (size_t)N * (size_t)K);
    if (!h->P) { free(h); return NULL; }
    h->N = N; h->K = K;
    pack_b_16x4(B, h->P, N, K);
    return h;
#else
    (void)B; (void)N; (void)K;
    return NULL;
#endif
}

ORC_API void orc_free_b(void* handle) {
    orc_packed_b* h = (orc_packed_b*)handle;
    if (h) { free(h->P); free(h); }
}

/* returns 0 on success, -1 when the handle does not fit (caller uses the scalar path) */
ORC_API int orc_gemm_u8s8s32_packed(const uint8_t* A, const void* handle, int32_t* C,
                                    int64_t M, int64_t N, int64_t K) {
#if defined(__x86_64__)
    const orc_packed_b* h = (const orc_packed_b*)handle;
    if (!h || h->N != N || h->K != K) return -1;
    gemm_vnni_packed(A, h->P, C, M, N, K);
    return 0;
#else
    (void)A; (void)handle; (void)C; (void)M; (void)N; (void)K;
    return -1;
#endif
}

/*
 * DL Boost path end to end.  Returns the ISA path taken:
 * 2 = avx512-vnni micro-kernel, 0 = scalar fallback (no VNNI, or N%32 / K%4).
 */
ORC_API int orc_gemm_u8s8s32_dlboost(const uint8_t* A, const int8_t* B, int32_t* C,
                                     int64_t M, int64_t N, int64_t K) {
    void* h = orc_pack_b(B, N, K);
    if (h) {
        orc_gemm_u8s8s32_packed(A, h, C, M, N, K);
        orc_free_b(h);
        return 2;
    }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        orc_gemm_u8s8s32_scalar(A + i * K, B, C + i * N, 1, N, K);
    return 0;
}

/* ops/cuda/dense.py:11-17, B stored (N,K); double accumulate, one rounding to fp32. */
ORC_API void orc_gemm_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            const float* a = A + i * K;
            const float* b = B + j * K;
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) acc += (double)a[k] * (double)b[k];
            C[i * N + j] = (float)acc;
        }
}

/* ops/cuda/batch_matmul.py:12-19 */
ORC_API void orc_bmm_f32(const float* A, const float* B, float* C,
                         int64_t batch, int64_t M, int64_t N, int64_t K) {
    for (int64_t b = 0; b < batch; ++b)
        orc_gemm_f32(A + b * M * K, B + b * N * K, C + b * M * N, M, N, K);
}

/*
 * ops/cuda/conv2d.py:166-196.  In (N,H,W,CI), Wt (CO,KH,KW,CI), Out (N,HO,WO,CO),
 * HO = (H - ((KH-1)*dil+1) + 2*pad)/stride + 1 (conv2d.py:168-175); taps that fall into
 * the zero padding contribute nothing.  stride/pad/dil act on the height, the *_w values on the width
 * (conv2d.py:143-153 accepts an int or a pair for each).
 */
ORC_API void orc_conv2d_nhwc_f32(const float* In, const float* Wt, float* Out,
                                 int64_t N, int64_t H, int64_t W, int64_t CI, int64_t CO,
                                 int64_t KH, int64_t KW, int64_t stride, int64_t stride_w, int64_t pad, int64_t pad_w,
                                     int64_t dil, int64_t dil_w) {
    const int64_t HO = (H - ((KH - 1) * dil + 1) + 2 * pad) / stride + 1;
    const int64_t WO = (W - ((KW - 1) * dil_w + 1) + 2 * pad_w) / stride_w + 1;
#pragma omp parallel for collapse(3) schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t y = 0; y < HO; ++y)
            for (int64_t x = 0; x < WO; ++x)
                for (int64_t f = 0; f < CO; ++f) {
                    double acc = 0.0;
                    for (int64_t ry = 0; ry < KH; ++ry) {
                        const int64_t iy = y * stride + ry * dil - pad;
                        if (iy < 0 || iy >= H) continue;
                        for (int64_t rx = 0; rx < KW; ++rx) {
                            const int64_t ix = x * stride_w + rx * dil_w - pad_w;
                            if (ix < 0 || ix >= W) continue;
                            const float* a = In + ((n * H + iy) * W + ix) * CI;
                            const float* w = Wt + ((f * KH + ry) * KW + rx) * CI;
                            for (int64_t c = 0; c < CI; ++c) acc += (double)a[c] * (double)w[c];
                        }
                    }
                    Out[((n * HO + y) * WO + x) * CO + f] = (float)acc;
                }
}

/*
 * ops/x86/conv2d_int8.py:74-93 with the filter in KRSC order.  uint8 input, int8 filter, int32 sum;
 * the padding value is 0 (conv2d_int8.py:68-72 pads with the dtype's zero).
 */
ORC_API void orc_conv2d_nhwc_u8s8s32(const uint8_t* In, const int8_t* Wt, int32_t* Out,
                                     int64_t N, int64_t H, int64_t W, int64_t CI, int64_t CO,
                                     int64_t KH, int64_t KW, int64_t stride, int64_t stride_w, int64_t pad, int64_t pad_w,
                                     int64_t dil, int64_t dil_w) {
    const int64_t HO = (H - ((KH - 1) * dil + 1) + 2 * pad) / stride + 1;
    const int64_t WO = (W - ((KW - 1) * dil_w + 1) + 2 * pad_w) / stride_w + 1;
#pragma omp parallel for collapse(3) schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t y = 0; y < HO; ++y)
            for (int64_t x = 0; x < WO; ++x)
                for (int64_t f = 0; f < CO; ++f) {
                    int32_t acc = 0;
                    for (int64_t ry = 0; ry < KH; ++ry) {
                        const int64_t iy = y * stride + ry * dil - pad;
                        if (iy < 0 || iy >= H) continue;
                        for (int64_t rx = 0; rx < KW; ++rx) {
                            const int64_t ix = x * stride_w + rx * dil_w - pad_w;
                            if (ix < 0 || ix >= W) continue;
                            const uint8_t* a = In + ((n * H + iy) * W + ix) * CI;
                            const int8_t* w = Wt + ((f * KH + ry) * KW + rx) * CI;
                            for (int64_t c = 0; c < CI; ++c) acc += (int32_t)a[c] * (int32_t)w[c];
                        }
                    }
                    Out[((n * HO + y) * WO + x) * CO + f] = acc;
                }
}

/*
 * The operator with the reference's operand shapes (conv2d_int8.py:50-52,74-93): filter
 * (CO/cb, KH, KW, CI/4, cb, 4) for w_format "OhwI<cb>o4i", output (N, HO, WO, CO/cb, cb); the loop
 * nest and index expressions are those of the te.compute, with the padded input formed explicitly.
 */
ORC_API int orc_conv2d_nhwc_u8s8s32_blocked(const uint8_t* In, const int8_t* Wb, int32_t* Out,
                                            int64_t N, int64_t H, int64_t W, int64_t CI, int64_t CO,
                                            int64_t KH, int64_t KW, int64_t stride, int64_t pad, int64_t dil,
                                            int64_t cb) {
    if (cb <= 0 || CO % cb || CI % 4) return -1;
    const int64_t HO = (H - ((KH - 1) * dil + 1) + 2 * pad) / stride + 1;
    const int64_t WO = (W - ((KW - 1) * dil + 1) + 2 * pad) / stride + 1;
    const int64_t HP = H + 2 * pad, WP = W + 2 * pad;
    uint8_t* P = (uint8_t*)calloc((size_t)(N * HP * WP * CI), 1);
    if (!P) return -2;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t y = 0; y < H; ++y)
            memcpy(P + ((n * HP + y + pad) * WP + pad) * CI, In + (n * H + y) * W * CI, (size_t)(W * CI));
    const int64_t ICC = CI / 4;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t yy = 0; yy < HO; ++yy)
            for (int64_t xx = 0; xx < WO; ++xx)
                for (int64_t occ = 0; occ < CO / cb; ++occ)
                    for (int64_t ocb = 0; ocb < cb; ++ocb) {
                        int32_t acc = 0;
                        for (int64_t ry = 0; ry < KH; ++ry)
                            for (int64_t rx = 0; rx < KW; ++rx)
                                for (int64_t icc = 0; icc < ICC; ++icc)
                                    for (int64_t icb = 0; icb < 4; ++icb) {
                                        const int32_t a = P[((n * HP + yy * stride + ry * dil) * WP + xx * stride + rx * dil) * CI + icc * 4 + icb];
                                        const int32_t w = Wb[((((occ * KH + ry) * KW + rx) * ICC + icc) * cb + ocb) * 4 + icb];
                                        acc += a * w;
                                    }
                        Out[(((n * HO + yy) * WO + xx) * (CO / cb) + occ) * cb + ocb] = acc;
                    }
    free(P);
    return 0;
}
