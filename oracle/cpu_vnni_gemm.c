/*
 * TEST / BENCHMARK INFRASTRUCTURE -- never linked into the product library.
 *
 * The CPU baseline leg of the benchmark: the same int8 Gemm (per-row dynamic quantisation of A, constant int8 B,
 * fp32 dequantise + bias epilogue) written the way the reference's x86 path computes it, so that the GPU figure has
 * an honest CPU figure beside it rather than a scalar loop:
 *   - B is repacked once to [K/4][N][4] (ncnn packs constant weights at create_pipeline, src/layer/x86/gemm_x86.cpp);
 *   - signed x signed on VNNI: vpdpbusd multiplies unsigned by signed bytes, so A is offset by +128 and the surplus
 *     128 * sum_k B[j][k] is subtracted afterwards -- the trick of src/layer/x86/gemm_int8.h:109-126 (there with +127);
 *   - OpenMP over row blocks, 4 rows x 64 columns of int32 accumulators in registers.
 * The integer accumulators equal the scalar oracle's exactly; the float epilogue repeats its statements.
 * Compiled for any x86-64 (the intrinsics sit behind target attributes); cpu_vnni_available() says whether the host
 * can run it.
 */
#include <immintrin.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* OpenMP width of the calls that follow (the benchmark reports one thread and all threads) */
ORACLE_API void cpu_vnni_set_num_threads(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n > 0 ? n : 1);
#else
    (void)n;
#endif
}

ORACLE_API int cpu_vnni_available(void)
{
    __builtin_cpu_init();
    return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512vnni");
}

/* packed size in bytes for B[N][K]: K rounded up to 4, N rounded up to 64, plus N int32 column sums */
ORACLE_API size_t cpu_vnni_packed_bytes(int N, int K)
{
    const size_t k4 = (size_t)(K + 3) / 4, n64 = (size_t)(N + 63) / 64 * 64;
    return k4 * n64 * 4 + n64 * sizeof(int32_t);
}

ORACLE_API void cpu_vnni_pack_b(const int8_t* bq, size_t bq_stride, int N, int K, void* packed)
{
    const size_t k4 = (size_t)(K + 3) / 4, n64 = (size_t)(N + 63) / 64 * 64;
    int8_t* p = (int8_t*)packed;
    int32_t* colsum = (int32_t*)(p + k4 * n64 * 4);
    memset(p, 0, k4 * n64 * 4);
    for (size_t j = 0; j < n64; j++) colsum[j] = 0;
    for (int j = 0; j < N; j++)
    {
        int32_t s = 0;
        for (int k = 0; k < K; k++)
        {
            const int8_t v = bq[(size_t)j * bq_stride + k];
            p[((size_t)(k / 4) * n64 + j) * 4 + (k & 3)] = v;
            s += v;
        }
        colsum[j] = s;
    }
}

__attribute__((target("avx512f,avx512bw,avx512vnni"))) static void rows4_block(const uint8_t* au, size_t au_stride, int rows, const int8_t* p,
                                                                                size_t n64, size_t k4, size_t j0, int32_t* acc /* [4][64] */)
{
    __m512i c[4][4];
    for (int r = 0; r < 4; r++)
        for (int v = 0; v < 4; v++) c[r][v] = _mm512_setzero_si512();
    for (size_t kk = 0; kk < k4; kk++)
    {
        const int8_t* bp = p + (kk * n64 + j0) * 4;
        const __m512i b0 = _mm512_loadu_si512((const void*)(bp));
        const __m512i b1 = _mm512_loadu_si512((const void*)(bp + 64));
        const __m512i b2 = _mm512_loadu_si512((const void*)(bp + 128));
        const __m512i b3 = _mm512_loadu_si512((const void*)(bp + 192));
        for (int r = 0; r < 4; r++) /* all four rows, whatever `rows` is: constant trip counts keep the accumulators in registers */
        {
            int32_t a4;
            memcpy(&a4, au + (size_t)r * au_stride + kk * 4, 4);
            const __m512i av = _mm512_set1_epi32(a4);
            c[r][0] = _mm512_dpbusd_epi32(c[r][0], av, b0);
            c[r][1] = _mm512_dpbusd_epi32(c[r][1], av, b1);
            c[r][2] = _mm512_dpbusd_epi32(c[r][2], av, b2);
            c[r][3] = _mm512_dpbusd_epi32(c[r][3], av, b3);
        }
    }
    (void)rows;
    for (int r = 0; r < 4; r++)
        for (int v = 0; v < 4; v++) _mm512_storeu_si512((void*)(acc + r * 64 + v * 16), c[r][v]);
}

/*
 * a: fp32 [M][K] (row stride a_stride).  Per row: absmax, scale 127/absmax (1 when the row is zero), quantise with
 * round-half-away and clamp to [-127,127] (Gemm::forward_int8, src/layer/gemm.cpp:807-821), then the int8 product
 * against the packed B and the epilogue  out = (float)acc * (1/(sA*sB)) + bias[j]   (broadcast type 4, alpha = beta = 1;
 * with n_b_scales == N: ((float)acc * (1/sA)) * (1/sB_j) + bias[j]).  acc_out (optional) receives the int32 sums.
 */
__attribute__((target("avx512f,avx512bw,avx512vnni"))) ORACLE_API int cpu_vnni_gemm(const float* a, size_t a_stride, int M, int N, int K, const void* packed,
                                                                                    const float* b_scales, int n_b_scales, const float* bias, float* out,
                                                                                    size_t out_stride, int32_t* acc_out)
{
    const size_t k4 = (size_t)(K + 3) / 4, n64 = (size_t)(N + 63) / 64 * 64;
    const int8_t* p = (const int8_t*)packed;
    const int32_t* colsum = (const int32_t*)(p + k4 * n64 * 4);
    int failed = 0;
#pragma omp parallel
    {
        uint8_t* au = (uint8_t*)aligned_alloc(64, ((size_t)4 * k4 * 4 + 127) & ~(size_t)63);
        int32_t acc[4 * 64];
        float sa[4];
        if (!au)
        {
#pragma omp atomic write
            failed = 1;
        }
        else
            memset(au, 128, (size_t)4 * k4 * 4); /* the micro-kernel multiplies all four rows, also when fewer are asked for */
#pragma omp for schedule(dynamic, 4)
        for (int i0 = 0; i0 < M; i0 += 4)
        {
            if (!au) continue;
            const int rows = M - i0 < 4 ? M - i0 : 4;
            for (int r = 0; r < rows; r++)
            {
                const float* ar = a + (size_t)(i0 + r) * a_stride;
                float absmax = 0.f;
                for (int k = 0; k < K; k++)
                {
                    const float v = ar[k] < 0.f ? -ar[k] : ar[k];
                    if (v > absmax) absmax = v;
                }
                sa[r] = absmax == 0.f ? 1.f : 127.f / absmax;
                uint8_t* q = au + (size_t)r * k4 * 4;
                for (int k = 0; k < K; k++)
                {
                    const float v = ar[k] * sa[r];
                    int iv = (int)(v < 0.f ? v - 0.5f : v + 0.5f); /* round half away from zero */
                    /* v +- 0.5f can itself round up at |v| just below a half: redo such values exactly */
                    if ((double)iv - (double)v > 0.5) iv--;
                    if ((double)v - (double)iv > 0.5) iv++;
                    if (iv > 127) iv = 127;
                    if (iv < -127) iv = -127;
                    q[k] = (uint8_t)(iv + 128);
                }
                for (size_t k = (size_t)K; k < k4 * 4; k++) q[k] = 128; /* K padding: (0 + 128) against zero weights */
            }
            for (size_t j0 = 0; j0 < n64; j0 += 64)
            {
                rows4_block(au, k4 * 4, rows, p, n64, k4, j0, acc);
                for (int r = 0; r < rows; r++)
                    for (int jj = 0; jj < 64 && j0 + jj < (size_t)N; jj++)
                    {
                        const size_t j = j0 + jj;
                        const int32_t s = acc[r * 64 + jj] - 128 * colsum[j];
                        if (acc_out) acc_out[(size_t)(i0 + r) * N + j] = s;
                        float f;
                        if (n_b_scales == 1)
                        {
                            const float descale = 1.f / (sa[r] * b_scales[0]);
                            f = (float)s * descale;
                        }
                        else
                        {
                            const float da = 1.f / sa[r];
                            const float db = 1.f / b_scales[j];
                            f = (float)s * da;
                            f = f * db;
                        }
                        if (bias) f = f + bias[j] * 1.f;
                        f = f * 1.f;
                        out[(size_t)(i0 + r) * out_stride + j] = f;
                    }
            }
        }
        free(au);
    }
    return failed ? -1 : 0;
}
