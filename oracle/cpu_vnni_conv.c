/*
 * TEST / BENCHMARK INFRASTRUCTURE -- never linked into the product library.
 *
 * CPU baseline of the quantised convolution family, written the way the reference's x86 path computes it (the class of
 * src/layer/x86/convolution_im2col_gemm_int8.h and src/layer/x86/convolutiondepthwise_3x3_int8.h): channel-interleaved
 * int8 activations, weights repacked once, im2col rows multiplied on VNNI, a vectorised dequantise / bias / activation /
 * requantise epilogue, OpenMP over blocks of output pixels.  Results equal the scalar oracle's bit for bit: the integer
 * sums are exact, and every float statement of Convolution::forward_int8 (src/layer/convolution.cpp:383-508) and
 * ConvolutionDepthWise::forward_int8 (src/layer/convolutiondepthwise.cpp:505-559) is one IEEE binary32 operation here too.
 *
 * Layout: activations are channels-last, [n][h][w][c] (fp32 or int8); outputs [n][outh*outw][num_output].
 *   convolution: the border-padded image is stored as unsigned bytes q + 128 (vpdpbusd multiplies unsigned by signed);
 *                the surplus 128 * sum_k w[j][k] is taken off afterwards, as in cpu_vnni_gemm.c.  K runs (ky, kx, c).
 *   depthwise:   signed bytes, 16 channels per vector, one 32-bit multiply-add per tap.
 * The glue layers a whole-model pass needs (element-wise sum, ReLU, pooling) are here as plain loops in the reference's
 * order of operations.
 */
#include <float.h>
#include <immintrin.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))
#define VNNI __attribute__((target("avx512f,avx512bw,avx512vl,avx512vnni")))

/* scalar statements of the oracle, for the activation types that are not vectorised here */
float oracle_activation(float v, int type, const float* p);

typedef struct
{
    int w, h, c, n; /* input */
    int num_output;
    int kernel_w, kernel_h, dilation_w, dilation_h, stride_w, stride_h;
    int pad_left, pad_right, pad_top, pad_bottom; /* explicit (already resolved) borders */
    float pad_value;
} cpu_conv_desc;

/* round half away from zero, NaN and magnitudes beyond the int range -> -127, clamp to [-127, 127]: the oracle's
 * float2int8 (what ncnn's scalar x86 build computes), on 16 lanes.  Returns int32 lanes. */
VNNI static inline __m512i f2i8_lanes(__m512 v)
{
    const __m512 t = _mm512_roundscale_ps(v, _MM_FROUND_TO_ZERO | _MM_FROUND_NO_EXC);
    const __m512 diff = _mm512_sub_ps(v, t); /* exact: same sign, |diff| < 1 */
    const __m512 absdiff = _mm512_abs_ps(diff);
    const __mmask16 away = _mm512_cmp_ps_mask(absdiff, _mm512_set1_ps(0.5f), _CMP_GE_OQ);
    const __m512 one = _mm512_castsi512_ps(_mm512_or_si512(_mm512_and_si512(_mm512_castps_si512(v), _mm512_set1_epi32((int)0x80000000u)),
                                                           _mm512_castps_si512(_mm512_set1_ps(1.f))));
    __m512 r = _mm512_mask_add_ps(t, away, t, one);
    const __mmask16 in_range = _mm512_cmp_ps_mask(r, _mm512_set1_ps(2147483648.f), _CMP_LT_OQ) & _mm512_cmp_ps_mask(r, _mm512_set1_ps(-2147483648.f), _CMP_GE_OQ);
    r = _mm512_max_ps(r, _mm512_set1_ps(-127.f));
    r = _mm512_min_ps(r, _mm512_set1_ps(127.f));
    r = _mm512_mask_mov_ps(_mm512_set1_ps(-127.f), in_range, r);
    return _mm512_cvtps_epi32(r);
}

VNNI static inline __m512 activate_lanes(__m512 f, int type, const float* p)
{
    if (type == 0) return f;
    if (type == 1) return _mm512_max_ps(f, _mm512_setzero_ps()); /* fmaxf(v, 0): NaN -> 0 */
    if (type == 2)
    {
        const __mmask16 pos = _mm512_cmp_ps_mask(f, _mm512_setzero_ps(), _CMP_GT_OQ);
        return _mm512_mask_mov_ps(_mm512_mul_ps(f, _mm512_set1_ps(p[0])), pos, f);
    }
    if (type == 3)
    {
        const __m512 lo = _mm512_set1_ps(p[0]), hi = _mm512_set1_ps(p[1]);
        f = _mm512_mask_mov_ps(f, _mm512_cmp_ps_mask(f, lo, _CMP_LT_OQ), lo);
        f = _mm512_mask_mov_ps(f, _mm512_cmp_ps_mask(f, hi, _CMP_GT_OQ), hi);
        return f;
    }
    float tmp[16];
    _mm512_storeu_ps(tmp, f);
    for (int i = 0; i < 16; i++) tmp[i] = oracle_activation(tmp[i], type, p);
    return _mm512_loadu_ps(tmp);
}

/* (acc int32 lanes) -> dequantise, bias, activation, optional requantise; stores `lanes` (<= 16) values */
VNNI static inline void epilogue_store(__m512i acc, const float* scale_in, const float* bias, const float* scale_out_lanes, float scale_out_uniform,
                                       int act_type, const float* act_params, void* out, int requant, int lanes)
{
    const __mmask16 m = (__mmask16)((1u << lanes) - 1u);
    __m512 f = _mm512_mul_ps(_mm512_cvtepi32_ps(acc), _mm512_maskz_loadu_ps(m, scale_in));
    if (bias) f = _mm512_add_ps(f, _mm512_maskz_loadu_ps(m, bias));
    f = activate_lanes(f, act_type, act_params);
    if (requant)
    {
        const __m512 so = scale_out_lanes ? _mm512_maskz_loadu_ps(m, scale_out_lanes) : _mm512_set1_ps(scale_out_uniform);
        const __m512i q = f2i8_lanes(_mm512_mul_ps(f, so));
        _mm_mask_storeu_epi8(out, m, _mm512_cvtepi32_epi8(q));
    }
    else
        _mm512_mask_storeu_ps(out, m, f);
}

/* The border-padded copy of the input lives in a buffer the calling thread keeps and grows (the reference takes such
 * blobs from a pool allocator): a fresh allocation per layer would spend more time in page faults than in arithmetic. */
static void* staging(size_t bytes)
{
    static __thread void* buf = 0;
    static __thread size_t cap = 0;
    if (bytes > cap)
    {
        free(buf);
        cap = (bytes + ((size_t)1 << 20)) & ~(((size_t)1 << 20) - 1);
        buf = aligned_alloc(64, cap);
        if (!buf) cap = 0;
    }
    return buf;
}

/* ------------------------------------------------------------------------------------------------ convolution */

#define PIX 6 /* output pixels per block: 6 x 64 int32 accumulators in 24 registers */

VNNI static void pix_block(const uint8_t* a, size_t a_stride, int rows, const int8_t* p, size_t n64, size_t k4, size_t j0, int32_t* acc /* [PIX][64] */)
{
    __m512i c[PIX][4];
    for (int r = 0; r < PIX; r++)
        for (int v = 0; v < 4; v++) c[r][v] = _mm512_setzero_si512();
    for (size_t kk = 0; kk < k4; kk++)
    {
        const int8_t* bp = p + (kk * n64 + j0) * 4;
        const __m512i b0 = _mm512_loadu_si512((const void*)(bp));
        const __m512i b1 = _mm512_loadu_si512((const void*)(bp + 64));
        const __m512i b2 = _mm512_loadu_si512((const void*)(bp + 128));
        const __m512i b3 = _mm512_loadu_si512((const void*)(bp + 192));
        for (int r = 0; r < PIX; r++)
        {
            int32_t a4;
            memcpy(&a4, a + (size_t)r * a_stride + kk * 4, 4);
            const __m512i av = _mm512_set1_epi32(a4);
            c[r][0] = _mm512_dpbusd_epi32(c[r][0], av, b0);
            c[r][1] = _mm512_dpbusd_epi32(c[r][1], av, b1);
            c[r][2] = _mm512_dpbusd_epi32(c[r][2], av, b2);
            c[r][3] = _mm512_dpbusd_epi32(c[r][3], av, b3);
        }
    }
    /* all PIX rows, whatever `rows` is: a constant trip count keeps the accumulators in registers */
    (void)rows;
    for (int r = 0; r < PIX; r++)
        for (int v = 0; v < 4; v++) _mm512_storeu_si512((void*)(acc + r * 64 + v * 16), c[r][v]);
}

/* fp32 or int8 channels-last image -> border-padded unsigned image q + 128, [n][H][W][c] */
VNNI static uint8_t* padded_u8(const cpu_conv_desc* d, const void* x, int x_elemsize, float in_scale, size_t buffer_bytes)
{
    const int H = d->h + d->pad_top + d->pad_bottom, W = d->w + d->pad_left + d->pad_right, c = d->c;
    uint8_t* out = (uint8_t*)staging(buffer_bytes);
    if (!out) return 0;
    const uint8_t border = (uint8_t)((int)(int8_t)d->pad_value + 128);
    const __m512 vs = _mm512_set1_ps(in_scale);
#pragma omp parallel for schedule(static)
    for (int row = 0; row < d->n * H; row++)
    {
        const int b = row / H, y = row - b * H - d->pad_top;
        uint8_t* o = out + (size_t)row * W * c;
        if (y < 0 || y >= d->h)
        {
            memset(o, border, (size_t)W * c);
            continue;
        }
        memset(o, border, (size_t)d->pad_left * c);
        memset(o + (size_t)(d->pad_left + d->w) * c, border, (size_t)d->pad_right * c);
        uint8_t* dst = o + (size_t)d->pad_left * c;
        const size_t count = (size_t)d->w * c, base = ((size_t)b * d->h + y) * d->w * c;
        if (x_elemsize == 1)
        {
            const int8_t* src = (const int8_t*)x + base;
            for (size_t i = 0; i < count; i++) dst[i] = (uint8_t)(src[i] + 128);
        }
        else
        {
            const float* src = (const float*)x + base;
            for (size_t i = 0; i < count; i += 16)
            {
                const int lanes = count - i < 16 ? (int)(count - i) : 16;
                const __mmask16 m = (__mmask16)((1u << lanes) - 1u);
                const __m512i q = f2i8_lanes(_mm512_mul_ps(_mm512_maskz_loadu_ps(m, src + i), vs));
                _mm_mask_storeu_epi8(dst + i, m, _mm512_cvtepi32_epi8(_mm512_add_epi32(q, _mm512_set1_epi32(128))));
            }
        }
    }
    return out;
}

/*
 * Convolution (group 1).  packed: cpu_vnni_pack_b of the weights reordered to [num_output][kernel_h][kernel_w][c].
 * x fp32 (quantised here with in_scale) or int8; scale_in[j] = 0 where the weight scale is 0, else 1/(in_scale*w_scale[j]);
 * scale_out NULL -> fp32 output, else int8 output float2int8(v * scale_out[0]).
 */
VNNI ORACLE_API int cpu_vnni_conv_nhwc(const cpu_conv_desc* d, const void* x, int x_elemsize, float in_scale, const void* packed,
                                       const float* scale_in, const float* bias, const float* scale_out, int act_type, const float* act_params, void* out)
{
    const int c = d->c, N = d->num_output;
    const int H = d->h + d->pad_top + d->pad_bottom, W = d->w + d->pad_left + d->pad_right;
    const int outw = (W - (d->dilation_w * (d->kernel_w - 1) + 1)) / d->stride_w + 1;
    const int outh = (H - (d->dilation_h * (d->kernel_h - 1) + 1)) / d->stride_h + 1;
    const size_t K = (size_t)d->kernel_w * d->kernel_h * c, k4 = (K + 3) / 4, n64 = (size_t)(N + 63) / 64 * 64;
    const long long npix = (long long)d->n * outh * outw, nblocks = (npix + PIX - 1) / PIX;
    const int direct = d->kernel_w == 1 && d->kernel_h == 1 && d->stride_w == 1 && d->stride_h == 1 && K % 4 == 0; /* rows are the pixels themselves */
    /* the micro-kernel always reads PIX rows: both buffers carry a block of slack behind the last row */
    const size_t img_bytes = ((size_t)d->n * H * W * c + (size_t)PIX * k4 * 4 + 127) & ~(size_t)63;
    const size_t rows_bytes = direct ? 0 : (size_t)nblocks * PIX * k4 * 4;
    uint8_t* img = padded_u8(d, x, x_elemsize, in_scale, img_bytes + rows_bytes);
    if (!img) return -100;
    const int8_t* p = (const int8_t*)packed;
    const int32_t* colsum = (const int32_t*)(p + k4 * n64 * 4);
    const int requant = scale_out != 0;
    const size_t out_elem = requant ? 1 : 4;
    const uint8_t* a = img;
    size_t a_stride = (size_t)c;
    if (!direct)
    {
        /* im2col: one row of K bytes per output pixel, K running (ky, kx, c) */
        uint8_t* rows = img + img_bytes;
        a = rows;
        a_stride = k4 * 4;
#pragma omp parallel for schedule(static)
        for (long long pix = 0; pix < nblocks * PIX; pix++)
        {
            uint8_t* row = rows + (size_t)pix * k4 * 4;
            if (pix >= npix)
            {
                memset(row, 128, k4 * 4);
                continue;
            }
            const int b = (int)(pix / ((long long)outh * outw));
            const int rem = (int)(pix - (long long)b * outh * outw);
            const int oy = rem / outw, ox = rem - oy * outw;
            const uint8_t* src = img + (((size_t)b * H + (size_t)oy * d->stride_h) * W + (size_t)ox * d->stride_w) * c;
            uint8_t* o = row;
            for (int ky = 0; ky < d->kernel_h; ky++)
            {
                const uint8_t* line = src + (size_t)ky * d->dilation_h * W * c;
                if (d->dilation_w == 1)
                {
                    memcpy(o, line, (size_t)d->kernel_w * c);
                    o += (size_t)d->kernel_w * c;
                }
                else
                    for (int kx = 0; kx < d->kernel_w; kx++, o += c) memcpy(o, line + (size_t)kx * d->dilation_w * c, (size_t)c);
            }
            for (size_t k = K; k < k4 * 4; k++) row[k] = 128;
        }
    }
    /* one task = one 64-channel panel of the weights (it stays in the core's cache) over a run of pixel blocks */
    const long long chunk = 8, nchunks = (nblocks + chunk - 1) / chunk;
    const long long npanels = (long long)(n64 / 64);
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (long long panel = 0; panel < npanels; panel++)
        for (long long ch = 0; ch < nchunks; ch++)
        {
            int32_t acc[PIX * 64];
            const size_t j0 = (size_t)panel * 64;
            const long long blk_end = (ch + 1) * chunk < nblocks ? (ch + 1) * chunk : nblocks;
            for (long long blk = ch * chunk; blk < blk_end; blk++)
            {
                const long long p0 = blk * PIX;
                const int cnt = npix - p0 < PIX ? (int)(npix - p0) : PIX;
                pix_block(a + (size_t)p0 * a_stride, a_stride, cnt, p, n64, k4, j0, acc);
                for (int r = 0; r < cnt; r++)
                    for (int v = 0; v < 4; v++)
                    {
                        const size_t j = j0 + (size_t)v * 16;
                        if (j >= (size_t)N) break;
                        const int lanes = (size_t)N - j < 16 ? (int)((size_t)N - j) : 16;
                        const __mmask16 m = (__mmask16)((1u << lanes) - 1u);
                        const __m512i s = _mm512_sub_epi32(_mm512_loadu_si512((const void*)(acc + r * 64 + v * 16)),
                                                           _mm512_slli_epi32(_mm512_maskz_loadu_epi32(m, colsum + j), 7));
                        epilogue_store(s, scale_in + j, bias ? bias + j : 0, 0, requant ? scale_out[0] : 0.f, act_type, act_params,
                                       (char*)out + ((size_t)(p0 + r) * N + j) * out_elem, requant, lanes);
                    }
            }
        }
    return 0;
}

/* ------------------------------------------------------------------------------------------------ depthwise */

/*
 * ConvolutionDepthWise with group == c == num_output.  weight_taps: int8 [kernel_h*kernel_w][c] (tap-major).
 * in_scales / scale_in / scale_out hold one value per channel (scale_out NULL -> fp32 output).
 */
VNNI ORACLE_API int cpu_dwconv_nhwc(const cpu_conv_desc* d, const void* x, int x_elemsize, const float* in_scales, const int8_t* weight_taps,
                                    const float* scale_in, const float* bias, const float* scale_out, int act_type, const float* act_params, void* out)
{
    const int c = d->c, H = d->h + d->pad_top + d->pad_bottom, W = d->w + d->pad_left + d->pad_right;
    const int outw = (W - (d->dilation_w * (d->kernel_w - 1) + 1)) / d->stride_w + 1;
    const int outh = (H - (d->dilation_h * (d->kernel_h - 1) + 1)) / d->stride_h + 1;
    const int taps = d->kernel_w * d->kernel_h;
    int8_t* img = (int8_t*)staging((size_t)d->n * H * W * c + 64);
    if (!img) return -100;
    const int8_t border = (int8_t)d->pad_value;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < d->n * H; row++)
    {
        const int b = row / H, y = row - b * H - d->pad_top;
        int8_t* o = img + (size_t)row * W * c;
        memset(o, border, (size_t)W * c);
        if (y < 0 || y >= d->h) continue;
        int8_t* dst = o + (size_t)d->pad_left * c;
        const size_t base = ((size_t)b * d->h + y) * d->w * c;
        if (x_elemsize == 1)
            memcpy(dst, (const int8_t*)x + base, (size_t)d->w * c);
        else
            for (int px = 0; px < d->w; px++)
                for (int j = 0; j < c; j += 16)
                {
                    const int lanes = c - j < 16 ? c - j : 16;
                    const __mmask16 m = (__mmask16)((1u << lanes) - 1u);
                    const __m512 v = _mm512_mul_ps(_mm512_maskz_loadu_ps(m, (const float*)x + base + (size_t)px * c + j), _mm512_maskz_loadu_ps(m, in_scales + j));
                    _mm_mask_storeu_epi8(dst + (size_t)px * c + j, m, _mm512_cvtepi32_epi8(f2i8_lanes(v)));
                }
    }
    const int requant = scale_out != 0;
    const size_t out_elem = requant ? 1 : 4;
    if (taps > 49) return -1;
#pragma omp parallel for schedule(static)
    for (int orow = 0; orow < d->n * outh; orow++)
    {
        const int b = orow / outh, oy = orow - b * outh;
        for (int j = 0; j < c; j += 16)
        {
            const int lanes = c - j < 16 ? c - j : 16;
            const __mmask16 m = (__mmask16)((1u << lanes) - 1u);
            __m512i wv[49]; /* this channel group's taps, widened once per output row */
            for (int t = 0; t < taps; t++) wv[t] = _mm512_cvtepi8_epi32(_mm_maskz_loadu_epi8(m, weight_taps + (size_t)t * c + j));
            for (int ox = 0; ox < outw; ox++)
            {
                const int8_t* src = img + (((size_t)b * H + (size_t)oy * d->stride_h) * W + (size_t)ox * d->stride_w) * c + j;
                __m512i acc = _mm512_setzero_si512();
                for (int ky = 0; ky < d->kernel_h; ky++)
                    for (int kx = 0; kx < d->kernel_w; kx++)
                    {
                        const __m128i xv = _mm_maskz_loadu_epi8(m, src + ((size_t)ky * d->dilation_h * W + (size_t)kx * d->dilation_w) * c);
                        acc = _mm512_add_epi32(acc, _mm512_mullo_epi32(_mm512_cvtepi8_epi32(xv), wv[ky * d->kernel_w + kx]));
                    }
                epilogue_store(acc, scale_in + j, bias ? bias + j : 0, requant ? scale_out + j : 0, 0.f, act_type, act_params,
                               (char*)out + (((size_t)orow * outw + ox) * c + j) * out_elem, requant, lanes);
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------ glue layers */

/* Eltwise SUM of two fp32 blobs (src/layer/eltwise.cpp) */
ORACLE_API void cpu_add_f32(const float* a, const float* b, float* out, size_t count)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)count; i++) out[i] = a[i] + b[i];
}

/* ReLU::forward_inplace with slope 0 (src/layer/relu.cpp): fp32 or int8 */
ORACLE_API void cpu_relu(void* x, int elemsize, size_t count)
{
    if (elemsize == 4)
    {
        float* f = (float*)x;
#pragma omp parallel for schedule(static)
        for (long long i = 0; i < (long long)count; i++) f[i] = f[i] < 0.f ? 0.f : f[i];
    }
    else
    {
        int8_t* q = (int8_t*)x;
#pragma omp parallel for schedule(static)
        for (long long i = 0; i < (long long)count; i++) q[i] = q[i] < 0 ? 0 : q[i];
    }
}

/* Pooling MAX over kernel x kernel windows, the default pad mode: the right / bottom edge is padded so that the last
 * window is complete (src/layer/pooling.cpp:153-235); padded taps never win.  Channels-last fp32 or int8. */
ORACLE_API void cpu_maxpool_nhwc(const void* x, int elemsize, int n, int h, int w, int c, int kernel, int stride, void* out, int outh, int outw)
{
#pragma omp parallel for schedule(static)
    for (int orow = 0; orow < n * outh; orow++)
    {
        const int b = orow / outh, oy = orow - b * outh;
        for (int ox = 0; ox < outw; ox++)
            for (int j = 0; j < c; j++)
            {
                if (elemsize == 4)
                {
                    float best = -FLT_MAX;
                    for (int ky = 0; ky < kernel; ky++)
                        for (int kx = 0; kx < kernel; kx++)
                        {
                            const int y = oy * stride + ky, xx = ox * stride + kx;
                            if (y >= h || xx >= w) continue;
                            const float v = ((const float*)x)[(((size_t)b * h + y) * w + xx) * c + j];
                            if (v > best) best = v;
                        }
                    ((float*)out)[((size_t)orow * outw + ox) * c + j] = best;
                }
                else
                {
                    int best = -128;
                    for (int ky = 0; ky < kernel; ky++)
                        for (int kx = 0; kx < kernel; kx++)
                        {
                            const int y = oy * stride + ky, xx = ox * stride + kx;
                            if (y >= h || xx >= w) continue;
                            const int v = ((const int8_t*)x)[(((size_t)b * h + y) * w + xx) * c + j];
                            if (v > best) best = v;
                        }
                    ((int8_t*)out)[((size_t)orow * outw + ox) * c + j] = (int8_t)best;
                }
            }
    }
}

/* global average pooling: the sum runs over the pixels in index order, then one division (src/layer/pooling.cpp:60-80) */
ORACLE_API void cpu_global_avgpool_nhwc(const float* x, int n, int hw, int c, float* out)
{
#pragma omp parallel for schedule(static)
    for (int bj = 0; bj < n * c; bj++)
    {
        const int b = bj / c, j = bj - b * c;
        float s = 0.f;
        for (int i = 0; i < hw; i++) s += x[((size_t)b * hw + i) * c + j];
        out[(size_t)b * c + j] = s / (float)hw;
    }
}
