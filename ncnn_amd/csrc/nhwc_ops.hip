// Device-resident blobs and the small fp32 layers that sit between the int8 layers.
//
// While a net runs, a 3-D blob lives in HBM channels-last: [n][h*w][cp] with cp = 16*ceil(c/16), fp32 or int8,
// pad channels zero.  That is the K-contiguous operand the convolution kernels want, every elementwise or
// window kernel is coalesced along channels, and one pixel's channels of an int8 blob are whole 16-byte words.
// 1-D and 2-D blobs are dense [n][h][w].  ncnn's planar layout ([c][cstep] planes) exists only at the host
// boundary: chw_to_nhwc after the upload, nhwc_to_chw before the download (and for Flatten, whose output order
// is the planar one).
//
// Each kernel follows the reference's scalar statement order for its element (window sums run ky-major, kx-minor;
// the global average sums pixels in index order), so fp32 results equal the host loops' bit for bit; Softmax
// alone reduces in parallel and uses the device expf.
#include <float.h>

#include "common.h"

namespace ncnnhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ---- planar <-> channels-last.  One workgroup: 64 pixels x 64 channels; a wavefront reads 64 consecutive
// pixels of one plane and each lane writes 16 consecutive channels of its pixel.
template<typename T>
__global__ __launch_bounds__(256) void chw_to_nhwc_kernel(const T* __restrict__ src, size_t cstep, size_t nstep, int c, int hw, int cp, T* __restrict__ dst)
{
    const int pix = blockIdx.x * 64 + (threadIdx.x & 63);
    const int q0 = blockIdx.y * 64 + (threadIdx.x >> 6) * 16;
    const int img = blockIdx.z;
    if (pix >= hw || q0 >= cp) return;
    const T* sp = src + (size_t)img * nstep + pix;
    __attribute__((aligned(16))) T v[16];
#pragma unroll
    for (int e = 0; e < 16; e++) v[e] = (q0 + e < c) ? sp[(size_t)(q0 + e) * cstep] : (T)0;
    T* dp = dst + ((size_t)img * hw + pix) * cp + q0;
#pragma unroll
    for (int e = 0; e < 16; e += 16 / sizeof(T))
        *reinterpret_cast<v4i*>(dp + e) = *reinterpret_cast<const v4i*>(v + e);
}

template<typename T>
__global__ __launch_bounds__(256) void nhwc_to_chw_kernel(const T* __restrict__ src, int c, int hw, int cp, T* __restrict__ dst, size_t cstep, size_t nstep)
{
    const int pix = blockIdx.x * 64 + (threadIdx.x & 63);
    const int q0 = blockIdx.y * 64 + (threadIdx.x >> 6) * 16;
    const int img = blockIdx.z;
    if (pix >= hw || q0 >= cp) return;
    const T* sp = src + ((size_t)img * hw + pix) * cp + q0;
    __attribute__((aligned(16))) T v[16];
#pragma unroll
    for (int e = 0; e < 16; e += 16 / sizeof(T))
        *reinterpret_cast<v4i*>(v + e) = *reinterpret_cast<const v4i*>(sp + e);
    T* dp = dst + (size_t)img * nstep + pix;
#pragma unroll
    for (int e = 0; e < 16; e++)
        if (q0 + e < c) dp[(size_t)(q0 + e) * cstep] = v[e];
}

// ---- narrow fp32 blobs: an image of at most 4 channels kept at 4 floats per pixel (instead of 16) as it comes from the
// host; the first convolution quantises straight from it, anything else widens it first
__global__ __launch_bounds__(256) void chw_to_nhwc4_f32_kernel(const float* __restrict__ src, size_t cstep, size_t nstep, int c, int hw, float* __restrict__ dst)
{
    const int pix = blockIdx.x * 256 + threadIdx.x;
    const int img = blockIdx.y;
    if (pix >= hw) return;
    const float* sp = src + (size_t)img * nstep + pix;
    v4f v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 4; q++)
        if (q < c) v[q] = sp[(size_t)q * cstep];
    *reinterpret_cast<v4f*>(dst + ((size_t)img * hw + pix) * 4) = v;
}

__global__ __launch_bounds__(256) void widen_nhwc4_f32_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t pixels)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= pixels) return;
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    v4f* dp = reinterpret_cast<v4f*>(dst + i * 16);
    dp[0] = *reinterpret_cast<const v4f*>(src + i * 4);
    dp[1] = zero;
    dp[2] = zero;
    dp[3] = zero;
}

// ---- Quantize on a channels-last blob: 16 channels of one pixel per thread (64 bytes in, 16 out)
__global__ __launch_bounds__(256) void quantize_nhwc_kernel(const float* __restrict__ src, int8_t* __restrict__ dst, size_t chunks, int c, int cp,
                                                             const float* __restrict__ scales, int nscales)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= chunks) return;
    const int q0 = (int)(i % (size_t)(cp / 16)) * 16;
    const float* sp = src + i * 16;
    v4i out;
#pragma unroll
    for (int w = 0; w < 4; w++)
    {
        const v4f x = *reinterpret_cast<const v4f*>(sp + w * 4);
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            const int q = q0 + w * 4 + e;
            int v = 0;
            if (q < c) v = float2int8(mul_rn(x[e], nscales == 1 ? scales[0] : scales[q]));
            word |= (uint32_t)(v & 0xff) << (8 * e);
        }
        out[w] = (int)word;
    }
    *reinterpret_cast<v4i*>(dst + i * 16) = out;
}

// ---- flat elementwise kernels (they run over pad channels too: zeros stay zeros)
__global__ __launch_bounds__(256) void int8_to_f32_kernel(const int8_t* __restrict__ src, float* __restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = (float)src[i];
}

__global__ __launch_bounds__(256) void relu_f32_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n4, float slope)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    v4f v = reinterpret_cast<const v4f*>(src)[i];
#pragma unroll
    for (int e = 0; e < 4; e++)
        if (v[e] < 0.f) v[e] = slope == 0.f ? 0.f : mul_rn(v[e], slope);
    reinterpret_cast<v4f*>(dst)[i] = v;
}

__global__ __launch_bounds__(256) void relu_s8_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i] < 0 ? (int8_t)0 : src[i];
}

__global__ __launch_bounds__(256) void scale_f32_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n, float scale)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = mul_rn(src[i], scale);
}

// Eltwise (src/layer/eltwise.cpp:14-178): op 0 product, 1 sum (optionally with coefficients), 2 max.
// first = 1: dst = a (op) b with the coefficients of the first two inputs; first = 0: dst = dst (op) b.
__global__ __launch_bounds__(256) void eltwise_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ dst, size_t n4, int op,
                                                       int weighted, float ca, float cb, int first)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const v4f x = reinterpret_cast<const v4f*>(a)[i];
    const v4f y = reinterpret_cast<const v4f*>(b)[i];
    v4f o;
#pragma unroll
    for (int e = 0; e < 4; e++)
    {
        if (op == 0)
            o[e] = mul_rn(x[e], y[e]);
        else if (op == 2)
            o[e] = fmaxf(x[e], y[e]);
        else if (weighted)
            o[e] = add_rn(first ? mul_rn(x[e], ca) : x[e], mul_rn(y[e], cb));
        else
            o[e] = add_rn(x[e], y[e]);
    }
    reinterpret_cast<v4f*>(dst)[i] = o;
}

// ---- Pooling (src/layer/pooling.cpp:18-415) on a channels-last fp32 blob: 4 channels of one output pixel per thread
struct PoolGeom
{
    int w, h, cp, outw, outh;
    int kw, kh, sw, sh, pad_top, pad_left;
    int type;              // 0 max, 1 average
    int count_include_pad; // average only
    int cx0, cx1, cy0, cy1; // average without count_include_pad: taps inside this rectangle (image coordinates) make up the divisor
};

__global__ __launch_bounds__(256) void pooling_nhwc_kernel(const float* __restrict__ src, float* __restrict__ dst, PoolGeom g, size_t total)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int groups = g.cp / 4;
    const int q4 = (int)(i % (size_t)groups);
    size_t rest = i / (size_t)groups;
    const int ox = (int)(rest % (size_t)g.outw);
    rest /= (size_t)g.outw;
    const int oy = (int)(rest % (size_t)g.outh);
    const int img = (int)(rest / (size_t)g.outh);
    const float* base = src + (size_t)img * g.h * g.w * g.cp + q4 * 4;
    const int y0 = oy * g.sh - g.pad_top, x0 = ox * g.sw - g.pad_left;
    v4f r;
    if (g.type == 0)
    {
        r = v4f{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
        for (int ky = 0; ky < g.kh; ky++)
            for (int kx = 0; kx < g.kw; kx++)
            {
                const int y = y0 + ky, x = x0 + kx;
                const bool in = (unsigned)y < (unsigned)g.h && (unsigned)x < (unsigned)g.w;
                const v4f v = *reinterpret_cast<const v4f*>(base + (in ? ((size_t)y * g.w + x) * g.cp : (size_t)0)); // unconditional: loads overlap
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = in ? fmaxf(r[e], v[e]) : r[e];
            }
    }
    else
    {
        r = v4f{0.f, 0.f, 0.f, 0.f};
        int area = 0;
        for (int ky = 0; ky < g.kh; ky++)
            for (int kx = 0; kx < g.kw; kx++)
            {
                const int y = y0 + ky, x = x0 + kx;
                const bool in = (unsigned)y < (unsigned)g.h && (unsigned)x < (unsigned)g.w;
                // which taps take part: all of them with count_include_pad, else those inside the counted rectangle (the
                // reference skips the others even where they lie on the image); a tap off the image is the border's zero
                const bool counted = g.count_include_pad || (x >= g.cx0 && x < g.cx1 && y >= g.cy0 && y < g.cy1);
                if (counted)
                {
                    v4f v = {0.f, 0.f, 0.f, 0.f};
                    if (in) v = *reinterpret_cast<const v4f*>(base + ((size_t)y * g.w + x) * g.cp);
#pragma unroll
                    for (int e = 0; e < 4; e++) r[e] = add_rn(r[e], v[e]);
                    area++;
                }
            }
        const float div = g.count_include_pad ? (float)(g.kw * g.kh) : (float)area;
#pragma unroll
        for (int e = 0; e < 4; e++) r[e] = div_rn(r[e], div);
    }
    *reinterpret_cast<v4f*>(dst + (((size_t)img * g.outh + oy) * g.outw + ox) * g.cp + q4 * 4) = r;
}

// Max pooling of an int8 blob, 16 channels of one output pixel per thread.  Quantize (round, clamp to [-127,127]) is
// monotonic for a positive scale, so the maximum of the quantised values is the quantised maximum; a window without
// any pixel gives -127, which is what -FLT_MAX quantises to.
// The 16 bytes are compared as eight pairs of 16-bit lanes: the even bytes of a dword moved into the high byte of
// each half (v << 8, low bytes cleared), the odd bytes kept where they are (low bytes cleared); a signed 16-bit
// maximum (v_pk_max_i16) of two such values whose low bytes are zero orders them like the signed bytes on top.
// blockIdx.y = output row, blockIdx.z = sample: no division except the channel-group split of the column index.
typedef short v2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_i16(uint32_t a, uint32_t b)
{
    const v2s x = __builtin_bit_cast(v2s, a), y = __builtin_bit_cast(v2s, b);
    const v2s m = {x[0] > y[0] ? x[0] : y[0], x[1] > y[1] ? x[1] : y[1]};
    return __builtin_bit_cast(uint32_t, m);
}

__global__ __launch_bounds__(256) void maxpool_nhwc_s8_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst, PoolGeom g, unsigned groups, unsigned groups_magic)
{
    const unsigned r = blockIdx.x * 256 + threadIdx.x;
    if (r >= (unsigned)g.outw * groups) return;
    unsigned ox = groups == 1 ? r : __umulhi(r, groups_magic); // r / groups; exact: r * groups < 2^32 (checked at launch)
    if (ox * groups > r) ox--;
    const unsigned q16 = r - ox * groups;
    const int oy = blockIdx.y, img = blockIdx.z;
    const int8_t* base = src + (size_t)img * g.h * g.w * g.cp + q16 * 16;
    const int y0 = oy * g.sh - g.pad_top, x0 = (int)ox * g.sw - g.pad_left;
    const uint32_t lowest = 0x81008100u; // -127 in the high byte of both halves
    uint32_t even[4], odd[4];
#pragma unroll
    for (int d = 0; d < 4; d++) even[d] = odd[d] = lowest;
    for (int ky = 0; ky < g.kh; ky++)
        for (int kx = 0; kx < g.kw; kx++)
        {
            const int y = y0 + ky, x = x0 + kx;
            const bool in = (unsigned)y < (unsigned)g.h && (unsigned)x < (unsigned)g.w;
            const v4i v = *reinterpret_cast<const v4i*>(base + (in ? ((size_t)y * g.w + x) * g.cp : (size_t)0)); // unconditional: loads overlap
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                // a tap outside the image contributes -127, which changes no maximum
                const uint32_t w = in ? (uint32_t)v[d] : 0x81818181u;
                even[d] = pk_max_i16(even[d], (w << 8) & 0xff00ff00u);
                odd[d] = pk_max_i16(odd[d], w & 0xff00ff00u);
            }
        }
    v4i o;
#pragma unroll
    for (int d = 0; d < 4; d++) o[d] = (int)(((even[d] >> 8) & 0x00ff00ffu) | odd[d]);
    *reinterpret_cast<v4i*>(dst + (((size_t)img * g.outh + oy) * g.outw + ox) * g.cp + q16 * 16) = o;
}

// global pooling: [n][hw][cp] -> dense [n][c]; one thread per (sample, channel) walks the pixels in index order
// (q8 != 0: the quantised value float2int8(result * q8_scale) is stored instead, for a consumer that would quantise it so)
__global__ __launch_bounds__(64) void global_pooling_nhwc_kernel(const float* __restrict__ src, float* __restrict__ dst, int c, int hw, int cp, int type,
                                                                int8_t* __restrict__ q8, float q8_scale)
{
    const int q = blockIdx.x * 64 + threadIdx.x; // one wavefront per workgroup: the few channels spread over as many CUs as possible
    const int img = blockIdx.y;
    if (q >= c) return;
    const float* p = src + (size_t)img * hw * cp + q;
    // eight loads in flight, then folded in pixel order (the order of the reference's loop)
    float r = type == 0 ? p[0] : 0.f;
    int i = 0;
    for (; i + 8 <= hw; i += 8)
    {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = p[(size_t)(i + e) * cp];
#pragma unroll
        for (int e = 0; e < 8; e++) r = type == 0 ? fmaxf(r, v[e]) : add_rn(r, v[e]);
    }
    for (; i < hw; i++) r = type == 0 ? fmaxf(r, p[(size_t)i * cp]) : add_rn(r, p[(size_t)i * cp]);
    if (type != 0) r = div_rn(r, (float)hw);
    if (q8)
        q8[(size_t)img * c + q] = (int8_t)float2int8(mul_rn(r, q8_scale));
    else
        dst[(size_t)img * c + q] = r;
}

// ---- Softmax over a dense vector (src/layer/softmax.cpp), one workgroup per sample
__global__ __launch_bounds__(256) void softmax_kernel(const float* __restrict__ src, float* __restrict__ dst, int count)
{
    __shared__ float red[256];
    const float* p = src + (size_t)blockIdx.x * count;
    float* o = dst + (size_t)blockIdx.x * count;
    float m = -FLT_MAX;
    for (int i = threadIdx.x; i < count; i += 256) m = fmaxf(m, p[i]);
    red[threadIdx.x] = m;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1)
    {
        if ((int)threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    m = red[0];
    __syncthreads();
    float sum = 0.f;
    for (int i = threadIdx.x; i < count; i += 256)
    {
        const float e = expf(p[i] - m);
        o[i] = e;
        sum += e;
    }
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1)
    {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    sum = red[0];
    for (int i = threadIdx.x; i < count; i += 256) o[i] = div_rn(o[i], sum);
}

// ---- depthwise int8 convolution on channels-last blobs (ConvolutionDepthWise::forward_int8, channels == group
// == num_output, src/layer/convolutiondepthwise.cpp:505-559).  One thread: 16 channels of one output pixel;
// weights repacked to [tap][cp].  Memory bound: one 16-byte load per tap, neighbours served by the caches.
struct DwNhwcGeom
{
    int w, h, cp, c, outw, outh;
    int kw, kh, dw, dh, sw, sh, pad_top, pad_left;
    int pad_byte;
    int out_f32;
};

__global__ __launch_bounds__(256) void dwconv_nhwc_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ wpk, DwNhwcGeom g,
                                                           const float* __restrict__ scale_in, const float* __restrict__ bias,
                                                           const float* __restrict__ scale_out, ncnnhip_activation act, void* __restrict__ out, size_t total)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int chunks = g.cp / 16;
    const int q0 = (int)(i % (size_t)chunks) * 16;
    size_t rest = i / (size_t)chunks;
    const int ox = (int)(rest % (size_t)g.outw);
    rest /= (size_t)g.outw;
    const int oy = (int)(rest % (size_t)g.outh);
    const int img = (int)(rest / (size_t)g.outh);
    const int8_t* base = x + (size_t)img * g.h * g.w * g.cp + q0;
    const int y0 = oy * g.sh - g.pad_top, x0 = ox * g.sw - g.pad_left;
    const int padw = (int)((uint32_t)(g.pad_byte & 0xff) * 0x01010101u);

    int acc[16];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0;
    for (int ky = 0; ky < g.kh; ky++)
        for (int kx = 0; kx < g.kw; kx++)
        {
            const int y = y0 + ky * g.dh, xx = x0 + kx * g.dw;
            const bool in = (unsigned)y < (unsigned)g.h && (unsigned)xx < (unsigned)g.w;
            v4i v = *reinterpret_cast<const v4i*>(base + (in ? ((size_t)y * g.w + xx) * g.cp : (size_t)0)); // unconditional: loads can overlap
            if (!in) v = v4i{padw, padw, padw, padw};
            const v4i wv = *reinterpret_cast<const v4i*>(wpk + (size_t)(ky * g.kw + kx) * g.cp + q0);
#pragma unroll
            for (int wd = 0; wd < 4; wd++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[wd * 4 + e] += (int)(int8_t)(v[wd] >> (8 * e)) * (int)(int8_t)(wv[wd] >> (8 * e));
        }

    const size_t o = (((size_t)img * g.outh + oy) * g.outw + ox) * g.cp + q0;
    float f[16];
#pragma unroll
    for (int e = 0; e < 16; e++)
    {
        const int q = q0 + e;
        float r = 0.f;
        if (q < g.c)
        {
            r = mul_rn((float)acc[e], scale_in[q]);
            if (bias) r = add_rn(r, bias[q]);
            r = apply_activation(r, act);
            if (!g.out_f32) r = float2int8_as_float(mul_rn(r, scale_out[q]));
        }
        f[e] = r;
    }
    if (g.out_f32)
    {
#pragma unroll
        for (int wd = 0; wd < 4; wd++) *reinterpret_cast<v4f*>(static_cast<float*>(out) + o + wd * 4) = v4f{f[wd * 4], f[wd * 4 + 1], f[wd * 4 + 2], f[wd * 4 + 3]};
    }
    else
    {
        v4i pk;
#pragma unroll
        for (int wd = 0; wd < 4; wd++)
        {
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) word |= (uint32_t)((int)f[wd * 4 + e] & 0xff) << (8 * e);
            pk[wd] = (int)word;
        }
        *reinterpret_cast<v4i*>(static_cast<int8_t*>(out) + o) = pk;
    }
}

// 3x3, dilation 1: the fast path.  v_dot4_i32_i8 sums four byte products of one dword pair, so the four bytes must be
// four TAPS of one channel: a thread owns 4 channels of OUTS adjacent output pixels, loads each kernel row's input
// pixels as dwords (4 channels each), transposes them with 8 v_perm_b32 into "one channel, pixels x0..x0+3" and
// multiplies against weights packed per channel and kernel row as (w0, w1, w2, 0).  At stride 1 the same transposed
// dwords serve the next output pixel against the weights shifted one byte up, (0, w0, w1, w2), so OUTS = 2.
// Consecutive lanes are consecutive channel quads of a pixel: every load and store of a wavefront is a contiguous
// run.  The kernel is bound by VALU issue (index arithmetic + ~20 single-rounded fp32 instructions of requantising
// epilogue per output), so everything per-thread is amortised over as many outputs as the registers allow.
template<int STRIDE, int ROWS>
__global__ __launch_bounds__(256) void dwconv3x3_nhwc_kernel(const int8_t* __restrict__ x, const uint32_t* __restrict__ wrow /* [3][cp] */, DwNhwcGeom g,
                                                              const float* __restrict__ scale_in, const float* __restrict__ bias,
                                                              const float* __restrict__ scale_out, ncnnhip_activation act, void* __restrict__ out,
                                                              unsigned quads, unsigned quads_magic, unsigned xgroups, unsigned rowgroups, unsigned rowgroups_magic)
{
    constexpr int OUTS = STRIDE == 1 ? 2 : 1;
    constexpr int PIX = STRIDE == 1 ? 4 : 3;          // input pixels per kernel row
    constexpr int IN_ROWS = (ROWS - 1) * STRIDE + 3;  // input rows under ROWS output rows
    // blockIdx.y = (sample, group of ROWS output rows); within the rows a thread is (x group, channel quad), quads
    // fastest.  Each input row is loaded and transposed once and serves every output row of the group it lies under.
    // xg = r / quads by multiplication with ceil(2^32 / quads), exact here because r * quads < 2^32; the sample index
    // likewise (blockIdx.y * rowgroups < 2^32), on the scalar unit.
    const unsigned r = blockIdx.x * 256 + threadIdx.x;
    if (r >= xgroups * quads) return;
    unsigned xg = __umulhi(r, quads_magic);
    if (xg * quads > r) xg--;
    const unsigned q0 = (r - xg * quads) * 4;
    const unsigned ox0 = xg * OUTS;
    unsigned img = rowgroups == 1 ? blockIdx.y : __umulhi(blockIdx.y, rowgroups_magic);
    if (img * rowgroups > blockIdx.y) img--;
    const unsigned oy0 = (blockIdx.y - img * rowgroups) * ROWS;
    const int8_t* base = x + (size_t)img * g.h * g.w * g.cp + q0;
    const int y0 = (int)oy0 * STRIDE - g.pad_top, x0 = (int)ox0 * STRIDE - g.pad_left;
    const uint32_t padw = (uint32_t)(g.pad_byte & 0xff) * 0x01010101u;

    // column offsets (clamped into the image so that every load is unconditional) and their validity
    unsigned xoff[PIX];
    bool xin[PIX];
#pragma unroll
    for (int p = 0; p < PIX; p++)
    {
        const int xx = x0 + p;
        xin[p] = (unsigned)xx < (unsigned)g.w;
        xoff[p] = (unsigned)(xin[p] ? xx : 0) * (unsigned)g.cp;
    }

    // weights: 4 channels x (w0,w1,w2,0) per kernel row; shifted one byte up, (0,w0,w1,w2), for the second output pixel
    v4i wv[3], wv1[3];
#pragma unroll
    for (int ky = 0; ky < 3; ky++)
    {
        wv[ky] = *reinterpret_cast<const v4i*>(wrow + (size_t)ky * g.cp + q0);
#pragma unroll
        for (int c = 0; c < 4; c++) wv1[ky][c] = (int)((uint32_t)wv[ky][c] << 8);
    }

    int acc[ROWS][OUTS][4];
#pragma unroll
    for (int iy = 0; iy < IN_ROWS; iy++)
    {
        const int y = y0 + iy;
        const bool yin = (unsigned)y < (unsigned)g.h;
        const unsigned rowoff = (unsigned)(yin ? y : 0) * (unsigned)g.w * (unsigned)g.cp; // one sample < 2^31 bytes
        uint32_t d[4];
#pragma unroll
        for (int p = 0; p < PIX; p++)
        {
            const uint32_t v = *reinterpret_cast<const uint32_t*>(base + rowoff + xoff[p]);
            d[p] = (yin && xin[p]) ? v : padw;
        }
        if (PIX == 3) d[3] = 0;
        // 4x4 byte transpose: t[c] = (pixel0.c, pixel1.c, pixel2.c, pixel3.c)
        const uint32_t p01l = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u), p01h = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
        const uint32_t p23l = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u), p23h = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
        const uint32_t t[4] = {__builtin_amdgcn_perm(p23l, p01l, 0x05040100u), __builtin_amdgcn_perm(p23l, p01l, 0x07060302u),
                               __builtin_amdgcn_perm(p23h, p01h, 0x05040100u), __builtin_amdgcn_perm(p23h, p01h, 0x07060302u)};
#pragma unroll
        for (int ro = 0; ro < ROWS; ro++)
        {
            const int ky = iy - ro * STRIDE; // this input row is kernel row ky of output row ro (compile time)
            if (ky < 0 || ky > 2) continue;
#pragma unroll
            for (int c = 0; c < 4; c++)
            {
                // kernel row 0 is an output row's first contribution: it starts from a literal zero (no register to clear)
                acc[ro][0][c] = __builtin_amdgcn_sdot4((int)t[c], wv[ky][c], ky == 0 ? 0 : acc[ro][0][c], false);
                if (OUTS == 2) acc[ro][1][c] = __builtin_amdgcn_sdot4((int)t[c], wv1[ky][c], ky == 0 ? 0 : acc[ro][1][c], false);
            }
        }
    }

    // per-channel tables: one vector load each when the channel count is a multiple of 4 (uniform), else clamped scalars
    // Pad channels (from g.c up) get scale 0, bias -0 and output scale 0: whatever the activation, a finite value times a
    // zero output scale is a zero byte, so the int8 epilogues need no select per value (the fp32 one keeps its own).
    float s_in[4], s_b[4], s_out[4];
    if ((g.c & 3) == 0)
    {
        const bool real = q0 < (unsigned)g.c; // a quad is real or it is not
        const unsigned qc = real ? q0 : (unsigned)g.c - 4;
        const v4f a = *reinterpret_cast<const v4f*>(scale_in + qc);
        const v4f b = bias ? *reinterpret_cast<const v4f*>(bias + qc) : v4f{-0.f, -0.f, -0.f, -0.f}; // x + -0 = x for every x
        const v4f c = g.out_f32 ? v4f{0.f, 0.f, 0.f, 0.f} : *reinterpret_cast<const v4f*>(scale_out + qc);
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            s_in[e] = real ? a[e] : 0.f;
            s_b[e] = real ? b[e] : -0.f;
            s_out[e] = real ? c[e] : 0.f;
        }
    }
    else
    {
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            const bool real = (int)q0 + e < g.c;
            const int qc = real ? (int)q0 + e : g.c - 1;
            s_in[e] = real ? scale_in[qc] : 0.f;
            s_b[e] = (real && bias) ? bias[qc] : -0.f;
            s_out[e] = (real && !g.out_f32) ? scale_out[qc] : 0.f;
        }
    }
    // A clip whose operand cannot be NaN (finite tables: an int32 times a finite scale plus a finite bias is finite or
    // infinite) is max-then-min, two instructions for the reference's two compare-and-selects, with the same result.
    // If the clipped value times the output scale also stays below 2^31, float2int8 needs no out-of-range branch.
    // And with finite values the clip folds into the requantising clamp (clip_folds_into_requantise).
    const float clip_abs = fmaxf(fabsf(act.p0), fabsf(act.p1));
    bool finite_tables = fabsf(act.p0) < INFINITY && fabsf(act.p1) < INFINITY;
    float q_lo[4], q_hi[4];
#pragma unroll
    for (int e = 0; e < 4; e++)
    {
        finite_tables = finite_tables && fabsf(s_in[e]) < 0x1p90f && fabsf(s_b[e]) < 0x1p120f && mul_rn(clip_abs, fabsf(s_out[e])) < 2147483648.f
                        && clip_folds_into_requantise(act.p0, act.p1, s_out[e]);
        q_lo[e] = __builtin_amdgcn_fmed3f(mul_rn(act.p0, s_out[e]), -127.f, 127.f);
        q_hi[e] = __builtin_amdgcn_fmed3f(mul_rn(act.p1, s_out[e]), -127.f, 127.f);
    }
    const size_t off00 = (((size_t)img * g.outh + oy0) * g.outw + ox0) * g.cp + q0; // output (row 0, pixel 0) of this thread
    // no negative clamp bound (ReLU6 and its like): the rounding is one conversion (pack4_nonneg)
    auto emit = [&](auto clip_tag) {
        constexpr bool FAST_CLIP = decltype(clip_tag)::value > 0;
        constexpr bool NONNEG = decltype(clip_tag)::value > 1;
#pragma unroll
        for (int ro = 0; ro < ROWS; ro++)
#pragma unroll
        for (int o = 0; o < OUTS; o++)
        {
            const unsigned ox = ox0 + o, oy = oy0 + ro;
            if (ox >= (unsigned)g.outw || oy >= (unsigned)g.outh) continue;
            const size_t off = off00 + (size_t)(unsigned)((ro * g.outw + o) * g.cp); // (uniform: a scalar product, one 64-bit add)
            float f[4];
#pragma unroll
            for (int e = 0; e < 4; e++)
            {
                float v = add_rn(mul_rn((float)acc[ro][o][e], s_in[e]), s_b[e]);
                if (!FAST_CLIP)
                    v = apply_activation(v, act);
                else if (g.out_f32)
                    v = clip_not_nan(v, act.p0, act.p1); // (to int8: folded into the clamp below)
                f[e] = g.out_f32 ? v : mul_rn(v, s_out[e]);
            }
            if (!g.out_f32)
            {
                if (NONNEG)
                {
#pragma unroll
                    for (int e = 0; e < 4; e++) f[e] = __builtin_amdgcn_fmed3f(f[e], q_lo[e], q_hi[e]);
                }
                else if (FAST_CLIP)
                    float2int8_as_float_bounded_lanes_x4(f[0], f[1], f[2], f[3], q_lo, q_hi);
                else
                    float2int8_as_float_x4(f[0], f[1], f[2], f[3]);
            }
            if (g.out_f32)
            {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if ((int)q0 + e >= g.c) f[e] = 0.f;
                *reinterpret_cast<v4f*>(static_cast<float*>(out) + off) = v4f{f[0], f[1], f[2], f[3]};
            }
            else if (NONNEG)
                *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(out) + off) = pack4_nonneg(f[0], f[1], f[2], f[3]);
            else
                *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(out) + off) = pack4_quantised(f[0], f[1], f[2], f[3]);
        }
    };
    if (act.type == 3 && __all(finite_tables))
    {
        if (!g.out_f32 && __all(q_lo[0] >= 0.f && q_lo[1] >= 0.f && q_lo[2] >= 0.f && q_lo[3] >= 0.f))
            emit(std::integral_constant<int, 2>{});
        else
            emit(std::integral_constant<int, 1>{});
    }
    else
        emit(std::integral_constant<int, 0>{});
}

static inline int padded16(int c)
{
    return (c + 15) / 16 * 16;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_padded_channels(int c)
{
    return padded16(c);
}

int ncnnhip_chw_to_nhwc(const void* src_dev, int elemsize, int c, int hw, int batch, size_t cstep, size_t nstep, void* dst_dev, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && (elemsize == 1 || elemsize == 4), "ncnnhip_chw_to_nhwc: bad argument");
    NCNNHIP_REQUIRE(c > 0 && hw > 0 && batch > 0 && batch <= 65535 && cstep >= (size_t)hw, "ncnnhip_chw_to_nhwc: bad shape");
    const int cp = padded16(c);
    dim3 grid(ceil_div(hw, 64), ceil_div(cp, 64), batch);
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_chw_to_nhwc: too many channels");
    if (elemsize == 4)
        hipLaunchKernelGGL(chw_to_nhwc_kernel<float>, grid, dim3(256), 0, as_stream(stream), (const float*)src_dev, cstep, nstep, c, hw, cp, (float*)dst_dev);
    else
        hipLaunchKernelGGL(chw_to_nhwc_kernel<int8_t>, grid, dim3(256), 0, as_stream(stream), (const int8_t*)src_dev, cstep, nstep, c, hw, cp, (int8_t*)dst_dev);
    return launch_status("chw_to_nhwc_kernel");
}

int ncnnhip_chw_to_nhwc4_f32(const float* src_dev, int c, int hw, int batch, size_t cstep, size_t nstep, float* dst_dev, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && c >= 1 && c <= 4 && hw > 0 && batch > 0 && batch <= 65535 && cstep >= (size_t)hw, "ncnnhip_chw_to_nhwc4_f32: bad argument");
    hipLaunchKernelGGL(chw_to_nhwc4_f32_kernel, dim3(ceil_div(hw, 256), batch), dim3(256), 0, as_stream(stream), src_dev, cstep, nstep, c, hw, dst_dev);
    return launch_status("chw_to_nhwc4_f32_kernel");
}

int ncnnhip_widen_nhwc4_f32(const float* src_dev, float* dst_dev, size_t pixels, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && pixels > 0, "ncnnhip_widen_nhwc4_f32: bad argument");
    hipLaunchKernelGGL(widen_nhwc4_f32_kernel, dim3((unsigned)ceil_div((long long)pixels, 256)), dim3(256), 0, as_stream(stream), src_dev, dst_dev, pixels);
    return launch_status("widen_nhwc4_f32_kernel");
}

int ncnnhip_nhwc_to_chw(const void* src_dev, int elemsize, int c, int hw, int batch, void* dst_dev, size_t cstep, size_t nstep, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && (elemsize == 1 || elemsize == 4), "ncnnhip_nhwc_to_chw: bad argument");
    NCNNHIP_REQUIRE(c > 0 && hw > 0 && batch > 0 && batch <= 65535 && cstep >= (size_t)hw, "ncnnhip_nhwc_to_chw: bad shape");
    const int cp = padded16(c);
    dim3 grid(ceil_div(hw, 64), ceil_div(cp, 64), batch);
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_nhwc_to_chw: too many channels");
    if (elemsize == 4)
        hipLaunchKernelGGL(nhwc_to_chw_kernel<float>, grid, dim3(256), 0, as_stream(stream), (const float*)src_dev, c, hw, cp, (float*)dst_dev, cstep, nstep);
    else
        hipLaunchKernelGGL(nhwc_to_chw_kernel<int8_t>, grid, dim3(256), 0, as_stream(stream), (const int8_t*)src_dev, c, hw, cp, (int8_t*)dst_dev, cstep, nstep);
    return launch_status("nhwc_to_chw_kernel");
}

int ncnnhip_quantize_nhwc(const float* src_dev, int8_t* dst_dev, size_t npix, int c, const float* scales_dev, int nscales, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && scales_dev && c > 0 && (nscales == 1 || nscales == c), "ncnnhip_quantize_nhwc: bad argument");
    if (npix == 0) return NCNNHIP_OK;
    const int cp = padded16(c);
    const size_t chunks = npix * (size_t)(cp / 16);
    hipLaunchKernelGGL(quantize_nhwc_kernel, dim3(ceil_div((long long)chunks, 256)), dim3(256), 0, as_stream(stream), src_dev, dst_dev, chunks, c, cp, scales_dev, nscales);
    return launch_status("quantize_nhwc_kernel");
}

int ncnnhip_int8_to_f32(const int8_t* src_dev, float* dst_dev, size_t count, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev, "ncnnhip_int8_to_f32: null pointer");
    if (count == 0) return NCNNHIP_OK;
    hipLaunchKernelGGL(int8_to_f32_kernel, dim3(ceil_div((long long)count, 256)), dim3(256), 0, as_stream(stream), src_dev, dst_dev, count);
    return launch_status("int8_to_f32_kernel");
}

int ncnnhip_relu(const void* src_dev, void* dst_dev, int elemsize, size_t count, float slope, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && (elemsize == 1 || elemsize == 4), "ncnnhip_relu: bad argument");
    if (count == 0) return NCNNHIP_OK;
    if (elemsize == 1)
    {
        hipLaunchKernelGGL(relu_s8_kernel, dim3(ceil_div((long long)count, 256)), dim3(256), 0, as_stream(stream), (const int8_t*)src_dev, (int8_t*)dst_dev, count);
        return launch_status("relu_s8_kernel");
    }
    NCNNHIP_REQUIRE(count % 4 == 0, "ncnnhip_relu: fp32 element count must be a multiple of 4 (device blobs are padded to it)");
    hipLaunchKernelGGL(relu_f32_kernel, dim3(ceil_div((long long)(count / 4), 256)), dim3(256), 0, as_stream(stream), (const float*)src_dev, (float*)dst_dev, count / 4, slope);
    return launch_status("relu_f32_kernel");
}

int ncnnhip_scale(const float* src_dev, float* dst_dev, size_t count, float scale, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev, "ncnnhip_scale: null pointer");
    if (count == 0) return NCNNHIP_OK;
    hipLaunchKernelGGL(scale_f32_kernel, dim3(ceil_div((long long)count, 256)), dim3(256), 0, as_stream(stream), src_dev, dst_dev, count, scale);
    return launch_status("scale_f32_kernel");
}

int ncnnhip_eltwise(const float* const* srcs_dev, int nsrc, int op_type, const float* coeffs_host, int ncoeffs, float* dst_dev, size_t count, void* stream)
{
    NCNNHIP_REQUIRE(srcs_dev && dst_dev && nsrc >= 2 && op_type >= 0 && op_type <= 2, "ncnnhip_eltwise: bad argument");
    NCNNHIP_REQUIRE(count % 4 == 0, "ncnnhip_eltwise: element count must be a multiple of 4 (device blobs are padded to it)");
    const int weighted = op_type == 1 && ncoeffs != 0;
    NCNNHIP_REQUIRE(!weighted || (coeffs_host && ncoeffs >= nsrc), "ncnnhip_eltwise: one coefficient per input required");
    if (count == 0) return NCNNHIP_OK;
    const size_t n4 = count / 4;
    dim3 grid(ceil_div((long long)n4, 256));
    hipLaunchKernelGGL(eltwise_kernel, grid, dim3(256), 0, as_stream(stream), srcs_dev[0], srcs_dev[1], dst_dev, n4, op_type, weighted,
                       weighted ? coeffs_host[0] : 1.f, weighted ? coeffs_host[1] : 1.f, 1);
    for (int b = 2; b < nsrc; b++)
        hipLaunchKernelGGL(eltwise_kernel, grid, dim3(256), 0, as_stream(stream), (const float*)dst_dev, srcs_dev[b], dst_dev, n4, op_type, weighted, 1.f,
                           weighted ? coeffs_host[b] : 1.f, 0);
    return launch_status("eltwise_kernel");
}

int ncnnhip_pooling_nhwc(const ncnnhip_pool_desc* desc, const float* src_dev, float* dst_dev, void* stream)
{
    NCNNHIP_REQUIRE(desc && src_dev && dst_dev, "ncnnhip_pooling_nhwc: null pointer");
    const ncnnhip_pool_desc& d = *desc;
    NCNNHIP_REQUIRE(d.w > 0 && d.h > 0 && d.c > 0 && d.batch > 0 && (d.pooling_type == 0 || d.pooling_type == 1), "ncnnhip_pooling_nhwc: bad shape or type");
    const int cp = padded16(d.c);
    if (d.global_pooling)
    {
        NCNNHIP_REQUIRE(d.batch <= 65535, "ncnnhip_pooling_nhwc: batch above 65535");
        hipLaunchKernelGGL(global_pooling_nhwc_kernel, dim3(ceil_div(d.c, 64), d.batch), dim3(64), 0, as_stream(stream), src_dev, dst_dev, d.c, d.w * d.h, cp, d.pooling_type,
                           (int8_t*)0, 0.f);
        return launch_status("global_pooling_nhwc_kernel");
    }
    NCNNHIP_REQUIRE(d.kernel_w > 0 && d.kernel_h > 0 && d.stride_w > 0 && d.stride_h > 0 && d.outw > 0 && d.outh > 0, "ncnnhip_pooling_nhwc: bad window");
    // every window must start inside the padded image the reference would build
    NCNNHIP_REQUIRE(d.pad_top >= 0 && d.pad_left >= 0, "ncnnhip_pooling_nhwc: negative pads");
    PoolGeom g;
    g.w = d.w;
    g.h = d.h;
    g.cp = cp;
    g.outw = d.outw;
    g.outh = d.outh;
    g.kw = d.kernel_w;
    g.kh = d.kernel_h;
    g.sw = d.stride_w;
    g.sh = d.stride_h;
    g.pad_top = d.pad_top;
    g.pad_left = d.pad_left;
    g.type = d.pooling_type;
    g.count_include_pad = d.avgpool_count_include_pad;
    // all four zero: the image itself.  Any other rectangle is taken as it is, an empty one too (pad parameters that leave
    // nothing to count: the reference then divides 0 by 0)
    const bool own_rect = d.count_x0 != 0 || d.count_x1 != 0 || d.count_y0 != 0 || d.count_y1 != 0;
    g.cx0 = own_rect ? d.count_x0 : 0;
    g.cx1 = own_rect ? d.count_x1 : d.w;
    g.cy0 = own_rect ? d.count_y0 : 0;
    g.cy1 = own_rect ? d.count_y1 : d.h;
    const size_t total = (size_t)d.batch * d.outh * d.outw * (cp / 4);
    hipLaunchKernelGGL(pooling_nhwc_kernel, dim3(ceil_div((long long)total, 256)), dim3(256), 0, as_stream(stream), src_dev, dst_dev, g, total);
    return launch_status("pooling_nhwc_kernel");
}

int ncnnhip_maxpool_nhwc_int8(const ncnnhip_pool_desc* desc, const int8_t* src_dev, int8_t* dst_dev, void* stream)
{
    NCNNHIP_REQUIRE(desc && src_dev && dst_dev, "ncnnhip_maxpool_nhwc_int8: null pointer");
    const ncnnhip_pool_desc& d = *desc;
    NCNNHIP_REQUIRE(d.w > 0 && d.h > 0 && d.c > 0 && d.batch > 0 && d.pooling_type == 0 && !d.global_pooling, "ncnnhip_maxpool_nhwc_int8: windowed max pooling only");
    NCNNHIP_REQUIRE(d.kernel_w > 0 && d.kernel_h > 0 && d.stride_w > 0 && d.stride_h > 0 && d.outw > 0 && d.outh > 0, "ncnnhip_maxpool_nhwc_int8: bad window");
    NCNNHIP_REQUIRE(d.pad_top >= 0 && d.pad_left >= 0, "ncnnhip_maxpool_nhwc_int8: negative pads");
    NCNNHIP_REQUIRE(((reinterpret_cast<uintptr_t>(src_dev) | reinterpret_cast<uintptr_t>(dst_dev)) & 15) == 0, "ncnnhip_maxpool_nhwc_int8: blobs must be 16-byte aligned");
    PoolGeom g;
    g.w = d.w;
    g.h = d.h;
    g.cp = padded16(d.c);
    g.outw = d.outw;
    g.outh = d.outh;
    g.kw = d.kernel_w;
    g.kh = d.kernel_h;
    g.sw = d.stride_w;
    g.sh = d.stride_h;
    g.pad_top = d.pad_top;
    g.pad_left = d.pad_left;
    g.type = 0;
    g.count_include_pad = 0;
    const unsigned groups = (unsigned)g.cp / 16;
    NCNNHIP_REQUIRE(d.batch <= 65535 && d.outh <= 65535 && (unsigned long long)d.outw * groups * groups < (1ull << 32), "ncnnhip_maxpool_nhwc_int8: extent too large");
    const unsigned groups_magic = groups > 1 ? (unsigned)(((1ull << 32) + groups - 1) / groups) : 0u;
    hipLaunchKernelGGL(maxpool_nhwc_s8_kernel, dim3(ceil_div((long long)d.outw * groups, 256), (unsigned)d.outh, (unsigned)d.batch), dim3(256), 0, as_stream(stream),
                       src_dev, dst_dev, g, groups, groups_magic);
    return launch_status("maxpool_nhwc_s8_kernel");
}

int ncnnhip_global_pooling_nhwc_quantised(const ncnnhip_pool_desc* desc, const float* src_dev, float scale, int8_t* dst_dev, void* stream)
{
    NCNNHIP_REQUIRE(desc && src_dev && dst_dev, "ncnnhip_global_pooling_nhwc_quantised: null pointer");
    const ncnnhip_pool_desc& d = *desc;
    NCNNHIP_REQUIRE(d.w > 0 && d.h > 0 && d.c > 0 && d.batch > 0 && d.batch <= 65535 && (d.pooling_type == 0 || d.pooling_type == 1),
                    "ncnnhip_global_pooling_nhwc_quantised: bad shape or pooling type");
    hipLaunchKernelGGL(global_pooling_nhwc_kernel, dim3(ceil_div(d.c, 64), d.batch), dim3(64), 0, as_stream(stream), src_dev, (float*)0, d.c, d.w * d.h, padded16(d.c),
                       d.pooling_type, dst_dev, scale);
    return launch_status("global_pooling_nhwc_kernel");
}

int ncnnhip_softmax(const float* src_dev, float* dst_dev, int count, int batch, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && count > 0 && batch > 0, "ncnnhip_softmax: bad argument");
    hipLaunchKernelGGL(softmax_kernel, dim3(batch), dim3(256), 0, as_stream(stream), src_dev, dst_dev, count);
    return launch_status("softmax_kernel");
}

static size_t dwconv_packed_bytes(int channels, int kernel_w, int kernel_h)
{
    const size_t cp = (size_t)padded16(channels);
    // [taps][cp] bytes, then for a 3x3 kernel [3][cp] dwords holding each kernel row as (w0, w1, w2, 0)
    return (size_t)kernel_w * kernel_h * cp + ((kernel_w == 3 && kernel_h == 3) ? 3 * cp * 4 : 0);
}

int ncnnhip_dwconv_packed_bytes(int channels, int kernel_w, int kernel_h, size_t* bytes)
{
    NCNNHIP_REQUIRE(channels > 0 && kernel_w > 0 && kernel_h > 0 && bytes, "ncnnhip_dwconv_packed_bytes: bad argument");
    *bytes = dwconv_packed_bytes(channels, kernel_w, kernel_h);
    return NCNNHIP_OK;
}

int ncnnhip_dwconv_pack_weights(int channels, int kernel_w, int kernel_h, const int8_t* weight_host, int8_t* packed_host)
{
    NCNNHIP_REQUIRE(channels > 0 && kernel_w > 0 && kernel_h > 0 && weight_host && packed_host, "ncnnhip_dwconv_pack_weights: bad argument");
    const int cp = padded16(channels), taps = kernel_w * kernel_h;
    for (int t = 0; t < taps; t++)
        for (int q = 0; q < cp; q++) packed_host[(size_t)t * cp + q] = q < channels ? weight_host[(size_t)q * taps + t] : (int8_t)0;
    if (kernel_w == 3 && kernel_h == 3)
    {
        int8_t* rows = packed_host + (size_t)taps * cp;
        for (int ky = 0; ky < 3; ky++)
            for (int q = 0; q < cp; q++)
                for (int kx = 0; kx < 4; kx++) rows[((size_t)ky * cp + q) * 4 + kx] = (q < channels && kx < 3) ? weight_host[(size_t)q * 9 + ky * 3 + kx] : (int8_t)0;
    }
    return NCNNHIP_OK;
}

int ncnnhip_dwconv_int8_nhwc(const ncnnhip_conv_desc* desc, const int8_t* nhwc_dev, const int8_t* packed_weight_dev, const float* scale_in_dev,
                             const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act, void* out_nhwc_dev, void* stream)
{
    NCNNHIP_REQUIRE(desc && nhwc_dev && packed_weight_dev && scale_in_dev && out_nhwc_dev, "ncnnhip_dwconv_int8_nhwc: null pointer");
    const ncnnhip_conv_desc& d = *desc;
    NCNNHIP_REQUIRE(d.group == d.c && d.num_output == d.c, "ncnnhip_dwconv_int8_nhwc: needs channels == group == num_output");
    int outw, outh;
    int ret = ncnnhip_conv_out_shape(desc, &outw, &outh);
    if (ret) return ret;
    int pad_top, pad_left;
    ret = ncnnhip_conv_resolved_pads(desc, &pad_top, &pad_left);
    if (ret) return ret;
    DwNhwcGeom g;
    g.w = d.w;
    g.h = d.h;
    g.c = d.c;
    g.cp = padded16(d.c);
    g.outw = outw;
    g.outh = outh;
    g.kw = d.kernel_w;
    g.kh = d.kernel_h;
    g.dw = d.dilation_w;
    g.dh = d.dilation_h;
    g.sw = d.stride_w;
    g.sh = d.stride_h;
    g.pad_top = pad_top;
    g.pad_left = pad_left;
    g.pad_byte = (int)(signed char)d.pad_value;
    g.out_f32 = scale_out_dev ? 0 : 1;
    // the fast path indexes output rows with blockIdx.y and one sample with 31 bits; anything larger takes the generic kernel
    const bool fits_fast = (size_t)d.batch * outh <= 65535 && (size_t)d.batch * outh * outw < (1ull << 32) && (size_t)outw * (g.cp / 4) * (g.cp / 4) < (1ull << 32) &&
                           (size_t)d.h * d.w * g.cp < (1ull << 31);
    if (fits_fast && d.kernel_w == 3 && d.kernel_h == 3 && d.dilation_w == 1 && d.dilation_h == 1 && d.stride_w == d.stride_h && (d.stride_w == 1 || d.stride_w == 2))
    {
        const uint32_t* wrow = reinterpret_cast<const uint32_t*>(packed_weight_dev + (size_t)9 * g.cp);
        const unsigned quads = (unsigned)g.cp / 4;
        const unsigned xgroups = (unsigned)ceil_div(outw, d.stride_w == 1 ? 2 : 1);
        const size_t row_threads = (size_t)xgroups * quads;
        const unsigned quads_magic = (unsigned)(((1ull << 32) + quads - 1) / quads);
        // up to four output rows per thread share their input rows; fewer when that leaves too few threads for the chip
        int rows_per_thread = 1;
        for (int rp = 2; rp <= 4; rp *= 2)
            if ((size_t)d.batch * ceil_div(outh, rp) * row_threads >= 256 * 256 * 2) rows_per_thread = rp;
        const unsigned rowgroups = (unsigned)ceil_div(outh, rows_per_thread);
        const unsigned rowgroups_magic = rowgroups > 1 ? (unsigned)((1ull << 32) / rowgroups + 1) : 0u;
        dim3 grid3(ceil_div((long long)row_threads, 256), (unsigned)((size_t)d.batch * rowgroups));
#define LAUNCH_DW(S_, R_)                                                                                                                                   \
    hipLaunchKernelGGL((dwconv3x3_nhwc_kernel<S_, R_>), grid3, dim3(256), 0, as_stream(stream), nhwc_dev, wrow, g, scale_in_dev, bias_dev, scale_out_dev, act, \
                       out_nhwc_dev, quads, quads_magic, xgroups, rowgroups, rowgroups_magic)
        if (d.stride_w == 1)
        {
            if (rows_per_thread == 4)
                LAUNCH_DW(1, 4);
            else if (rows_per_thread == 2)
                LAUNCH_DW(1, 2);
            else
                LAUNCH_DW(1, 1);
        }
        else
        {
            if (rows_per_thread == 4)
                LAUNCH_DW(2, 4);
            else if (rows_per_thread == 2)
                LAUNCH_DW(2, 2);
            else
                LAUNCH_DW(2, 1);
        }
#undef LAUNCH_DW
        return launch_status("dwconv3x3_nhwc_kernel");
    }
    const size_t total = (size_t)d.batch * outh * outw * (g.cp / 16);
    hipLaunchKernelGGL(dwconv_nhwc_kernel, dim3(ceil_div((long long)total, 256)), dim3(256), 0, as_stream(stream), nhwc_dev, packed_weight_dev, g, scale_in_dev,
                       bias_dev, scale_out_dev, act, out_nhwc_dev, total);
    return launch_status("dwconv_nhwc_kernel");
}

} // extern "C"
