// A depthwise convolution and the 1x1 convolution that consumes it, in one launch: the pair that closes an inverted-residual
// block (ConvolutionDepthWise::forward_int8, src/layer/convolutiondepthwise.cpp:505-559, requantised to int8, then
// Convolution::forward_int8 with a 1x1 kernel, src/layer/convolution.cpp:383-508).  The reference requantises between the
// two layers and so does this kernel: the depthwise result of a block of 16 pixels is computed, requantised and kept in LDS
// as int8, exactly the bytes the depthwise layer would have written, and the 1x1 convolution reads it from there.
//
// It exists for small feature maps, where a forward pass is a chain of launches that each use a fraction of the chip: one
// launch less per block, and no round trip of the intermediate blob.  One workgroup = 16 output pixels x 64 output
// channels; the depthwise tile is recomputed by every channel group (cheap at these sizes, prohibitive on large maps: the
// caller picks).
//   phase 1: thread = 16 channels of one pixel (the generic depthwise kernel's arithmetic), result into LDS [16][Kp + 16];
//   phase 2: wavefront = one block of 16 output channels: v_mfma_i32_16x16x64_i8 with the weights' rows as the A operand
//            (16 bytes per lane from global memory, rows of Kp bytes, zero-filled from the input's channels up) and the
//            pixels as the B operand (16 bytes per lane from LDS), so that a lane ends up with 4 consecutive channels of one
//            pixel: one dword of the int8 output or one 16-byte piece of the fp32 output;
//   epilogue: the convolution's (scale_in, bias, activation, requantise) or its fused tail (residual, ReLU, int8 copy).
#include <string.h>

#include <atomic>

#include "common.h"
#include "conv_nhwc.h"

namespace ncnnhip {

typedef int v4i_dp __attribute__((ext_vector_type(4)));
typedef float v4f_dp __attribute__((ext_vector_type(4)));

struct DwPwGeom
{
    int w, h, cp, c, outw, outh;
    int kw, kh, dw, dh, sw, sh, pad_top, pad_left;
    int pad_byte;
    int npix; // batch * outh * outw
    int Kp;   // bytes of one weight row of the 1x1 convolution: cp rounded up to 64
    int cout, out_cp;
};

static constexpr int DP_PIX = 16;

__global__ __launch_bounds__(256) void dwconv_pointwise_int8_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ dw_w /* [kh*kw][cp] */, DwPwGeom g,
                                                                     const float* __restrict__ dw_scale_in, const float* __restrict__ dw_bias,
                                                                     const float* __restrict__ dw_scale_out, ncnnhip_activation dw_act,
                                                                     const int8_t* __restrict__ rows /* [padded16(cout)][Kp] */, const float* __restrict__ scale_in,
                                                                     const float* __restrict__ bias, const float* __restrict__ scale_out, ncnnhip_activation act,
                                                                     void* __restrict__ out, const float* __restrict__ residual, int relu_after,
                                                                     int8_t* __restrict__ q8_out, float q8_scale)
{
    extern __shared__ __align__(16) int8_t dp_tile[]; // [DP_PIX][Kp + 16]: the rows start 16 bytes apart in the banks
    const int pitch = g.Kp + 16;
    const int tid = threadIdx.x;
    const int n0 = blockIdx.x * DP_PIX;

    // ---- phase 1: the depthwise layer's output for pixels n0 .. n0+15, all channels, as int8
    {
        const int chunks = g.cp >> 4, kchunks = g.Kp >> 4;
        const int padw = (int)((uint32_t)(g.pad_byte & 0xff) * 0x01010101u);
        const int per_img = g.outh * g.outw;
        for (int item = tid; item < DP_PIX * kchunks; item += 256)
        {
            const int p = item / kchunks, chunk = item - p * kchunks;
            const int n = n0 + p;
            v4i_dp pk = {0, 0, 0, 0};
            if (n < g.npix && chunk < chunks)
            {
                const int img = n / per_img, rest = n - img * per_img;
                const int oy = rest / g.outw, ox = rest - oy * g.outw;
                const int q0 = chunk * 16;
                const int8_t* base = x + (size_t)img * g.h * g.w * g.cp + q0;
                const int y0 = oy * g.sh - g.pad_top, x0 = ox * g.sw - g.pad_left;
                int acc[16];
#pragma unroll
                for (int e = 0; e < 16; e++) acc[e] = 0;
                for (int ky = 0; ky < g.kh; ky++)
                    for (int kx = 0; kx < g.kw; kx++)
                    {
                        const int y = y0 + ky * g.dh, xx = x0 + kx * g.dw;
                        const bool in = (unsigned)y < (unsigned)g.h && (unsigned)xx < (unsigned)g.w;
                        v4i_dp v = *reinterpret_cast<const v4i_dp*>(base + (in ? ((size_t)y * g.w + xx) * g.cp : (size_t)0));
                        if (!in) v = v4i_dp{padw, padw, padw, padw};
                        const v4i_dp wv = *reinterpret_cast<const v4i_dp*>(dw_w + (size_t)(ky * g.kw + kx) * g.cp + q0);
#pragma unroll
                        for (int wd = 0; wd < 4; wd++)
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[wd * 4 + e] += (int)(int8_t)(v[wd] >> (8 * e)) * (int)(int8_t)(wv[wd] >> (8 * e));
                    }
#pragma unroll
                for (int wd = 0; wd < 4; wd++)
                {
                    uint32_t word = 0;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                    {
                        const int q = q0 + wd * 4 + e;
                        float r = 0.f;
                        if (q < g.c)
                        {
                            r = mul_rn((float)acc[wd * 4 + e], dw_scale_in[q]);
                            if (dw_bias) r = add_rn(r, dw_bias[q]);
                            r = apply_activation(r, dw_act);
                            r = float2int8_as_float(mul_rn(r, dw_scale_out[q]));
                        }
                        word |= (uint32_t)((int)r & 0xff) << (8 * e);
                    }
                    pk[wd] = (int)word;
                }
            }
            *reinterpret_cast<v4i_dp*>(dp_tile + (size_t)p * pitch + chunk * 16) = pk;
        }
    }
    __syncthreads();

    // ---- phase 2: 16 pixels x 16 output channels per wavefront
    const int lane = tid & 63, wave = tid >> 6, c16 = lane & 15, q = lane >> 4;
    const int cb = blockIdx.y * 4 + wave;
    if (cb * 16 >= g.out_cp) return;
    v4i_dp acc = {0, 0, 0, 0};
    {
        const int8_t* wr = rows + (size_t)(cb * 16 + c16) * g.Kp + q * 16;
        const int8_t* tp = dp_tile + (size_t)c16 * pitch + q * 16;
        const int ksteps = g.Kp >> 6;
        for (int ks = 0; ks < ksteps; ks++)
        {
            const v4i_dp a = *reinterpret_cast<const v4i_dp*>(wr + ks * 64);
            const v4i_dp b = *reinterpret_cast<const v4i_dp*>(tp + ks * 64);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc, 0, 0, 0);
        }
    }
    // acc[r]: channel cb*16 + 4q + r of pixel n0 + c16
    const int n = n0 + c16;
    if (n >= g.npix) return;
    const int ch0 = cb * 16 + 4 * q;
    const size_t o = (size_t)n * g.out_cp + ch0;
    float f[4];
#pragma unroll
    for (int r = 0; r < 4; r++)
    {
        const int ch = ch0 + r;
        float v = 0.f;
        if (ch < g.cout)
        {
            v = mul_rn((float)acc[r], scale_in[ch]);
            if (bias) v = add_rn(v, bias[ch]);
            v = apply_activation(v, act);
            if (scale_out) v = float2int8_as_float(mul_rn(v, scale_out[ch]));
        }
        f[r] = v;
    }
    if (scale_out)
    {
        uint32_t word = 0;
#pragma unroll
        for (int r = 0; r < 4; r++) word |= (uint32_t)((int)f[r] & 0xff) << (8 * r);
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(out) + o) = word;
        return;
    }
    if (residual)
    {
        const v4f_dp rv = *reinterpret_cast<const v4f_dp*>(residual + o);
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (ch0 + r < g.cout) f[r] = add_rn(f[r], rv[r]);
    }
    if (relu_after)
    {
#pragma unroll
        for (int r = 0; r < 4; r++) f[r] = f[r] < 0.f ? 0.f : f[r]; // the ReLU layer's statement (src/layer/relu.cpp:36-37): a NaN stays
    }
    *reinterpret_cast<v4f_dp*>(static_cast<float*>(out) + o) = v4f_dp{f[0], f[1], f[2], f[3]};
    if (q8_out)
    {
        uint32_t word = 0;
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const float qv = ch0 + r < g.cout ? float2int8_as_float(mul_rn(f[r], q8_scale)) : 0.f;
            word |= (uint32_t)((int)qv & 0xff) << (8 * r);
        }
        *reinterpret_cast<uint32_t*>(q8_out + o) = word;
    }
}

static inline int round_up_int(int v, int m)
{
    return (v + m - 1) / m * m;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_dwconv_pointwise_supported(const ncnnhip_conv_desc* dw_desc, int num_output)
{
    if (!dw_desc || num_output < 1) return 0;
    const ncnnhip_conv_desc& d = *dw_desc;
    if (d.group != d.c || d.num_output != d.c || d.c < 1 || d.batch < 1) return 0;
    int outw = 0, outh = 0;
    if (ncnnhip_conv_out_shape(dw_desc, &outw, &outh) != NCNNHIP_OK) return 0;
    const int Kp = round_up_int(ncnnhip_padded_channels(d.c), 64);
    if (Kp > 4096) return 0; // 16 x (Kp + 16) bytes of LDS
    if ((long long)d.batch * outh * outw > (1ll << 30) || (size_t)d.h * d.w * ncnnhip_padded_channels(d.c) >= ((size_t)1 << 31)) return 0;
    return 1;
}

int ncnnhip_dwconv_pointwise_packed_bytes(int channels, int num_output, size_t* bytes)
{
    NCNNHIP_REQUIRE(channels >= 1 && num_output >= 1 && bytes, "ncnnhip_dwconv_pointwise_packed_bytes: bad argument");
    *bytes = (size_t)ncnnhip_padded_channels(num_output) * (size_t)round_up_int(ncnnhip_padded_channels(channels), 64);
    return NCNNHIP_OK;
}

int ncnnhip_dwconv_pointwise_pack_weights(int channels, int num_output, const int8_t* weight_host, int8_t* packed_host)
{
    NCNNHIP_REQUIRE(channels >= 1 && num_output >= 1 && weight_host && packed_host, "ncnnhip_dwconv_pointwise_pack_weights: bad argument");
    const size_t Kp = (size_t)round_up_int(ncnnhip_padded_channels(channels), 64);
    const size_t rows = (size_t)ncnnhip_padded_channels(num_output);
    memset(packed_host, 0, rows * Kp);
    for (int p = 0; p < num_output; p++) memcpy(packed_host + (size_t)p * Kp, weight_host + (size_t)p * channels, (size_t)channels);
    return NCNNHIP_OK;
}

int ncnnhip_dwconv_pointwise_int8(const ncnnhip_conv_desc* dw_desc, const int8_t* nhwc_dev, const int8_t* dw_packed_weight_dev, const float* dw_scale_in_dev,
                                  const float* dw_bias_dev, const float* dw_scale_out_dev, ncnnhip_activation dw_act, int num_output,
                                  const int8_t* pointwise_rows_dev, const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev,
                                  ncnnhip_activation act, void* out_nhwc_dev, const ncnnhip_conv_fusion* fusion, void* stream)
{
    NCNNHIP_REQUIRE(dw_desc && nhwc_dev && dw_packed_weight_dev && dw_scale_in_dev && dw_scale_out_dev && pointwise_rows_dev && scale_in_dev && out_nhwc_dev,
                    "ncnnhip_dwconv_pointwise_int8: null pointer");
    NCNNHIP_REQUIRE(ncnnhip_dwconv_pointwise_supported(dw_desc, num_output), "ncnnhip_dwconv_pointwise_int8: shape not supported");
    NCNNHIP_REQUIRE(!(fusion && scale_out_dev), "ncnnhip_dwconv_pointwise_int8: the fused tail belongs to the fp32 output");
    const ncnnhip_conv_desc& d = *dw_desc;
    int outw = 0, outh = 0, pad_top = 0, pad_left = 0;
    int ret = ncnnhip_conv_out_shape(dw_desc, &outw, &outh);
    if (ret) return ret;
    ret = ncnnhip_conv_resolved_pads(dw_desc, &pad_top, &pad_left);
    if (ret) return ret;
    DwPwGeom g;
    g.w = d.w;
    g.h = d.h;
    g.c = d.c;
    g.cp = ncnnhip_padded_channels(d.c);
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
    g.npix = d.batch * outh * outw;
    g.Kp = round_up_int(g.cp, 64);
    g.cout = num_output;
    g.out_cp = ncnnhip_padded_channels(num_output);
    const uintptr_t al = reinterpret_cast<uintptr_t>(nhwc_dev) | reinterpret_cast<uintptr_t>(dw_packed_weight_dev) | reinterpret_cast<uintptr_t>(pointwise_rows_dev)
                         | reinterpret_cast<uintptr_t>(out_nhwc_dev) | reinterpret_cast<uintptr_t>(fusion ? fusion->residual_dev : nullptr)
                         | reinterpret_cast<uintptr_t>(fusion ? fusion->quantised_out_dev : nullptr);
    NCNNHIP_REQUIRE((al & 15) == 0, "ncnnhip_dwconv_pointwise_int8: operands must be 16-byte aligned");
    const size_t lds = (size_t)DP_PIX * (size_t)(g.Kp + 16);
    static std::atomic<unsigned char> raised[64];
    if (lds > 48 * 1024)
    {
        int device = 0;
        NCNNHIP_CHECK(hipGetDevice(&device));
        if (device < 0 || device >= 64 || !raised[device].load(std::memory_order_acquire))
        {
            NCNNHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(dwconv_pointwise_int8_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
            if (device >= 0 && device < 64) raised[device].store(1, std::memory_order_release);
        }
    }
    const dim3 grid((unsigned)ceil_div(g.npix, DP_PIX), (unsigned)ceil_div(g.out_cp, 64));
    hipLaunchKernelGGL(dwconv_pointwise_int8_kernel, grid, dim3(256), lds, as_stream(stream), nhwc_dev, dw_packed_weight_dev, g, dw_scale_in_dev, dw_bias_dev,
                       dw_scale_out_dev, dw_act, pointwise_rows_dev, scale_in_dev, bias_dev, scale_out_dev, act, out_nhwc_dev,
                       fusion ? fusion->residual_dev : nullptr, fusion ? fusion->relu_after : 0, fusion ? fusion->quantised_out_dev : nullptr,
                       fusion ? fusion->quantise_scale : 0.f);
    return launch_status("dwconv_pointwise_int8_kernel");
}

} // extern "C"
