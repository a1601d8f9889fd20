// int8 Convolution (implicit GEMM on the matrix cores) and ConvolutionDepthWise (direct,
// bandwidth-bound) with the fused dequantise / requantise epilogue.
#include "epilogues.h"
#include "mfma_tile.h"

namespace ncnnhip {

struct ResolvedPads
{
    int top, bottom, left, right;
};

// Padding as Convolution::make_padding resolves it: literal pads, or SAME_UPPER (-233) /
// SAME_LOWER (-234) computed from the kernel extent and stride.
static ResolvedPads resolve_pads(const ncnnhip_conv_desc& d)
{
    ResolvedPads p = {0, 0, 0, 0};
    const int kext_w = d.dilation_w * (d.kernel_w - 1) + 1;
    const int kext_h = d.dilation_h * (d.kernel_h - 1) + 1;
    if (d.pad_left > 0 || d.pad_right > 0 || d.pad_top > 0 || d.pad_bottom > 0)
    {
        p.top = d.pad_top;
        p.bottom = d.pad_bottom;
        p.left = d.pad_left;
        p.right = d.pad_right;
        return p;
    }
    const bool upper = d.pad_left == -233 && d.pad_right == -233 && d.pad_top == -233 && d.pad_bottom == -233;
    const bool lower = d.pad_left == -234 && d.pad_right == -234 && d.pad_top == -234 && d.pad_bottom == -234;
    if (upper || lower)
    {
        const int wpad = kext_w + (d.w - 1) / d.stride_w * d.stride_w - d.w;
        const int hpad = kext_h + (d.h - 1) / d.stride_h * d.stride_h - d.h;
        if (wpad > 0 || hpad > 0)
        {
            const int hs = hpad / 2, hl = hpad - hpad / 2;
            const int ws = wpad / 2, wl = wpad - wpad / 2;
            p.top = upper ? hs : hl;
            p.bottom = upper ? hl : hs;
            p.left = upper ? ws : wl;
            p.right = upper ? wl : ws;
        }
    }
    return p;
}

static int check_desc(const ncnnhip_conv_desc* d, const char* who)
{
    NCNNHIP_REQUIRE(d, "%s: null descriptor", who);
    NCNNHIP_REQUIRE(d->w >= 1 && d->h >= 1 && d->c >= 1 && d->batch >= 1 && d->num_output >= 1, "%s: bad blob shape", who);
    NCNNHIP_REQUIRE(d->kernel_w >= 1 && d->kernel_h >= 1 && d->dilation_w >= 1 && d->dilation_h >= 1 && d->stride_w >= 1 && d->stride_h >= 1,
                    "%s: bad kernel geometry", who);
    NCNNHIP_REQUIRE(d->kernel_h * d->dilation_h < 32767 && d->kernel_w * d->dilation_w < 32767, "%s: kernel extent too large", who);
    return NCNNHIP_OK;
}

template<int BM, int BN>
__global__ __launch_bounds__(256) void conv_tile_kernel(DenseOperand wgt, Im2colOperand src, ConvEpilogue epi, int cout_g, int npix, int K,
                                                         size_t weight_group_stride)
{
    const int g = blockIdx.z;
    wgt.base += (size_t)g * weight_group_stride;
    src.group_channel0 = g * src.cin_g;
    epi.out_channel0 = g * cout_g;
    mfma_tile_body<BM, BN, Im2colOperand, ConvEpilogue>(wgt, src, epi, cout_g, npix, K, blockIdx.y * BM, blockIdx.x * BN);
}

// Depthwise: one thread per output pixel, channel and image from the grid.  The kernel taps of
// the channel sit in registers; traffic is the int8 input (read through L1/L2, each byte reused
// by up to kh*kw neighbours) and one output element per thread.
struct DwParams
{
    const int8_t* x;
    size_t x_cstep, x_nstep;
    int w, h;
    int kw, kh, dw, dh, sw, sh;
    int pad_top, pad_left;
    int outw, outh;
    int pad_byte;
    const int8_t* weight;
    const float* scale_in;
    const float* bias;
    const float* scale_out;
    ncnnhip_activation act;
    void* out;
    size_t out_cstep, out_nstep;
    int32_t* acc_out;
    int channels;
};

template<int KW, int KH>
__global__ __launch_bounds__(256) void dwconv_kernel(DwParams p)
{
    const int ch = blockIdx.y;
    const int img = blockIdx.z;
    const int pix = blockIdx.x * 256 + threadIdx.x;
    const int kw = KW ? KW : p.kw;
    const int kh = KH ? KH : p.kh;
    if (pix >= p.outw * p.outh) return;
    const int oy = pix / p.outw;
    const int ox = pix - oy * p.outw;
    const int iy0 = oy * p.sh - p.pad_top;
    const int ix0 = ox * p.sw - p.pad_left;
    const int8_t* xc = p.x + (size_t)img * p.x_nstep + (size_t)ch * p.x_cstep;
    const int8_t* wc = p.weight + (size_t)ch * kw * kh;

    int acc = 0;
#pragma unroll
    for (int ky = 0; ky < kh; ky++)
    {
        const int iy = iy0 + ky * p.dh;
        const bool yok = (unsigned)iy < (unsigned)p.h;
#pragma unroll
        for (int kx = 0; kx < kw; kx++)
        {
            const int ix = ix0 + kx * p.dw;
            const int v = (yok && (unsigned)ix < (unsigned)p.w) ? (int)xc[iy * p.w + ix] : p.pad_byte;
            acc += v * (int)wc[ky * kw + kx];
        }
    }

    const size_t plane = (size_t)p.outw * p.outh;
    if (p.acc_out) p.acc_out[((size_t)img * p.channels + ch) * plane + pix] = acc;
    float f = mul_rn((float)acc, p.scale_in[ch]);
    if (p.bias) f = add_rn(f, p.bias[ch]);
    f = apply_activation(f, p.act);
    const size_t o = (size_t)img * p.out_nstep + (size_t)ch * p.out_cstep + pix;
    if (p.scale_out)
        static_cast<int8_t*>(p.out)[o] = (int8_t)float2int8(mul_rn(f, p.scale_out[ch]));
    else
        static_cast<float*>(p.out)[o] = f;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_conv_out_shape(const ncnnhip_conv_desc* desc, int* outw, int* outh)
{
    int ret = check_desc(desc, "ncnnhip_conv_out_shape");
    if (ret) return ret;
    const ResolvedPads p = resolve_pads(*desc);
    // A SAME mode gives a negative border where the kernel's extent is below the stride in one dimension while the other
    // dimension needs a border (3 x 1 at stride 3 on 37 x 20: bottom = -1).  The reference's border copy then writes every
    // source row into a blob with fewer rows (src/layer/padding.cpp:62-87), out of bounds and with a result that depends on
    // the order its threads run in: no result to reproduce, so the layer is refused.
    NCNNHIP_REQUIRE(p.top >= 0 && p.bottom >= 0 && p.left >= 0 && p.right >= 0,
                    "convolution: the padding mode resolves to a negative border (top %d bottom %d left %d right %d): kernel extent below the stride in one "
                    "dimension, a border needed in the other; the reference's border copy runs out of bounds for such a layer", p.top, p.bottom, p.left, p.right);
    const int W = desc->w + p.left + p.right;
    const int H = desc->h + p.top + p.bottom;
    const int ow = (W - (desc->dilation_w * (desc->kernel_w - 1) + 1)) / desc->stride_w + 1;
    const int oh = (H - (desc->dilation_h * (desc->kernel_h - 1) + 1)) / desc->stride_h + 1;
    NCNNHIP_REQUIRE(ow >= 1 && oh >= 1, "convolution output is empty (%d x %d)", ow, oh);
    if (outw) *outw = ow;
    if (outh) *outh = oh;
    return NCNNHIP_OK;
}

int ncnnhip_conv_resolved_pads(const ncnnhip_conv_desc* desc, int* pad_top, int* pad_left)
{
    int ret = check_desc(desc, "ncnnhip_conv_resolved_pads");
    if (ret) return ret;
    const ResolvedPads p = resolve_pads(*desc);
    if (pad_top) *pad_top = p.top;
    if (pad_left) *pad_left = p.left;
    return NCNNHIP_OK;
}

int ncnnhip_fold_input_scales(const float* w_scales, int n_w_scales, const float* in_scales, int n_in_scales, int num_output,
                              float* scale_in_out)
{
    NCNNHIP_REQUIRE(w_scales && in_scales && scale_in_out, "ncnnhip_fold_input_scales: null pointer");
    NCNNHIP_REQUIRE(n_w_scales >= 1 && num_output % n_w_scales == 0, "ncnnhip_fold_input_scales: %d weight scales for %d outputs", n_w_scales, num_output);
    NCNNHIP_REQUIRE(n_in_scales == 1 || n_in_scales == n_w_scales, "ncnnhip_fold_input_scales: %d input scales", n_in_scales);
    const int per = num_output / n_w_scales;
    for (int p = 0; p < num_output; p++)
    {
        // volatile keeps the host compiler from fusing or reassociating the two roundings
        volatile float ws = w_scales[p / per];
        volatile float is = n_in_scales == 1 ? in_scales[0] : in_scales[p / per];
        volatile float prod = is * ws;
        scale_in_out[p] = ws == 0.f ? 0.f : 1.f / prod;
    }
    return NCNNHIP_OK;
}

int ncnnhip_conv_int8(const ncnnhip_conv_desc* desc, const int8_t* x_dev, size_t x_cstep, size_t x_nstep,
                      const int8_t* weight_dev, const float* scale_in_dev, const float* bias_dev,
                      const float* scale_out_dev, ncnnhip_activation act, void* out_dev, size_t out_cstep,
                      size_t out_nstep, int32_t* acc_out_dev, void* stream)
{
    int ret = check_desc(desc, "ncnnhip_conv_int8");
    if (ret) return ret;
    NCNNHIP_REQUIRE(x_dev && weight_dev && scale_in_dev && out_dev, "ncnnhip_conv_int8: null pointer");
    const ncnnhip_conv_desc& d = *desc;
    if (d.group < 1 || d.c % d.group != 0 || d.num_output % d.group != 0)
    {
        set_error("ncnnhip_conv_int8: channels %d / num_output %d not divisible by group %d", d.c, d.num_output, d.group);
        return NCNNHIP_OOM; // the reference rejects an invalid group with -100
    }
    int outw, outh;
    ret = ncnnhip_conv_out_shape(desc, &outw, &outh);
    if (ret) return ret;
    const ResolvedPads pads = resolve_pads(d);
    const long long plane = (long long)outw * outh;
    const long long npix = plane * d.batch;
    NCNNHIP_REQUIRE(npix < (1ll << 31), "ncnnhip_conv_int8: too many output pixels");
    NCNNHIP_REQUIRE(x_cstep >= (size_t)d.w * d.h && out_cstep >= (size_t)plane, "ncnnhip_conv_int8: channel stride below plane size");
    NCNNHIP_REQUIRE((long long)d.c * (long long)x_cstep < (1ll << 31), "ncnnhip_conv_int8: one input sample exceeds 2 GiB");
    NCNNHIP_REQUIRE(d.batch == 1 || (x_nstep >= x_cstep * d.c && out_nstep >= out_cstep * d.num_output), "ncnnhip_conv_int8: batch stride too small");
    const int pad_byte = (int)(signed char)d.pad_value;
    const int cin_g = d.c / d.group;
    const int cout_g = d.num_output / d.group;

    if (d.c == d.group && d.group == d.num_output)
    {
        DwParams p;
        p.x = x_dev;
        p.x_cstep = x_cstep;
        p.x_nstep = x_nstep;
        p.w = d.w;
        p.h = d.h;
        p.kw = d.kernel_w;
        p.kh = d.kernel_h;
        p.dw = d.dilation_w;
        p.dh = d.dilation_h;
        p.sw = d.stride_w;
        p.sh = d.stride_h;
        p.pad_top = pads.top;
        p.pad_left = pads.left;
        p.outw = outw;
        p.outh = outh;
        p.pad_byte = pad_byte;
        p.weight = weight_dev;
        p.scale_in = scale_in_dev;
        p.bias = bias_dev;
        p.scale_out = scale_out_dev;
        p.act = act;
        p.out = out_dev;
        p.out_cstep = out_cstep;
        p.out_nstep = out_nstep;
        p.acc_out = acc_out_dev;
        p.channels = d.c;
        NCNNHIP_REQUIRE(d.c <= 65535 && d.batch <= 65535, "ncnnhip_conv_int8: depthwise channels/batch above 65535");
        dim3 grid(ceil_div(plane, 256), d.c, d.batch);
        if (d.kernel_w == 3 && d.kernel_h == 3)
            hipLaunchKernelGGL((dwconv_kernel<3, 3>), grid, dim3(256), 0, as_stream(stream), p);
        else
            hipLaunchKernelGGL((dwconv_kernel<0, 0>), grid, dim3(256), 0, as_stream(stream), p);
        return launch_status("dwconv_kernel");
    }

    const int K = cin_g * d.kernel_w * d.kernel_h;
    DenseOperand wgt;
    wgt.base = weight_dev;
    wgt.stride = (size_t)K;
    wgt.rows = cout_g;
    wgt.K = K;
    wgt.vec = (reinterpret_cast<uintptr_t>(weight_dev) & 15) == 0 && K % 16 == 0;

    Im2colOperand src;
    src.x = x_dev;
    src.cstep = x_cstep;
    src.nstep = x_nstep;
    src.w = d.w;
    src.h = d.h;
    src.cin_g = cin_g;
    src.kw = d.kernel_w;
    src.kh = d.kernel_h;
    src.dw = d.dilation_w;
    src.dh = d.dilation_h;
    src.sw = d.stride_w;
    src.sh = d.stride_h;
    src.pad_top = pads.top;
    src.pad_left = pads.left;
    src.outw = outw;
    src.outh = outh;
    src.npix = (int)npix;
    src.K = K;
    src.group_channel0 = 0;
    src.pad_byte = pad_byte;
    src.pix_base = 0;
    src.iy0 = src.ix0 = src.pix_ok = 0;

    ConvEpilogue epi;
    epi.scale_in = scale_in_dev;
    epi.bias = bias_dev;
    epi.scale_out = scale_out_dev;
    epi.act = act;
    epi.out = out_dev;
    epi.out_cstep = out_cstep;
    epi.out_nstep = out_nstep;
    epi.pix_per_img = (int)plane;
    epi.batch = d.batch;
    epi.out_channel0 = 0;
    epi.num_output = d.num_output;
    epi.acc_out = acc_out_dev;

    NCNNHIP_REQUIRE(d.group <= 65535, "ncnnhip_conv_int8: group above 65535");
    const size_t wgs = (size_t)cout_g * K;
    if (cout_g <= 64)
    {
        dim3 grid(ceil_div(npix, 128), ceil_div(cout_g, 64), d.group);
        hipLaunchKernelGGL((conv_tile_kernel<64, 128>), grid, dim3(256), 0, as_stream(stream), wgt, src, epi, cout_g, (int)npix, K, wgs);
    }
    else
    {
        dim3 grid(ceil_div(npix, 128), ceil_div(cout_g, 128), d.group);
        NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_conv_int8: num_output too large");
        hipLaunchKernelGGL((conv_tile_kernel<128, 128>), grid, dim3(256), 0, as_stream(stream), wgt, src, epi, cout_g, (int)npix, K, wgs);
    }
    return launch_status("conv_tile_kernel");
}

} // extern "C"
