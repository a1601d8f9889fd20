// int8 Convolution (group 1) as an implicit GEMM over a channels-last int8 copy of the activations.
//
// ncnn hands over [c][h][w] planes; a K-contiguous MFMA operand needs, for one output pixel, runs of
// consecutive input channels.  So the quantise pre-pass writes the blob as [n][h][w][Cp] int8 with the
// channel count padded to Cp = 16*ceil(c/16) (pad channels are zero), and the weights are repacked once at
// create_pipeline to [num_output][kh*kw][Cp] (K order tap-major, zero in the pad channels, K padded to a
// multiple of 64).  One 16-byte chunk of the im2col row is then one aligned 16-byte global load: channels
// q0..q0+15 of tap (ky,kx) at that pixel, or 16 border bytes when the tap falls outside the image.
//
// Kernel: BM output channels x BN output pixels per workgroup (4 wavefronts 2x2, v_mfma_i32_32x32x32_i8),
// K walked in 64-byte steps; the global loads of step t+1 are issued into registers before the MFMAs of step t
// and written to the other LDS buffer afterwards (one barrier per step).  Layers with few output pixels
// (ResNet tail at batch 1) split K over blockIdx.z: partial int32 sums are added atomically into a zeroed
// workspace -- integer addition, so the result is still exact -- and a second small kernel applies the epilogue.
#include "conv_nhwc.h"
#include "mfma_tile.h"

namespace ncnnhip {

__device__ __forceinline__ uint32_t pack4b(int a, int b, int c, int d)
{
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}

// [n][c][h][w] fp32 or int8  ->  [n][h][w][Cp] int8.  One thread: one pixel, 16 consecutive channels.
template<typename T>
__global__ __launch_bounds__(256) void to_nhwc_int8_kernel(const T* __restrict__ x, size_t cstep, size_t nstep, int c, int hw, int Cp,
                                                            const float* __restrict__ scales, int nscales, int8_t* __restrict__ out)
{
    const int pix = blockIdx.x * 256 + threadIdx.x;
    const int q0 = blockIdx.y * 16;
    const int img = blockIdx.z;
    if (pix >= hw) return;
    const T* xp = x + (size_t)img * nstep + pix;
    int v[16];
#pragma unroll
    for (int e = 0; e < 16; e++)
    {
        const int q = q0 + e;
        int val = 0;
        if (q < c)
        {
            if (sizeof(T) == 4)
            {
                const float s = nscales == 1 ? scales[0] : scales[q];
                val = float2int8(mul_rn((float)xp[(size_t)q * cstep], s));
            }
            else
                val = (int)xp[(size_t)q * cstep];
        }
        v[e] = val;
    }
    v4i pk;
    pk[0] = (int)pack4b(v[0], v[1], v[2], v[3]);
    pk[1] = (int)pack4b(v[4], v[5], v[6], v[7]);
    pk[2] = (int)pack4b(v[8], v[9], v[10], v[11]);
    pk[3] = (int)pack4b(v[12], v[13], v[14], v[15]);
    *reinterpret_cast<v4i*>(out + ((size_t)img * hw + pix) * Cp + q0) = pk;
}

__global__ __launch_bounds__(256) void zero_i32_kernel(int32_t* p, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

typedef float v4f __attribute__((ext_vector_type(4)));

// channels-last store of output channels p0..p0+3 (p0 % 4 == 0) of output pixel n: one 4-byte (int8) or 16-byte
// (fp32) word; channels at or beyond num_output are the blob's zero padding
__device__ __forceinline__ void store4_channels_last(const ConvEpilogue& e, int out_cp, int p0, int n, const int* acc)
{
    float f[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
    {
        const int p = p0 + k;
        float r = 0.f;
        if (p < e.num_output)
        {
            r = mul_rn((float)acc[k], e.scale_in[p]);
            if (e.bias) r = add_rn(r, e.bias[p]);
            r = apply_activation(r, e.act);
            if (e.scale_out) r = (float)float2int8(mul_rn(r, e.scale_out[p]));
        }
        f[k] = r;
    }
    const size_t o = (size_t)n * out_cp + p0;
    if (e.scale_out)
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(e.out) + o) = pack4b((int)f[0], (int)f[1], (int)f[2], (int)f[3]);
    else
        *reinterpret_cast<v4f*>(static_cast<float*>(e.out) + o) = v4f{f[0], f[1], f[2], f[3]};
}

template<int BM, int BN, bool SPLITK, bool CLAST>
__global__ __launch_bounds__(256) void conv_nhwc_kernel(const int8_t* __restrict__ wpk, const int8_t* __restrict__ x, NhwcGeom g, ConvEpilogue epi,
                                                         int steps_per_split, int32_t* __restrict__ partial, int out_cp)
{
    constexpr int TM = BM / 64, TN = BN / 64;
    constexpr int ACH = BM * 4 / 256 > 0 ? BM * 4 / 256 : 1; // 16-byte chunks of the weight tile per thread
    constexpr int BCH = BN * 4 / 256 > 0 ? BN * 4 / 256 : 1;
    __shared__ __attribute__((aligned(16))) int8_t lds[2][(BM + BN) * LDS_PITCH];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;

    const int total_steps = g.K / 64;
    const int step_begin = SPLITK ? blockIdx.z * steps_per_split : 0;
    int step_end = SPLITK ? step_begin + steps_per_split : total_steps;
    if (step_end > total_steps) step_end = total_steps;
    if (step_begin >= step_end) return;

    // ---- per-thread chunk assignment: chunk id = tid + 256*i -> tile row id>>2, K chunk j = tid&3 (same j for all i)
    const int j = threadIdx.x & 3;
    const bool a_thread = BM * 4 >= 256 || threadIdx.x < BM * 4;
    const bool b_thread = BN * 4 >= 256 || threadIdx.x < BN * 4;

    // weight rows
    const int8_t* a_ptr[ACH];
    bool a_ok[ACH];
#pragma unroll
    for (int i = 0; i < ACH; i++)
    {
        const int r = row0 + ((threadIdx.x + 256 * i) >> 2);
        a_ok[i] = a_thread && r < g.cout;
        a_ptr[i] = wpk + (size_t)(a_ok[i] ? r : 0) * g.K + j * 16;
    }
    // output pixels
    const int8_t* b_base[BCH];
    int b_iy0[BCH], b_ix0[BCH];
    bool b_ok[BCH];
#pragma unroll
    for (int i = 0; i < BCH; i++)
    {
        const int n = col0 + ((threadIdx.x + 256 * i) >> 2);
        b_ok[i] = b_thread && n < g.npix;
        const int nn = b_ok[i] ? n : 0;
        const int plane = g.outw * g.outh;
        const int img = nn / plane;
        const int rem = nn - img * plane;
        const int oy = rem / g.outw;
        const int ox = rem - oy * g.outw;
        b_iy0[i] = oy * g.sh - g.pad_top;
        b_ix0[i] = ox * g.sw - g.pad_left;
        b_base[i] = x + (size_t)img * g.H * g.W * g.Cp;
    }
    // this thread's position in K: tap (ky,kx) and first channel q0 of its 16-byte chunk, advanced by 64 per step
    int q0, ky, kx, tap;
    {
        const int k = step_begin * 64 + j * 16;
        tap = k / g.Cp;
        q0 = k - tap * g.Cp;
        ky = tap / g.kw;
        kx = tap - ky * g.kw;
    }

    v4i ra[ACH], rb[BCH];
    auto fetch = [&](int step) {
#pragma unroll
        for (int i = 0; i < ACH; i++) ra[i] = a_ok[i] ? *reinterpret_cast<const v4i*>(a_ptr[i] + (size_t)step * 64) : v4i{0, 0, 0, 0};
        const int dy = ky * g.dh, dx = kx * g.dw;
        const bool tap_ok = tap < g.ntaps;
#pragma unroll
        for (int i = 0; i < BCH; i++)
        {
            v4i v = {0, 0, 0, 0};
            if (b_ok[i] && tap_ok)
            {
                const int iy = b_iy0[i] + dy, ix = b_ix0[i] + dx;
                if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
                    v = *reinterpret_cast<const v4i*>(b_base[i] + ((size_t)iy * g.W + ix) * g.Cp + q0);
                else
                    v = v4i{g.pad_word, g.pad_word, g.pad_word, g.pad_word};
            }
            rb[i] = v;
        }
        // advance to the next step
        q0 += 64;
        while (q0 >= g.Cp)
        {
            q0 -= g.Cp;
            tap++;
            if (++kx == g.kw)
            {
                kx = 0;
                ky++;
            }
        }
    };
    auto stash = [&](int buf) {
        int8_t* As = lds[buf];
        int8_t* Bs = lds[buf] + BM * LDS_PITCH;
#pragma unroll
        for (int i = 0; i < ACH; i++)
            if (a_thread) *reinterpret_cast<v4i*>(As + ((threadIdx.x + 256 * i) >> 2) * LDS_PITCH + j * 16) = ra[i];
#pragma unroll
        for (int i = 0; i < BCH; i++)
            if (b_thread) *reinterpret_cast<v4i*>(Bs + ((threadIdx.x + 256 * i) >> 2) * LDS_PITCH + j * 16) = rb[i];
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

    fetch(step_begin);
    stash(0);
    __syncthreads();
    for (int t = step_begin; t < step_end; t++)
    {
        const int buf = (t - step_begin) & 1;
        if (t + 1 < step_end) fetch(t + 1);
        const int8_t* As = lds[buf];
        const int8_t* Bs = lds[buf] + BM * LDS_PITCH;
#pragma unroll
        for (int ks = 0; ks < 64; ks += 32)
        {
            v4i fa[TM], fb[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) fa[a] = *reinterpret_cast<const v4i*>(As + (wm * (BM / 2) + a * 32 + l32) * LDS_PITCH + ks + lhi * 16);
#pragma unroll
            for (int b = 0; b < TN; b++) fb[b] = *reinterpret_cast<const v4i*>(Bs + (wn * (BN / 2) + b * 32 + l32) * LDS_PITCH + ks + lhi * 16);
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++) acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[a], fb[b], acc[a][b], 0, 0, 0);
        }
        if (t + 1 < step_end) stash(buf ^ 1);
        __syncthreads();
    }

    if (CLAST)
    {
        // accumulator registers 4*rg..4*rg+3 of a lane are four consecutive output channels of one pixel
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
            for (int b = 0; b < TN; b++)
#pragma unroll
                for (int rg = 0; rg < 4; rg++)
                {
                    const int p0 = row0 + wm * (BM / 2) + a * 32 + 8 * rg + 4 * lhi;
                    const int gj = col0 + wn * (BN / 2) + b * 32 + l32;
                    if (p0 < out_cp && gj < g.npix)
                    {
                        const int v[4] = {acc[a][b][rg * 4], acc[a][b][rg * 4 + 1], acc[a][b][rg * 4 + 2], acc[a][b][rg * 4 + 3]};
                        if (SPLITK)
                        {
#pragma unroll
                            for (int k = 0; k < 4; k++)
                                if (p0 + k < g.cout) atomicAdd(partial + (size_t)gj * out_cp + p0 + k, v[k]);
                        }
                        else
                            store4_channels_last(epi, out_cp, p0, gj, v);
                    }
                }
        return;
    }
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int gi = row0 + wm * (BM / 2) + a * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                const int gj = col0 + wn * (BN / 2) + b * 32 + l32;
                if (gi < g.cout && gj < g.npix)
                {
                    if (SPLITK)
                        atomicAdd(partial + (size_t)gi * g.npix + gj, acc[a][b][r]);
                    else
                        epi(gi, gj, acc[a][b][r]);
                }
            }
}

// partial sums laid out [npix][out_cp]: one thread finishes four channels of one pixel
__global__ __launch_bounds__(256) void conv_splitk_finish_clast_kernel(const int32_t* __restrict__ partial, int npix, int out_cp, ConvEpilogue epi)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int groups = out_cp / 4;
    if (i >= (size_t)npix * groups) return;
    const int n = (int)(i / groups);
    const int p0 = (int)(i - (size_t)n * groups) * 4;
    const v4i v = *reinterpret_cast<const v4i*>(partial + (size_t)n * out_cp + p0);
    const int a[4] = {v[0], v[1], v[2], v[3]};
    store4_channels_last(epi, out_cp, p0, n, a);
}

__global__ __launch_bounds__(256) void conv_splitk_finish_kernel(const int32_t* __restrict__ partial, int cout, int npix, ConvEpilogue epi)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)cout * npix) return;
    const int p = (int)(i / npix);
    const int n = (int)(i - (size_t)p * npix);
    epi(p, n, partial[i]);
}

struct Pads4
{
    int top, bottom, left, right;
};

static Pads4 resolve_pads_nhwc(const ncnnhip_conv_desc& d)
{
    Pads4 p = {0, 0, 0, 0};
    const int kext_w = d.dilation_w * (d.kernel_w - 1) + 1, kext_h = d.dilation_h * (d.kernel_h - 1) + 1;
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
            p.top = upper ? hpad / 2 : hpad - hpad / 2;
            p.left = upper ? wpad / 2 : wpad - wpad / 2;
        }
    }
    return p;
}

static inline int padded_channels(int c)
{
    return (c + 15) / 16 * 16;
}
static inline int packed_k(const ncnnhip_conv_desc& d)
{
    return (d.kernel_w * d.kernel_h * padded_channels(d.c) + 63) / 64 * 64;
}

struct SplitPlan
{
    int bm, bn, splits, steps_per_split;
};

// enough workgroups to occupy the chip: shrink the tile first, then split K
static SplitPlan plan_launch(int cout, long long npix, int steps)
{
    SplitPlan p;
    p.bm = cout <= 64 ? 64 : 128;
    p.bn = 128;
    long long tiles = (long long)ceil_div(cout, p.bm) * ceil_div(npix, p.bn);
    if (tiles < 256 && npix <= 64 * 1024)
    {
        p.bn = 64;
        tiles = (long long)ceil_div(cout, p.bm) * ceil_div(npix, p.bn);
    }
    if (tiles < 128 && p.bm == 128)
    {
        p.bm = 64;
        tiles = (long long)ceil_div(cout, p.bm) * ceil_div(npix, p.bn);
    }
    p.splits = 1;
    if (tiles < 192 && steps >= 8)
    {
        int want = (int)((384 + tiles - 1) / tiles);
        int max_splits = steps / 4; // at least 4 K steps per split
        p.splits = want < max_splits ? want : max_splits;
        if (p.splits < 1) p.splits = 1;
    }
    p.steps_per_split = ceil_div(steps, p.splits);
    p.splits = ceil_div(steps, p.steps_per_split);
    return p;
}

} // namespace ncnnhip

using namespace ncnnhip;

// ---- narrow-input ("stem") convolution: up to 4 input channels ------------------------------------------------------
// A 3-channel image padded to 16 channels wastes 13/16 of every K step.  Instead the quantised input is kept as an image
// of 4 bytes per pixel with a zero border, [n][Hb][Wp][4], and one 16-byte K chunk is 4 NEIGHBOURING pixels x 4 channels:
// a kernel row of kw taps becomes G = ceil(kw/4) chunks (weights beyond kw are zero).  In the pipelined kernel's terms this
// is a convolution over pixels 4 bytes apart (Cp = 4) whose "taps" are G groups 4 pixels apart (dilation 4) contributing
// 16 bytes each (tapK = 16); the border is physical, so no gather ever leaves the image.  7x7x3: K 832 -> 256.
namespace ncnnhip {

struct StemShape
{
    int G, Hb, Wp, K, outw, outh;
    Pads4 pads;
};

static bool stem_supported(const ncnnhip_conv_desc& d)
{
    return d.group == 1 && d.c >= 1 && d.c <= 4 && d.dilation_w == 1 && ((int)(signed char)d.pad_value & 0xff) == 0;
}

static int stem_shape(const ncnnhip_conv_desc& d, StemShape& s)
{
    int ret = ncnnhip_conv_out_shape(&d, &s.outw, &s.outh);
    if (ret) return ret;
    s.pads = resolve_pads_nhwc(d);
    s.G = (d.kernel_w + 3) / 4;
    const int need_h = (s.outh - 1) * d.stride_h + (d.kernel_h - 1) * d.dilation_h + 1;
    const int need_w = (s.outw - 1) * d.stride_w + (s.G - 1) * 4 + 4;
    s.Hb = std::max(s.pads.top + d.h, need_h);
    s.Wp = (std::max(s.pads.left + d.w, need_w) + 3) & ~3; // whole groups of four pixels: the quantiser stores 16 bytes per thread
    s.K = (d.kernel_h * s.G * 16 + 63) / 64 * 64;
    return NCNNHIP_OK;
}

// one thread per pixel of the bordered image: 4 bytes out.  blockIdx.y = row of the bordered image, blockIdx.z = sample.
template<typename T>
__global__ __launch_bounds__(256) void quantize_stem_kernel(const T* __restrict__ src, int src_cp, int c, int h, int w, int top, int left, int Hb, int Wp,
                                                            const float* __restrict__ scale, uint32_t* __restrict__ image)
{
    const int xb = blockIdx.x * 256 + threadIdx.x;
    if (xb >= Wp) return;
    const int yb = blockIdx.y;
    const size_t img = blockIdx.z;
    const int y = yb - top, x = xb - left;
    uint32_t word = 0;
    if ((unsigned)y < (unsigned)h && (unsigned)x < (unsigned)w)
    {
        const T* p = src + ((img * h + y) * (size_t)w + x) * src_cp;
        if (sizeof(T) == 4)
        {
            const float sc = scale[0];
            float v[4] = {0.f, 0.f, 0.f, 0.f};
            if (src_cp == 4)
            {
                // the narrow image: one aligned 16-byte load per pixel (its unused channels are zero)
                const v4f t = *reinterpret_cast<const v4f*>(p);
                v[0] = t[0], v[1] = t[1], v[2] = t[2], v[3] = t[3];
            }
            else
            {
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (q < c) v[q] = (float)p[q];
            }
#pragma unroll
            for (int q = 0; q < 4; q++) v[q] = q < c ? mul_rn(v[q], sc) : 0.f;
            float2int8_as_float_x4(v[0], v[1], v[2], v[3]);
            word = pack4_quantised(v[0], v[1], v[2], v[3]);
        }
        else
        {
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (q < c) word |= (uint32_t)((int)p[q] & 255) << (8 * q);
        }
    }
    image[(img * Hb + yb) * (size_t)Wp + xb] = word;
}

// The same from the narrow fp32 image (4 floats per pixel): four neighbouring pixels of the bordered image per thread,
// up to four aligned 16-byte loads and one 16-byte store (Wp is a multiple of 4, the image 16-byte aligned).
__global__ __launch_bounds__(256) void quantize_stem_narrow_kernel(const float* __restrict__ src, int c, int h, int w, int top, int left, int Hb, int Wp,
                                                                   const float* __restrict__ scale, int8_t* __restrict__ image)
{
    const int xb0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (xb0 >= Wp) return;
    const int yb = blockIdx.y;
    const size_t img = blockIdx.z;
    const int y = yb - top;
    const bool row_in = (unsigned)y < (unsigned)h;
    const float* row = src + ((img * h + (row_in ? y : 0)) * (size_t)w) * 4;
    v4f t[4];
    bool in[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
    {
        const int x = xb0 + i - left;
        in[i] = row_in && (unsigned)x < (unsigned)w;
        t[i] = *reinterpret_cast<const v4f*>(row + (size_t)(in[i] ? x : 0) * 4); // unconditional: the four loads overlap
    }
    const float sc = scale[0];
    v4i word;
#pragma unroll
    for (int i = 0; i < 4; i++)
    {
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; q++) v[q] = q < c ? mul_rn(t[i][q], sc) : 0.f;
        float2int8_as_float_x4(v[0], v[1], v[2], v[3]);
        const uint32_t pk = pack4_quantised(v[0], v[1], v[2], v[3]);
        word[i] = in[i] ? (int)pk : 0;
    }
    *reinterpret_cast<v4i*>(image + ((img * Hb + yb) * (size_t)Wp + xb0) * 4) = word;
}

} // namespace ncnnhip

extern "C" {

int ncnnhip_conv_nhwc_sizes(const ncnnhip_conv_desc* desc, size_t* nhwc_bytes, size_t* packed_weight_bytes, size_t* workspace_bytes)
{
    NCNNHIP_REQUIRE(desc && desc->group == 1, "ncnnhip_conv_nhwc_sizes: channels-last path handles group 1 only");
    int outw, outh;
    int ret = ncnnhip_conv_out_shape(desc, &outw, &outh);
    if (ret) return ret;
    const int Cp = padded_channels(desc->c);
    if (nhwc_bytes) *nhwc_bytes = (size_t)desc->batch * desc->h * desc->w * Cp;
    if (packed_weight_bytes) *packed_weight_bytes = (size_t)desc->num_output * packed_k(*desc);
    if (workspace_bytes)
    {
        const long long npix = (long long)desc->batch * outw * outh;
        const SplitPlan p = plan_launch(desc->num_output, npix, packed_k(*desc) / 64);
        size_t words = p.splits > 1 ? SPLIT_COUNTER_BYTES / sizeof(int32_t) + (size_t)padded_channels(desc->num_output) * npix : 0;
        const size_t words_pipelined = conv_nhwc_pipelined_workspace_words(desc->num_output, npix, packed_k(*desc) / 64);
        if (words_pipelined > words) words = words_pipelined;
        *workspace_bytes = words * sizeof(int32_t);
    }
    return NCNNHIP_OK;
}

int ncnnhip_conv_pack_weights(const ncnnhip_conv_desc* desc, const int8_t* weight_host, int8_t* packed_host)
{
    NCNNHIP_REQUIRE(desc && weight_host && packed_host && desc->group == 1, "ncnnhip_conv_pack_weights: bad argument");
    const int c = desc->c, Cp = padded_channels(c), taps = desc->kernel_w * desc->kernel_h, K = packed_k(*desc);
    for (int p = 0; p < desc->num_output; p++)
    {
        int8_t* row = packed_host + (size_t)p * K;
        for (int k = 0; k < K; k++) row[k] = 0;
        for (int q = 0; q < c; q++)
            for (int t = 0; t < taps; t++) row[t * Cp + q] = weight_host[((size_t)p * c + q) * taps + t];
    }
    return NCNNHIP_OK;
}

int ncnnhip_to_nhwc_int8(const ncnnhip_conv_desc* desc, const void* x_dev, int x_elemsize, size_t x_cstep, size_t x_nstep,
                         const float* scales_dev, int nscales, int8_t* nhwc_dev, void* stream)
{
    NCNNHIP_REQUIRE(desc && x_dev && nhwc_dev, "ncnnhip_to_nhwc_int8: null pointer");
    NCNNHIP_REQUIRE(x_elemsize == 1 || (x_elemsize == 4 && scales_dev && (nscales == 1 || nscales == desc->c)), "ncnnhip_to_nhwc_int8: bad element size / scales");
    NCNNHIP_REQUIRE(desc->batch <= 65535, "ncnnhip_to_nhwc_int8: batch above 65535");
    const int hw = desc->w * desc->h, Cp = padded_channels(desc->c);
    NCNNHIP_REQUIRE(x_cstep >= (size_t)hw, "ncnnhip_to_nhwc_int8: channel stride below plane size");
    dim3 grid(ceil_div(hw, 256), Cp / 16, desc->batch);
    if (x_elemsize == 4)
        hipLaunchKernelGGL(to_nhwc_int8_kernel<float>, grid, dim3(256), 0, as_stream(stream), (const float*)x_dev, x_cstep, x_nstep, desc->c, hw, Cp, scales_dev, nscales, nhwc_dev);
    else
        hipLaunchKernelGGL(to_nhwc_int8_kernel<int8_t>, grid, dim3(256), 0, as_stream(stream), (const int8_t*)x_dev, x_cstep, x_nstep, desc->c, hw, Cp, (const float*)0, 1, nhwc_dev);
    return launch_status("to_nhwc_int8_kernel");
}

static NhwcGeom nhwc_geometry(const ncnnhip_conv_desc& d, int outw, int outh, long long npix)
{
    const Pads4 pads = resolve_pads_nhwc(d);
    NhwcGeom g;
    g.H = d.h;
    g.W = d.w;
    g.Cp = padded_channels(d.c);
    g.tapK = g.Cp;
    g.kw = d.kernel_w;
    g.kh = d.kernel_h;
    g.dw = d.dilation_w;
    g.dh = d.dilation_h;
    g.sw = d.stride_w;
    g.sh = d.stride_h;
    g.pad_top = pads.top;
    g.pad_left = pads.left;
    g.outw = outw;
    g.outh = outh;
    g.npix = (int)npix;
    g.ntaps = d.kernel_w * d.kernel_h;
    g.K = packed_k(d);
    g.cout = d.num_output;
    const int pb = (int)(signed char)d.pad_value & 0xff;
    g.pad_word = (int)((uint32_t)pb * 0x01010101u);
    return g;
}

// x_elemsize 1: nhwc_dev is the quantised blob.  4 / 2: it is the fp32 / fp16 blob, quantised with x_scale_dev[0] inside the
// one launch (channels-last output and a layer ncnnhip_conv_from_float_supported accepts).
static int conv_int8_nhwc_impl(const ncnnhip_conv_desc* desc, const void* nhwc_dev, int x_elemsize, const float* x_scale_dev, const int8_t* packed_weight_dev,
                               const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act, void* out_dev, int out_layout,
                               size_t out_cstep, size_t out_nstep, const ConvFusion& fusion, void* workspace_dev, size_t workspace_bytes, void* stream)
{
    NCNNHIP_REQUIRE(desc && nhwc_dev && packed_weight_dev && scale_in_dev && out_dev, "ncnnhip_conv_int8_nhwc: null pointer");
    NCNNHIP_REQUIRE(desc->group == 1, "ncnnhip_conv_int8_nhwc: group must be 1");
    int outw, outh;
    int ret = ncnnhip_conv_out_shape(desc, &outw, &outh);
    if (ret) return ret;
    const ncnnhip_conv_desc& d = *desc;
    const long long plane = (long long)outw * outh, npix = plane * d.batch;
    NCNNHIP_REQUIRE(out_layout == NCNNHIP_PLANAR || out_layout == NCNNHIP_CHANNELS_LAST, "ncnnhip_conv_int8_nhwc: unknown output layout %d", out_layout);
    const bool clast = out_layout == NCNNHIP_CHANNELS_LAST;
    const int out_cp = padded_channels(desc->num_output);
    NCNNHIP_REQUIRE(npix < (1ll << 31) && (clast || out_cstep >= (size_t)plane), "ncnnhip_conv_int8_nhwc: bad output extent");
    NCNNHIP_REQUIRE((long long)d.h * d.w * padded_channels(d.c) < (1ll << 31), "ncnnhip_conv_int8_nhwc: one input sample exceeds 2 GiB");
    const NhwcGeom g = nhwc_geometry(d, outw, outh, npix);
    const int pb = g.pad_word & 0xff;

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
    epi.acc_out = 0;

    hipStream_t st = as_stream(stream);
    if (clast && pb == 0 && conv_patch_pays(g, d.batch, x_elemsize))
        return launch_conv_patch(g, packed_weight_dev, nhwc_dev, x_elemsize, x_scale_dev, epi, fusion, out_cp, st);
    if (x_elemsize != 1)
    {
        NCNNHIP_REQUIRE(clast && x_scale_dev, "ncnnhip_conv_int8_nhwc_from_float: needs channels-last output and the input scale");
        return launch_conv_nhwc_staged(g, packed_weight_dev, nhwc_dev, x_elemsize, x_scale_dev, epi, fusion, out_cp, workspace_dev, workspace_bytes, st);
    }
    const int8_t* xq = static_cast<const int8_t*>(nhwc_dev);
    // zero border and channels-last output: the pipelined kernel
    if (clast && pb == 0) return launch_conv_nhwc_pipelined(g, packed_weight_dev, xq, epi, fusion, out_cp, workspace_dev, workspace_bytes, st);
    NCNNHIP_REQUIRE(!fusion.residual && !fusion.relu_after && !fusion.q8_out, "ncnnhip_conv_int8_nhwc_fused: needs channels-last output and a zero border value");
    const SplitPlan p = plan_launch(d.num_output, npix, g.K / 64);
    dim3 grid(ceil_div(npix, p.bn), ceil_div(d.num_output, p.bm), p.splits);
    NCNNHIP_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "ncnnhip_conv_int8_nhwc: grid too large");
    int32_t* partial = 0;
    if (p.splits > 1)
    {
        const size_t words = (size_t)out_cp * npix;
        NCNNHIP_REQUIRE(workspace_dev && workspace_bytes >= SPLIT_COUNTER_BYTES + words * sizeof(int32_t), "ncnnhip_conv_int8_nhwc: workspace of %zu bytes required",
                        SPLIT_COUNTER_BYTES + words * sizeof(int32_t));
        partial = (int32_t*)((char*)workspace_dev + SPLIT_COUNTER_BYTES); // the counter region belongs to the pipelined kernel: left untouched (zero)
        hipLaunchKernelGGL(zero_i32_kernel, dim3(ceil_div((long long)words, 256)), dim3(256), 0, st, partial, words);
    }
#define LAUNCH_NHWC(BM_, BN_)                                                                                                                       \
    do                                                                                                                                               \
    {                                                                                                                                                \
        if (p.splits > 1 && clast)                                                                                                                   \
            hipLaunchKernelGGL((conv_nhwc_kernel<BM_, BN_, true, true>), grid, dim3(256), 0, st, packed_weight_dev, xq, g, epi, p.steps_per_split, partial, out_cp); \
        else if (p.splits > 1)                                                                                                                       \
            hipLaunchKernelGGL((conv_nhwc_kernel<BM_, BN_, true, false>), grid, dim3(256), 0, st, packed_weight_dev, xq, g, epi, p.steps_per_split, partial, out_cp); \
        else if (clast)                                                                                                                              \
            hipLaunchKernelGGL((conv_nhwc_kernel<BM_, BN_, false, true>), grid, dim3(256), 0, st, packed_weight_dev, xq, g, epi, p.steps_per_split, partial, out_cp); \
        else                                                                                                                                         \
            hipLaunchKernelGGL((conv_nhwc_kernel<BM_, BN_, false, false>), grid, dim3(256), 0, st, packed_weight_dev, xq, g, epi, p.steps_per_split, partial, out_cp); \
    } while (0)
    if (p.bm == 128 && p.bn == 128)
        LAUNCH_NHWC(128, 128);
    else if (p.bm == 128)
        LAUNCH_NHWC(128, 64);
    else if (p.bn == 128)
        LAUNCH_NHWC(64, 128);
    else
        LAUNCH_NHWC(64, 64);
#undef LAUNCH_NHWC
    if (p.splits > 1 && clast)
        hipLaunchKernelGGL(conv_splitk_finish_clast_kernel, dim3(ceil_div((long long)(out_cp / 4) * npix, 256)), dim3(256), 0, st, partial, (int)npix, out_cp, epi);
    else if (p.splits > 1)
        hipLaunchKernelGGL(conv_splitk_finish_kernel, dim3(ceil_div((long long)d.num_output * npix, 256)), dim3(256), 0, st, partial, d.num_output, (int)npix, epi);
    return launch_status("conv_nhwc_kernel");
}

int ncnnhip_conv_int8_nhwc(const ncnnhip_conv_desc* desc, const int8_t* nhwc_dev, const int8_t* packed_weight_dev, const float* scale_in_dev,
                           const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act, void* out_dev, int out_layout,
                           size_t out_cstep, size_t out_nstep, void* workspace_dev, size_t workspace_bytes, void* stream)
{
    const ConvFusion none = {0, 0, 0, 0.f};
    return conv_int8_nhwc_impl(desc, nhwc_dev, 1, 0, packed_weight_dev, scale_in_dev, bias_dev, scale_out_dev, act, out_dev, out_layout, out_cstep, out_nstep, none,
                               workspace_dev, workspace_bytes, stream);
}

int ncnnhip_conv_fusion_supported(const ncnnhip_conv_desc* desc)
{
    return desc && desc->group == 1 && (int)(signed char)desc->pad_value == 0;
}

int ncnnhip_conv_int8_nhwc_fused(const ncnnhip_conv_desc* desc, const int8_t* nhwc_dev, const int8_t* packed_weight_dev, const float* scale_in_dev,
                                 const float* bias_dev, ncnnhip_activation act, float* out_dev, const ncnnhip_conv_fusion* fusion, void* workspace_dev,
                                 size_t workspace_bytes, void* stream)
{
    NCNNHIP_REQUIRE(fusion, "ncnnhip_conv_int8_nhwc_fused: null fusion");
    NCNNHIP_REQUIRE(ncnnhip_conv_fusion_supported(desc), "ncnnhip_conv_int8_nhwc_fused: needs group 1 and a zero border value");
    NCNNHIP_REQUIRE(!fusion->quantised_out_dev || fusion->quantise_scale != 0.f, "ncnnhip_conv_int8_nhwc_fused: quantised copy without a scale");
    ConvFusion f;
    f.residual = fusion->residual_dev;
    f.relu_after = fusion->relu_after;
    f.q8_out = fusion->quantised_out_dev;
    f.q8_scale = fusion->quantise_scale;
    return conv_int8_nhwc_impl(desc, nhwc_dev, 1, 0, packed_weight_dev, scale_in_dev, bias_dev, 0, act, out_dev, NCNNHIP_CHANNELS_LAST, 0, 0, f, workspace_dev,
                               workspace_bytes, stream);
}

int ncnnhip_conv_from_float_supported(const ncnnhip_conv_desc* desc)
{
    if (!desc || desc->group != 1 || (int)(signed char)desc->pad_value != 0) return 0;
    int outw = 0, outh = 0;
    if (ncnnhip_conv_out_shape(desc, &outw, &outh) != 0) return 0;
    const long long npix = (long long)outw * outh * desc->batch;
    if (npix >= (1ll << 31) || (long long)desc->h * desc->w * padded_channels(desc->c) >= (1ll << 31)) return 0;
    const NhwcGeom g = nhwc_geometry(*desc, outw, outh, npix);
    return (conv_patch_pays(g, desc->batch, 4) || conv_nhwc_staged_supported(g)) ? 1 : 0;
}

int ncnnhip_conv_small_tile_selected(const ncnnhip_conv_desc* desc, int elemsize)
{
    if (!desc || desc->group != 1 || (int)(signed char)desc->pad_value != 0 || (elemsize != 1 && elemsize != 2 && elemsize != 4)) return 0;
    int outw = 0, outh = 0;
    if (ncnnhip_conv_out_shape(desc, &outw, &outh) != 0) return 0;
    const long long npix = (long long)outw * outh * desc->batch;
    if (npix >= (1ll << 31) || (long long)desc->h * desc->w * padded_channels(desc->c) >= (1ll << 31)) return 0;
    return conv_patch_pays(nhwc_geometry(*desc, outw, outh, npix), desc->batch, elemsize) ? 1 : 0;
}

int ncnnhip_conv_from_float_workspace_bytes(const ncnnhip_conv_desc* desc, size_t* workspace_bytes)
{
    NCNNHIP_REQUIRE(workspace_bytes, "ncnnhip_conv_from_float_workspace_bytes: null pointer");
    *workspace_bytes = 0;
    NCNNHIP_REQUIRE(ncnnhip_conv_from_float_supported(desc), "ncnnhip_conv_from_float_workspace_bytes: this layer needs its separate Quantize pass");
    int outw = 0, outh = 0;
    int ret = ncnnhip_conv_out_shape(desc, &outw, &outh);
    if (ret) return ret;
    const NhwcGeom g = nhwc_geometry(*desc, outw, outh, (long long)outw * outh * desc->batch);
    if (!conv_patch_pays(g, desc->batch, 4)) *workspace_bytes = conv_nhwc_staged_workspace_bytes(g); // (the small-tile kernel needs none)
    return NCNNHIP_OK;
}

int ncnnhip_conv_int8_nhwc_from_float(const ncnnhip_conv_desc* desc, const void* nhwc_dev, int elemsize, const float* in_scale_dev,
                                      const int8_t* packed_weight_dev, const float* scale_in_dev, const float* bias_dev, const float* scale_out_dev,
                                      ncnnhip_activation act, void* out_dev, const ncnnhip_conv_fusion* fusion, void* workspace_dev, size_t workspace_bytes,
                                      void* stream)
{
    NCNNHIP_REQUIRE(elemsize == 4 || elemsize == 2, "ncnnhip_conv_int8_nhwc_from_float: activations are fp32 (4) or fp16 (2), not %d bytes", elemsize);
    NCNNHIP_REQUIRE(ncnnhip_conv_from_float_supported(desc), "ncnnhip_conv_int8_nhwc_from_float: this layer needs its separate Quantize pass");
    NCNNHIP_REQUIRE((reinterpret_cast<uintptr_t>(nhwc_dev) & 15) == 0, "ncnnhip_conv_int8_nhwc_from_float: the blob must be 16-byte aligned");
    ConvFusion f = {0, 0, 0, 0.f};
    if (fusion)
    {
        NCNNHIP_REQUIRE(!scale_out_dev, "ncnnhip_conv_int8_nhwc_from_float: the fused tail belongs to the fp32 output");
        NCNNHIP_REQUIRE(!fusion->quantised_out_dev || fusion->quantise_scale != 0.f, "ncnnhip_conv_int8_nhwc_from_float: quantised copy without a scale");
        f.residual = fusion->residual_dev;
        f.relu_after = fusion->relu_after;
        f.q8_out = fusion->quantised_out_dev;
        f.q8_scale = fusion->quantise_scale;
    }
    return conv_int8_nhwc_impl(desc, nhwc_dev, elemsize, in_scale_dev, packed_weight_dev, scale_in_dev, bias_dev, scale_out_dev, act, out_dev, NCNNHIP_CHANNELS_LAST,
                               0, 0, f, workspace_dev, workspace_bytes, stream);
}

int ncnnhip_conv_stem_supported(const ncnnhip_conv_desc* desc)
{
    return desc && stem_supported(*desc) ? 1 : 0;
}

int ncnnhip_conv_stem_sizes(const ncnnhip_conv_desc* desc, size_t* image_bytes, size_t* packed_weight_bytes, size_t* workspace_bytes)
{
    NCNNHIP_REQUIRE(desc && stem_supported(*desc), "ncnnhip_conv_stem_sizes: needs group 1, at most 4 input channels, dilation_w 1, zero border value");
    StemShape s;
    int ret = stem_shape(*desc, s);
    if (ret) return ret;
    if (image_bytes) *image_bytes = (size_t)desc->batch * s.Hb * s.Wp * 4;
    if (packed_weight_bytes) *packed_weight_bytes = (size_t)desc->num_output * s.K;
    if (workspace_bytes) *workspace_bytes = conv_nhwc_pipelined_workspace_words(desc->num_output, (long long)desc->batch * s.outw * s.outh, s.K / 64) * sizeof(int32_t);
    return NCNNHIP_OK;
}

int ncnnhip_conv_stem_pack_weights(const ncnnhip_conv_desc* desc, const int8_t* weight_host, int8_t* packed_host)
{
    NCNNHIP_REQUIRE(desc && weight_host && packed_host && stem_supported(*desc), "ncnnhip_conv_stem_pack_weights: bad argument");
    StemShape s;
    int ret = stem_shape(*desc, s);
    if (ret) return ret;
    const int c = desc->c, kw = desc->kernel_w, kh = desc->kernel_h;
    for (int p = 0; p < desc->num_output; p++)
    {
        int8_t* row = packed_host + (size_t)p * s.K;
        for (int k = 0; k < s.K; k++) row[k] = 0;
        for (int q = 0; q < c; q++)
            for (int ky = 0; ky < kh; ky++)
                for (int kx = 0; kx < kw; kx++)
                    row[(ky * s.G + kx / 4) * 16 + (kx % 4) * 4 + q] = weight_host[(((size_t)p * c + q) * kh + ky) * kw + kx];
    }
    return NCNNHIP_OK;
}

int ncnnhip_quantize_stem(const ncnnhip_conv_desc* desc, const void* nhwc_dev, int elemsize, int src_cp, const float* scale_dev, int8_t* image_dev, void* stream)
{
    NCNNHIP_REQUIRE(desc && nhwc_dev && image_dev && stem_supported(*desc), "ncnnhip_quantize_stem: bad argument");
    NCNNHIP_REQUIRE((elemsize == 4 && scale_dev) || elemsize == 1, "ncnnhip_quantize_stem: fp32 (with a scale) or int8 input");
    NCNNHIP_REQUIRE(src_cp >= desc->c, "ncnnhip_quantize_stem: source pixel stride below the channel count");
    StemShape s;
    int ret = stem_shape(*desc, s);
    if (ret) return ret;
    NCNNHIP_REQUIRE(s.Hb <= 65535 && desc->batch <= 65535, "ncnnhip_quantize_stem: extent too large");
    NCNNHIP_REQUIRE(elemsize != 4 || src_cp != 4 || (reinterpret_cast<uintptr_t>(nhwc_dev) & 15) == 0, "ncnnhip_quantize_stem: a 4-float-per-pixel image must be 16-byte aligned");
    dim3 grid((unsigned)ceil_div(s.Wp, 256), (unsigned)s.Hb, (unsigned)desc->batch);
    if (elemsize == 4 && src_cp == 4 && (reinterpret_cast<uintptr_t>(image_dev) & 15) == 0)
    {
        hipLaunchKernelGGL(quantize_stem_narrow_kernel, dim3((unsigned)ceil_div(s.Wp / 4, 256), (unsigned)s.Hb, (unsigned)desc->batch), dim3(256), 0, as_stream(stream),
                           (const float*)nhwc_dev, desc->c, desc->h, desc->w, s.pads.top, s.pads.left, s.Hb, s.Wp, scale_dev, image_dev);
        return launch_status("quantize_stem_narrow_kernel");
    }
    if (elemsize == 4)
        hipLaunchKernelGGL(quantize_stem_kernel<float>, grid, dim3(256), 0, as_stream(stream), (const float*)nhwc_dev, src_cp, desc->c, desc->h, desc->w, s.pads.top,
                           s.pads.left, s.Hb, s.Wp, scale_dev, (uint32_t*)image_dev);
    else
        hipLaunchKernelGGL(quantize_stem_kernel<int8_t>, grid, dim3(256), 0, as_stream(stream), (const int8_t*)nhwc_dev, src_cp, desc->c, desc->h, desc->w,
                           s.pads.top, s.pads.left, s.Hb, s.Wp, (const float*)0, (uint32_t*)image_dev);
    return launch_status("quantize_stem_kernel");
}

int ncnnhip_conv_int8_stem(const ncnnhip_conv_desc* desc, const int8_t* image_dev, const int8_t* packed_weight_dev, const float* scale_in_dev,
                           const float* bias_dev, const float* scale_out_dev, ncnnhip_activation act, void* out_dev, const ncnnhip_conv_fusion* fusion,
                           void* workspace_dev, size_t workspace_bytes, void* stream)
{
    NCNNHIP_REQUIRE(desc && image_dev && packed_weight_dev && scale_in_dev && out_dev, "ncnnhip_conv_int8_stem: null pointer");
    NCNNHIP_REQUIRE(stem_supported(*desc), "ncnnhip_conv_int8_stem: needs group 1, at most 4 input channels, dilation_w 1, zero border value");
    NCNNHIP_REQUIRE(!fusion || !scale_out_dev, "ncnnhip_conv_int8_stem: the fused tail belongs to the fp32 output");
    NCNNHIP_REQUIRE(!fusion || !fusion->quantised_out_dev || fusion->quantise_scale != 0.f, "ncnnhip_conv_int8_stem: quantised copy without a scale");
    const ncnnhip_conv_desc& d = *desc;
    StemShape s;
    int ret = stem_shape(d, s);
    if (ret) return ret;
    const long long plane = (long long)s.outw * s.outh, npix = plane * d.batch;
    NCNNHIP_REQUIRE(npix < (1ll << 31) && (long long)s.Hb * s.Wp * 4 < (1ll << 31), "ncnnhip_conv_int8_stem: extent too large");
    NhwcGeom g;
    g.H = s.Hb;
    g.W = s.Wp;
    g.Cp = 4;
    g.tapK = 16;
    g.kw = s.G;
    g.kh = d.kernel_h;
    g.dw = 4;
    g.dh = d.dilation_h;
    g.sw = d.stride_w;
    g.sh = d.stride_h;
    g.pad_top = g.pad_left = 0; // the border is part of the image
    g.outw = s.outw;
    g.outh = s.outh;
    g.npix = (int)npix;
    g.ntaps = d.kernel_h * s.G;
    g.K = s.K;
    g.cout = d.num_output;
    g.pad_word = 0;
    ConvEpilogue epi;
    epi.scale_in = scale_in_dev;
    epi.bias = bias_dev;
    epi.scale_out = scale_out_dev;
    epi.act = act;
    epi.out = out_dev;
    epi.out_cstep = epi.out_nstep = 0;
    epi.pix_per_img = (int)plane;
    epi.batch = d.batch;
    epi.out_channel0 = 0;
    epi.num_output = d.num_output;
    epi.acc_out = 0;
    ConvFusion f = {0, 0, 0, 0.f};
    if (fusion)
    {
        f.residual = fusion->residual_dev;
        f.relu_after = fusion->relu_after;
        f.q8_out = fusion->quantised_out_dev;
        f.q8_scale = fusion->quantise_scale;
    }
    return launch_conv_nhwc_pipelined(g, packed_weight_dev, image_dev, epi, f, padded_channels(d.num_output), workspace_dev, workspace_bytes, as_stream(stream));
}

} // extern "C"
