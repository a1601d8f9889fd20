// 1x1, stride-1, unpadded convolution with at most 64 input bytes per pixel and int8 output: the "expand" layers of
// an inverted-residual block and their like (Convolution::forward_int8 with kernel 1x1, src/layer/convolution.cpp:
// 370-470, followed by the requantisation of src/layer/convolution.cpp:472-512).
//
// These layers have almost no matrix work (K = 16..64) and a lot of output, so the general kernel's per-workgroup
// prologue, its LDS staging and its LDS transposition of the results dominate: it issues about 19 vector instructions
// per output value.  Here nothing goes through LDS and nothing is shared between wavefronts:
//   * v_mfma_i32_16x16x64_i8 takes the whole K in one instruction and is fed weights as the A operand and pixels as the
//     B operand, so that a lane's 4 accumulators are 4 consecutive CHANNELS (4*(lane/16) .. +4 of a 16-channel block)
//     of ONE pixel (lane%16 of a 16-pixel group): one dword of the channels-last output, and only 4 channels' worth of
//     scale/bias/clamp tables per lane;
//   * a wavefront keeps ONE 16-channel block for its whole life: the block's weights (16 bytes per lane) and tables
//     are loaded once and serve a run of 64-pixel blocks, four MFMAs each;
//   * operands come straight from global memory into the MFMA's registers (16 bytes per lane), the next block's while
//     the current one is being requantised;
//   * the four packed words of a lane (same channels, four pixel groups) and those of the lanes 16, 32 and 48 away
//     (same pixels, the other channels) are a 4x4 matrix across lane rows and registers: four lane-row swaps transpose
//     it, after which every lane holds 16 consecutive output bytes of one pixel: one 16-byte store.
// About 9 vector instructions per output value at 4+ wavefronts per SIMD.  Activations: none, ReLU, clip (literal or,
// when the tables allow it, folded into the requantising clamp: clip_folds_into_requantise in common.h), others.
#include "common.h"
#include "conv_nhwc.h"

namespace ncnnhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ACT: 0 none, 1 ReLU, 3 clip as written, 103 clip folded into the clamp (tame tables), 203 the same with no negative clamp
// bound (rounding by one conversion, pack16_nonneg), -1 anything else.
// acc[pg][r]: pixel group pg, channel r of the lane's four; returns one packed word per pixel group.
template<int ACT>
__device__ __forceinline__ void pointwise_requantise(const v4i (&acc)[4], const float (&s_in)[4], const float (&bias)[4], const float (&s_out)[4],
                                                     const float (&q_lo)[4], const float (&q_hi)[4], const ncnnhip_activation& act, uint32_t (&word)[4])
{
    float f[16];
#pragma unroll
    for (int pg = 0; pg < 4; pg++)
    {
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            float v = add_rn(mul_rn((float)acc[pg][r], s_in[r]), bias[r]);
            if (ACT == 1)
                v = fmaxf(v, 0.f);
            else if (ACT == 3)
            {
                if (v < act.p0) v = act.p0;
                if (v > act.p1) v = act.p1;
            }
            else if (ACT == -1)
                v = apply_activation(v, act);
            f[4 * pg + r] = mul_rn(v, s_out[r]);
        }
        if (ACT == 203)
        {
#pragma unroll
            for (int r = 0; r < 4; r++) f[4 * pg + r] = __builtin_amdgcn_fmed3f(f[4 * pg + r], q_lo[r], q_hi[r]);
        }
        else if (ACT == 103)
            float2int8_as_float_bounded_lanes_x4(f[4 * pg], f[4 * pg + 1], f[4 * pg + 2], f[4 * pg + 3], q_lo, q_hi);
        else
            float2int8_as_float_x4(f[4 * pg], f[4 * pg + 1], f[4 * pg + 2], f[4 * pg + 3]);
    }
    if (ACT == 203)
        pack16_nonneg(f, word[0], word[1], word[2], word[3]);
    else
        pack16_quantised(f, word[0], word[1], word[2], word[3]);
}

// grid: one wavefront per (run of `blocks_per_wave` 64-pixel blocks, 16-channel block), channel block fastest so that
// the wavefronts that read the same pixels run together; 4 independent wavefronts per workgroup.
__global__ __launch_bounds__(256) void conv_pointwise_int8_kernel(const int8_t* __restrict__ wpk /* [cout][64] */, const int8_t* __restrict__ x, int cp_in, int npix,
                                                                   int cout, int out_cp, const float* __restrict__ scale_in, const float* __restrict__ bias_tab,
                                                                   const float* __restrict__ scale_out, ncnnhip_activation act, int8_t* __restrict__ out,
                                                                   int channel_blocks, int blocks_per_wave, unsigned total_waves, unsigned cb_magic)
{
    const int lane = threadIdx.x & 63;
    const int c16 = lane & 15, q = lane >> 4;
    const unsigned wid = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
    if (wid >= total_waves) return;
    // wid = run * channel_blocks + cb, by multiplication (wid * channel_blocks < 2^32 is checked at launch)
    const unsigned run = channel_blocks == 1 ? wid : __umulhi(wid, cb_magic);
    const int cb = (int)(wid - run * (unsigned)channel_blocks);
    const int pixel_blocks = (npix + 63) >> 6;
    const int pb_begin = (int)run * blocks_per_wave;
    int pb_end = pb_begin + blocks_per_wave;
    if (pb_end > pixel_blocks) pb_end = pixel_blocks;

    // ---- weights: row = channel cb*16 + c16 (clamped: rows beyond cout give values nobody keeps), bytes q*16 .. +16
    v4i fw;
    {
        int ch = cb * 16 + c16;
        if (ch >= cout) ch = cout - 1;
        fw = *reinterpret_cast<const v4i*>(wpk + (size_t)ch * 64 + q * 16);
    }
    // ---- pixel operand of pixel group pg: lane = pixel pb*64 + pg*16 + c16, bytes q*16 .. +16.  Nothing is selected
    // after the load (a select would make the wavefront wait for the load where it is issued, not where it is used):
    // a lane whose bytes lie beyond the pixel (cp_in < 64) reads the pixel's first bytes instead, and they meet weights
    // that are zero there (the packed rows are zero-filled from cp_in up); a lane whose pixel lies beyond the end reads
    // the last pixel, and its results are never stored.  Address = uniform block base + a per-lane constant.
    const unsigned koff = q * 16 < cp_in ? q * 16 : 0;
    const unsigned lane_off = (unsigned)c16 * (unsigned)cp_in + koff;
    auto load_pixels = [&](int pb, v4i (&f)[4]) {
        if (pb * 64 + 64 <= npix) // uniform: a whole block
        {
            const int8_t* base = x + (size_t)pb * 64 * cp_in;
#pragma unroll
            for (int pg = 0; pg < 4; pg++) f[pg] = *reinterpret_cast<const v4i*>(base + (size_t)(pg * 16) * cp_in + lane_off);
        }
        else
        {
#pragma unroll
            for (int pg = 0; pg < 4; pg++)
            {
                int p = pb * 64 + pg * 16 + c16;
                if (p >= npix) p = npix - 1;
                f[pg] = *reinterpret_cast<const v4i*>(x + (size_t)p * cp_in + koff);
            }
        }
    };

    v4i fx[2][4];
    if (pb_begin < pb_end) load_pixels(pb_begin, fx[0]); // on its way while the tables are loaded and examined
    // ---- tables of the lane's channels cb*16 + 4q .. +4.  Channels from cout up (the blob's padding) get scale 0 and
    // bias -0: their bytes come out 0.  cout % 4 == 0 (checked at launch), so a quad is real or it is not.
    float s_in[4], bias[4], s_out[4], q_lo[4], q_hi[4];
    {
        const int ch0 = cb * 16 + 4 * q;
        const bool real = ch0 < cout;
        const int chl = real ? ch0 : 0;
        const v4f a = *reinterpret_cast<const v4f*>(scale_in + chl);
        const v4f b = bias_tab ? *reinterpret_cast<const v4f*>(bias_tab + chl) : v4f{-0.f, -0.f, -0.f, -0.f};
        const v4f c = *reinterpret_cast<const v4f*>(scale_out + chl);
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            s_in[e] = real ? a[e] : 0.f;
            bias[e] = real ? b[e] : -0.f; // x + -0 = x for every x
            s_out[e] = real ? c[e] : 0.f;
        }
    }
    // clip: can it be folded into the clamp?  (the general kernel's conditions, per wavefront)
    bool tame = false;
#pragma unroll
    for (int r = 0; r < 4; r++) q_lo[r] = q_hi[r] = 0.f;
    if (act.type == 3)
    {
        const float clip_abs = fmaxf(fabsf(act.p0), fabsf(act.p1));
        tame = fabsf(act.p0) < INFINITY && fabsf(act.p1) < INFINITY;
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            tame = tame && fabsf(s_in[r]) < 0x1p90f && fabsf(bias[r]) < 0x1p120f && mul_rn(clip_abs, fabsf(s_out[r])) < 2147483648.f
                   && clip_folds_into_requantise(act.p0, act.p1, s_out[r]);
            q_lo[r] = __builtin_amdgcn_fmed3f(mul_rn(act.p0, s_out[r]), -127.f, 127.f);
            q_hi[r] = __builtin_amdgcn_fmed3f(mul_rn(act.p1, s_out[r]), -127.f, 127.f);
        }
        tame = __all(tame);
    }
    const bool nonneg = tame && __all(q_lo[0] >= 0.f && q_lo[1] >= 0.f && q_lo[2] >= 0.f && q_lo[3] >= 0.f);
    const int mode = act.type == 0 ? 0 : act.type == 1 ? 1 : act.type == 3 ? (nonneg ? 203 : tame ? 103 : 3) : -1;

    const unsigned store_off = (unsigned)(q * 16 + c16) * (unsigned)out_cp + (unsigned)cb * 16; // within a 64-pixel block
    for (int pb0 = pb_begin; pb0 < pb_end; pb0 += 2)
    {
#pragma unroll
        for (int j = 0; j < 2; j++)
        {
            const int pb = pb0 + j;
            if (pb >= pb_end) break; // uniform
            if (pb + 1 < pb_end) load_pixels(pb + 1, fx[j ^ 1]); // in flight while this block is computed
            v4i acc[4];
#pragma unroll
            for (int pg = 0; pg < 4; pg++) acc[pg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw, fx[j][pg], v4i{0, 0, 0, 0}, 0, 0, 0);

            uint32_t word[4];
            if (mode == 203)
                pointwise_requantise<203>(acc, s_in, bias, s_out, q_lo, q_hi, act, word);
            else if (mode == 103)
                pointwise_requantise<103>(acc, s_in, bias, s_out, q_lo, q_hi, act, word);
            else if (mode == 1)
                pointwise_requantise<1>(acc, s_in, bias, s_out, q_lo, q_hi, act, word);
            else if (mode == 0)
                pointwise_requantise<0>(acc, s_in, bias, s_out, q_lo, q_hi, act, word);
            else if (mode == 3)
                pointwise_requantise<3>(acc, s_in, bias, s_out, q_lo, q_hi, act, word);
            else
                pointwise_requantise<-1>(acc, s_in, bias, s_out, q_lo, q_hi, act, word);

            // word[pg] in lane row q (16 lanes) = channels 4q..4q+3 of pixel pg*16 + c16.  Transposing the 4x4 matrix
            // (lane row, register) leaves lane row q with words 0..3 = channels 0..15 of pixel q*16 + c16:
            //   swap32(a, b): rows 2,3 of a <-> rows 0,1 of b;   swap16(a, b): rows 1,3 of a <-> rows 0,2 of b.
            auto s02 = __builtin_amdgcn_permlane32_swap(word[0], word[2], false, false);
            auto s13 = __builtin_amdgcn_permlane32_swap(word[1], word[3], false, false);
            auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
            auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
            const v4i pk = {(int)t01[0], (int)t01[1], (int)t23[0], (int)t23[1]};
            const int p = pb * 64 + q * 16 + c16;
            if (p < npix) *reinterpret_cast<v4i*>(out + (size_t)pb * 64 * out_cp + store_off) = pk;
        }
    }
}

bool conv_pointwise_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp)
{
    const bool dense = g.kw == 1 && g.kh == 1 && g.sw == 1 && g.sh == 1 && g.pad_top == 0 && g.pad_left == 0 && g.outw == g.W && g.outh == g.H && g.tapK == g.Cp;
    const bool plain = !fusion.residual && !fusion.relu_after && !fusion.q8_out && !epi.acc_out;
    const uintptr_t tables = reinterpret_cast<uintptr_t>(epi.scale_in) | reinterpret_cast<uintptr_t>(epi.bias) | reinterpret_cast<uintptr_t>(epi.scale_out);
    const bool aligned = ((tables | reinterpret_cast<uintptr_t>(epi.out)) & 15) == 0; // 16-byte table loads and stores
    return dense && plain && aligned && epi.scale_out && g.Cp <= 64 && g.Cp % 16 == 0 && g.K == 64 && g.cout % 4 == 0 && out_cp % 16 == 0 && g.npix >= (1 << 16); // below that the general kernel's finer split of the work is as fast or faster
}

int launch_conv_pointwise(const NhwcGeom& g, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, int out_cp, hipStream_t stream)
{
    NCNNHIP_REQUIRE(((reinterpret_cast<uintptr_t>(wpk) | reinterpret_cast<uintptr_t>(x)) & 15) == 0, "convolution: operands must be 16-byte aligned");
    const int channel_blocks = out_cp / 16;
    const int pixel_blocks = ceil_div(g.npix, 64);
    // long runs amortise the wavefront's weights and tables; short ones fill the chip: at least 4096 wavefronts, about
    // what the chip holds at once (measured best against 2048, 3072, 6144 and 8192 on MobileNetV2's layers at batch 32)
    int blocks_per_wave = 16;
    while (blocks_per_wave > 2 && (long long)ceil_div(pixel_blocks, blocks_per_wave) * channel_blocks < 4096) blocks_per_wave /= 2;
    const long long waves = (long long)ceil_div(pixel_blocks, blocks_per_wave) * channel_blocks;
    NCNNHIP_REQUIRE(waves * channel_blocks < (1ll << 32), "convolution: too many tiles");
    const unsigned cb_magic = channel_blocks > 1 ? (unsigned)((1ull << 32) / (unsigned)channel_blocks + 1) : 0u;
    hipLaunchKernelGGL(conv_pointwise_int8_kernel, dim3((unsigned)ceil_div(waves, 4)), dim3(256), 0, stream, wpk, x, g.Cp, g.npix, g.cout, out_cp, epi.scale_in,
                       epi.bias, epi.scale_out, epi.act, static_cast<int8_t*>(epi.out), channel_blocks, blocks_per_wave, (unsigned)waves, cb_magic);
    return launch_status("conv_pointwise_int8_kernel");
}

} // namespace ncnnhip
