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
//     it, after which every lane holds 16 consecutive output bytes of one pixel: one 16-byte store -- to global memory where
//     that is the whole pixel record, else to LDS, from where the workgroup's pixel blocks leave as whole lines.
// The same kernel serves the narrow-input first layer of a net (STEM: at most 4 input channels, the quantised image of 4
// bytes per pixel with its physical zero border, kernels of up to 4 x 4 taps at any stride): there a 16-byte operand
// chunk is 4 neighbouring pixels of one kernel row, and a lane finds its chunk by its output pixel's position in the
// bordered image.  Everything after the MFMAs is shared.  (KSTEPS > 1 -- longer K -- compiles and is bit-exact, but
// measured slower than the pipelined kernel and is not launched.)
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

// A workgroup owns G (1 or 2) 64-pixel blocks and ALL output channels of them: wavefront w works on pixel block w % G and
// on the 16-channel blocks w / G, w / G + 4 / G, ...  Every 128-byte line of the output is therefore written by one
// workgroup, within a few hundred cycles, through one L2: with a wavefront per (pixel run, channel block) spread over the
// chip, the 16-byte pieces of a line came from workgroups on different XCDs, each L2 wrote its pieces back as partial lines,
// and the layer ran at 1.3-2 TB/s of output (block2_expand of MobileNetV2 at batch 32: 21.4 us for 38.5 MB).
// The channel tables (input scale, bias, output scale, clamp bounds) are worked out once per workgroup into LDS, with the
// decision whether the clip folds into the clamp; a wavefront keeps its pixel block's four operands in registers for all
// its channel blocks and fetches the next channel block's weights while it requantises this one.
// KSTEPS: 64-byte K steps (MFMAs per result); STEM: the narrow-input geometry (g is the bordered image then: pixels 4 bytes
// apart, kw counts groups of 4 pixels, no padding left to apply).  G = 4 (one wavefront per pixel block, every channel block)
// exists for layers of one or two channel blocks.
template<int KSTEPS, bool STEM>
__global__ __launch_bounds__(256) void conv_pointwise_int8_kernel(const int8_t* __restrict__ wpk /* [cout][KSTEPS * 64] */, const int8_t* __restrict__ x, NhwcGeom g,
                                                                   int out_cp, const float* __restrict__ scale_in, const float* __restrict__ bias_tab,
                                                                   const float* __restrict__ scale_out, ncnnhip_activation act, int8_t* __restrict__ out,
                                                                   int channel_blocks, int G, int staged)
{
    extern __shared__ __attribute__((aligned(16))) float pw_tab[]; // [5][out_cp]: input scale, bias, output scale, clamp low, clamp high; then (staged) the G pixel blocks' results, [64][out_cp] bytes each
    typedef int v4i_dword_aligned __attribute__((ext_vector_type(4), aligned(4)));
    const int cp_in = g.Cp, npix = g.npix, cout = g.cout;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c16 = lane & 15, q = lane >> 4;
    const int pixel_blocks = (npix + 63) >> 6;
    const int pb = (int)blockIdx.x * G + (G == 4 ? wave : G == 2 ? (wave & 1) : 0);
    const int cb_first = G == 4 ? 0 : G == 2 ? (wave >> 1) : wave;
    const int cb_step = G == 4 ? 1 : 4 / G;
    const bool live = pb < pixel_blocks; // (uniform per wavefront; a dead wavefront still helps with the tables and the barrier)

    // ---- this wavefront's pixels: lane = pixel pb*64 + pg*16 + c16, bytes q*16 .. +16.  Nothing is selected after the load: a
    // lane whose bytes lie beyond the pixel (cp_in < 64) reads the pixel's first bytes instead, and they meet weights that are
    // zero there (the packed rows are zero-filled from cp_in up); a lane whose pixel lies beyond the end reads the last pixel,
    // and its results are never stored.
    const unsigned koff = q * 16 < cp_in ? q * 16 : 0;
    v4i fx[4][KSTEPS];
    {
        const int pbl = live ? pb : pixel_blocks - 1;
        if constexpr (STEM)
        {
            // chunk c = 4 * step + q of K is kernel row c / kw, pixel group c % kw: (row * dh * W + group * 4) pixels from the
            // output pixel's corner; chunks beyond the kernel meet zero weights and read the first chunk again
            int chunk_off[KSTEPS];
#pragma unroll
            for (int st = 0; st < KSTEPS; st++)
            {
                int c = 4 * st + q;
                if (c >= g.ntaps) c = 0;
                const int ky = small_div(c, g.kw);
                chunk_off[st] = (ky * g.dh * g.W + (c - ky * g.kw) * 4) * 4;
            }
            // the block's first pixel by (uniform) division, the lane's own by walking on from there
            const int plane = g.outw * g.outh;
            const int p0 = pbl * 64;
            const int img0 = p0 / plane, rem0 = p0 - img0 * plane;
            const int oy0 = rem0 / g.outw, ox0 = rem0 - oy0 * g.outw;
#pragma unroll
            for (int pg = 0; pg < 4; pg++)
            {
                int step = pg * 16 + c16;
                if (p0 + step >= npix) step = npix - 1 - p0; // a pixel beyond the end reads the last one; never stored
                int img = img0, oy = oy0, ox = ox0 + step;
                while (ox >= g.outw)
                {
                    ox -= g.outw;
                    if (++oy == g.outh)
                    {
                        oy = 0;
                        img++;
                    }
                }
                const int8_t* corner = x + ((size_t)(img * g.H + oy * g.sh) * g.W + ox * g.sw) * 4;
#pragma unroll
                for (int st = 0; st < KSTEPS; st++) fx[pg][st] = *reinterpret_cast<const v4i_dword_aligned*>(corner + chunk_off[st]);
            }
        }
        else
        {
#pragma unroll
            for (int pg = 0; pg < 4; pg++)
            {
                int p = pbl * 64 + pg * 16 + c16;
                if (p >= npix) p = npix - 1;
                fx[pg][0] = *reinterpret_cast<const v4i*>(x + (size_t)p * cp_in + koff);
            }
        }
    }
    struct Weights
    {
        v4i w[KSTEPS];
    };
    auto load_weights = [&](int cb) {
        int ch = cb * 16 + c16;
        if (ch >= cout) ch = cout - 1; // rows beyond cout give values that the zero tables turn into zero bytes
        Weights r;
#pragma unroll
        for (int st = 0; st < KSTEPS; st++) r.w[st] = *reinterpret_cast<const v4i*>(wpk + (size_t)ch * (KSTEPS * 64) + st * 64 + q * 16);
        return r;
    };
    Weights fw = load_weights(cb_first < channel_blocks ? cb_first : 0);

    // ---- tables of every channel, once per workgroup.  Channels from cout up (the blob's padding) get scale 0 and bias -0:
    // their bytes come out 0.  A clip folds into the requantising clamp when every table allows it (finite tables, products
    // below 2^31, an output scale that is not negative); without a negative clamp bound the rounding is one conversion.
    bool tame = act.type == 3, nonneg = true;
    {
        const float clip_abs = fmaxf(fabsf(act.p0), fabsf(act.p1));
        const bool clip_finite = fabsf(act.p0) < INFINITY && fabsf(act.p1) < INFINITY;
        for (int ch = threadIdx.x; ch < out_cp; ch += 256)
        {
            const bool real = ch < cout;
            const float si = real ? scale_in[ch] : 0.f;
            const float bi = (real && bias_tab) ? bias_tab[ch] : -0.f; // x + -0 = x for every x
            const float so = real ? scale_out[ch] : 0.f;
            const float lo = __builtin_amdgcn_fmed3f(mul_rn(act.p0, so), -127.f, 127.f);
            const float hi = __builtin_amdgcn_fmed3f(mul_rn(act.p1, so), -127.f, 127.f);
            tame = tame && clip_finite && fabsf(si) < 0x1p90f && fabsf(bi) < 0x1p120f && mul_rn(clip_abs, fabsf(so)) < 2147483648.f
                   && clip_folds_into_requantise(act.p0, act.p1, so);
            nonneg = nonneg && lo >= 0.f;
            pw_tab[ch] = si;
            pw_tab[out_cp + ch] = bi;
            pw_tab[2 * out_cp + ch] = so;
            pw_tab[3 * out_cp + ch] = lo;
            pw_tab[4 * out_cp + ch] = hi;
        }
        const int failed = __syncthreads_or((tame ? 0 : 1) | (nonneg ? 0 : 2));
        tame = !(failed & 1);
        nonneg = tame && !(failed & 2);
    }
    if (!live) return;
    const int mode = act.type == 0 ? 0 : act.type == 1 ? 1 : act.type == 3 ? (nonneg ? 203 : tame ? 103 : 3) : -1;

    const int p_store = pb * 64 + q * 16 + c16;
    int8_t* orow = out + (size_t)p_store * out_cp;
    // staged: the pixel block's results meet in LDS as they lie in the blob -- 64 consecutive pixel records are 64 * out_cp
    // consecutive bytes -- and leave as whole lines (a lane's own 16 bytes are 1/6 of a 96-byte record: one partial line per lane)
    int8_t* const stage_block = reinterpret_cast<int8_t*>(pw_tab + 5 * out_cp) + (size_t)(G == 4 ? wave : G == 2 ? (wave & 1) : 0) * 64 * out_cp;
    int8_t* const srow = stage_block + (q * 16 + c16) * out_cp;
    for (int cb = cb_first; cb < channel_blocks; cb += cb_step)
    {
        const Weights w_now = fw;
        if (cb + cb_step < channel_blocks) fw = load_weights(cb + cb_step); // in flight while this block is requantised
        const float* t = pw_tab + cb * 16 + 4 * q;
        const v4f vsi = *reinterpret_cast<const v4f*>(t), vbi = *reinterpret_cast<const v4f*>(t + out_cp), vso = *reinterpret_cast<const v4f*>(t + 2 * out_cp);
        const v4f vlo = *reinterpret_cast<const v4f*>(t + 3 * out_cp), vhi = *reinterpret_cast<const v4f*>(t + 4 * out_cp);
        const float s_in[4] = {vsi[0], vsi[1], vsi[2], vsi[3]}, bias[4] = {vbi[0], vbi[1], vbi[2], vbi[3]}, s_out[4] = {vso[0], vso[1], vso[2], vso[3]};
        const float q_lo[4] = {vlo[0], vlo[1], vlo[2], vlo[3]}, q_hi[4] = {vhi[0], vhi[1], vhi[2], vhi[3]};
        v4i acc[4];
#pragma unroll
        for (int pg = 0; pg < 4; pg++)
        {
            acc[pg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w_now.w[0], fx[pg][0], v4i{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
            for (int st = 1; st < KSTEPS; st++) acc[pg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w_now.w[st], fx[pg][st], acc[pg], 0, 0, 0);
        }

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
        if (staged)
            *reinterpret_cast<v4i*>(srow + cb * 16) = pk;
        else if (p_store < npix)
            *reinterpret_cast<v4i*>(orow + cb * 16) = pk;
    }
    if (staged)
    {
        // (wavefronts of pixel blocks beyond the end have left; the barrier counts those that remain)
        __syncthreads();
        const int waves_per_block = G == 4 ? 1 : 4 / G, my = G == 4 ? 0 : wave / G;
        const int pixels_here = npix - pb * 64 < 64 ? npix - pb * 64 : 64;
        const int nchunks = pixels_here * (out_cp >> 4);
        int8_t* const gblock = out + (size_t)pb * 64 * out_cp;
        for (int i = my * 64 + lane; i < nchunks; i += 64 * waves_per_block)
            *reinterpret_cast<v4i*>(gblock + (size_t)i * 16) = *reinterpret_cast<const v4i*>(stage_block + (size_t)i * 16);
    }
}

bool conv_pointwise_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp)
{
    const bool dense = g.kw == 1 && g.kh == 1 && g.sw == 1 && g.sh == 1 && g.pad_top == 0 && g.pad_left == 0 && g.outw == g.W && g.outh == g.H && g.tapK == g.Cp;
    const bool plain = !fusion.residual && !fusion.relu_after && !fusion.q8_out && !epi.acc_out;
    const uintptr_t tables = reinterpret_cast<uintptr_t>(epi.scale_in) | reinterpret_cast<uintptr_t>(epi.bias) | reinterpret_cast<uintptr_t>(epi.scale_out);
    const bool aligned = ((tables | reinterpret_cast<uintptr_t>(epi.out)) & 15) == 0; // 16-byte table loads and stores
    return dense && plain && aligned && epi.scale_out && g.Cp <= 64 && g.Cp % 16 == 0 && g.K == 64 && g.cout % 4 == 0 && out_cp % 16 == 0 && g.npix >= (1 << 16); // below that the general kernel's finer split of the work is as fast or faster (measured again with this kernel's present form on MobileNetV2's 28 x 28 to 7 x 7 layers at batch 32: 5.7-6.1 us there against 6.9-10 here)
}

// The narrow-input first layer (ncnnhip_conv_int8_stem presents it as pixels 4 bytes apart whose taps are groups of 4
// pixels, with the border inside the image): int8 output, no fused tail, as many pixels as the 1x1 layers need before this
// kernel is the faster one, and a K of ONE step (kernels of up to 4 rows of up to 4 taps: MobileNetV2's 3x3 first layer at
// batch 32 17.4 -> 10.3 us).  With four steps (ResNet-50's 7x7: 14 chunks) it measured SLOWER than the pipelined kernel,
// 18.9 against 16.1 us at batch 16 and 187 against 132 at batch 128: sixteen 16-byte gathers per lane from windows that
// overlap their neighbours' by half, fetched again by the wavefront that takes the other channel blocks.
bool conv_pointwise_stem_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp)
{
    const bool stem = g.Cp == 4 && g.tapK == 16 && g.dw == 4 && g.pad_top == 0 && g.pad_left == 0 && g.pad_word == 0 && g.ntaps == g.kw * g.kh;
    const bool plain = !fusion.residual && !fusion.relu_after && !fusion.q8_out && !epi.acc_out;
    const uintptr_t tables = reinterpret_cast<uintptr_t>(epi.scale_in) | reinterpret_cast<uintptr_t>(epi.bias) | reinterpret_cast<uintptr_t>(epi.scale_out);
    const bool aligned = ((tables | reinterpret_cast<uintptr_t>(epi.out)) & 15) == 0;
    return stem && plain && aligned && epi.scale_out && g.ntaps <= 4 && g.K == 64 && g.cout % 4 == 0 && out_cp % 16 == 0 &&
           g.npix >= (1 << 16) && (long long)g.npix + 64 < (1ll << 31);
}

int launch_conv_pointwise(const NhwcGeom& g, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, int out_cp, hipStream_t stream)
{
    NCNNHIP_REQUIRE(((reinterpret_cast<uintptr_t>(wpk) | reinterpret_cast<uintptr_t>(x)) & 15) == 0, "convolution: operands must be 16-byte aligned");
    const int channel_blocks = out_cp / 16;
    const int pixel_blocks = ceil_div(g.npix, 64);
    const size_t tab_bytes = (size_t)5 * out_cp * sizeof(float);
    NCNNHIP_REQUIRE(tab_bytes <= 60 * 1024, "convolution: %d output channels are too many for the pointwise kernel's tables", g.cout);
    if (g.Cp == 4 && g.tapK == 16)
    {
        // one wavefront per pixel block walks one or two channel blocks; more are dealt to wavefront pairs as below
        const int Gs = channel_blocks <= 2 ? 4 : 2;
        const dim3 grid((unsigned)ceil_div(pixel_blocks, Gs));
        NCNNHIP_REQUIRE(g.K == 64 && g.ntaps <= 4, "convolution: %d bytes of K in the narrow-input form of the pointwise kernel", g.K);
        hipLaunchKernelGGL((conv_pointwise_int8_kernel<1, true>), grid, dim3(256), tab_bytes, stream, wpk, x, g, out_cp, epi.scale_in, epi.bias, epi.scale_out,
                           epi.act, static_cast<int8_t*>(epi.out), channel_blocks, Gs, 0);
        return launch_status("conv_pointwise_int8_kernel (narrow input)");
    }
    // pixel blocks per workgroup: two, each with two wavefronts that take the even and the odd channel blocks (measured on
    // MobileNetV2's 16 -> 96 expansion on 112 x 112 at batch 32: 19.8 us, against 23.1 for one block with four wavefronts and
    // 31 for four blocks with one wavefront each); a layer too small for that many workgroups keeps one block per workgroup
    const int G = pixel_blocks >= 1024 ? 2 : 1;
    // results through LDS, leaving as whole lines, where a pixel record is several channel blocks long (MobileNetV2 at batch 32:
    // 16 -> 96 on 112 x 112 21.8 -> 20.6 us, 24 -> 144 on 56 x 56 11.25 -> 10.5); a record of one block is a lane's own 16 bytes
    // already (32 -> 16 on 112 x 112: 10.5 us direct, 12.3 staged)
    const int staged = channel_blocks > 1 && tab_bytes + (size_t)G * 64 * out_cp <= 60 * 1024;
    const size_t lds = tab_bytes + (staged ? (size_t)G * 64 * out_cp : 0);
    hipLaunchKernelGGL((conv_pointwise_int8_kernel<1, false>), dim3((unsigned)ceil_div(pixel_blocks, G)), dim3(256), lds, stream, wpk, x, g, out_cp, epi.scale_in,
                       epi.bias, epi.scale_out, epi.act, static_cast<int8_t*>(epi.out), channel_blocks, G, staged);
    return launch_status("conv_pointwise_int8_kernel");
}

} // namespace ncnnhip
