// The pipelined channels-last convolution kernel and its launch plan, shared by the translation units that instantiate it
// (conv_nhwc_pipelined.hip: one workgroup per tile; conv_nhwc_pipelined_split.hip: K split over workgroups, and the Gemm
// form; conv_nhwc_pipelined_staged.hip: the quantising loader).  Splitting the instantiations over three files is for
// build time only.
//
// int8 Convolution (group 1, zero border) on channels-last blobs, pipelined for the gfx950 matrix cores.
//
// GEMM view: D[pixel][channel] = sum_k X[pixel][k] * W[channel][k], k = (tap, input channel), both operands
// K-contiguous.  Pixels are the A operand and output channels the B operand of v_mfma_i32_32x32x32_i8, so a lane's
// accumulators are 16 pixels of ONE output channel: its scale, bias and requantisation factor are loaded once, and a
// wavefront store covers 32 consecutive channels of a pixel (128 contiguous bytes of an fp32 channels-last blob).
//
// One workgroup (4 wavefronts, 2x2) owns BM pixels x BN channels.  K is walked in 64-byte steps through a ring of
// LDS stages filled by direct global->LDS 16-byte loads, STAGES-1 steps ahead of the step being multiplied.  A
// stage holds [BM + BN rows][64 bytes]; the four 16-byte chunks of row r sit at position c ^ ((r >> 2) & 3) so
// that the 128-bit fragment reads of 16 consecutive rows spread over all banks; the swizzle is applied by choosing
// which source chunk a lane fetches.  The im2col gather is that choice of source address: (pixel, tap, 16
// channels) is one aligned 16-byte word of the blob, or -- outside the image, beyond the last tap, beyond the last
// pixel -- a line of zeros.
//
// Workgroup ids are dealt round-robin to the 8 XCDs; they are remapped so that an XCD works on consecutive tiles
// (channel tiles of one pixel tile are neighbours and share the activations in that XCD's L2).
// Small problems split K over workgroups inside the one launch: every workgroup of a tile but the last to finish
// dumps its accumulator registers to scratch (register-major, fully coalesced) and bumps the tile's counter; the
// last one adds the others' dumps to its own registers (integer addition: exact in any order), resets the counter
// and runs the normal epilogue.  Nobody waits for anybody, so the grid may be larger than the chip.
#ifndef NCNNHIP_CONV_NHWC_PIPELINED_KERNEL_H
#define NCNNHIP_CONV_NHWC_PIPELINED_KERNEL_H

#include <algorithm>
#include <mutex>
#include <type_traits>

#include "conv_nhwc.h"
#include "mfma_tile.h"

#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))
#define WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | ((((n) >> 4) & 3) << 14))

// ring depth of the direct-to-LDS pipeline: three stages everywhere; deeper rings (4 to 6 stages) measured no faster on any ResNet-50 /
// MobileNetV2 layer, alone or inside whole passes
#ifndef PIPE_RING
#define PIPE_RING 3
#endif

namespace ncnnhip {


// a line of zeros for gathers that leave the image (one copy per translation unit)
static __device__ __attribute__((aligned(64))) int8_t g_zero_line[64];

typedef float v4f __attribute__((ext_vector_type(4)));

// four already-quantised values (integers in [-127,127] held as floats) -> four bytes
__device__ __forceinline__ uint32_t pack4(const v4f& v)
{
    return pack4_quantised(v[0], v[1], v[2], v[3]);
}

// MODE: how a lane finds its source bytes.  0: any geometry; 1: dense (1x1, stride 1, unpadded: one row of npix pixels,
// also Gemm and InnerProduct); 2: taps of 16 or 32 bytes (the narrow-input image), a whole number of taps per K step.
// 3: any geometry whose taps are whole 64-byte steps (tapK % 64 == 0): a K step then lies inside ONE tap, the same for every
// lane, so the walk over taps is wavefront-uniform scalar arithmetic, and a lane's bounds test and address are computed
// once per tap instead of once per step (a tap of 256 channels is four steps: the other three are a load and an add).
// A template parameter because the choice sits inside the K loop: as run-time branches there it cost the 3x3 layers
// of ResNet-50's last stages 2-4 us each (15.4 against 11.4 us for 256 -> 256 on 14 x 14, batch 16).
//
// AIN: bytes per activation value.  1: the blob is int8 and goes global -> LDS directly, as described above.  4 (fp32)
// or 2 (fp16): the layer's Quantize pass happens here (Quantize::forward, src/layer/quantize.cpp:48-111, one scale):
// before the K loop the workgroup gathers its BM pixels x K im2col tile through registers, float2int8(value * scale)
// each value, and writes the bytes into a tile-sized LDS region (dynamic shared memory, BM * K bytes) in the layout a
// stage would have.  The weights of the tile (BN * K bytes) are requested in full before that and land in a region of
// their own while the loader works, so the K loop touches LDS only: no waits on memory, no barriers.  x points at the
// fp32 / fp16 blob, same channels-last geometry counted in values.
template<int BM, int BN, int STAGES, bool SPLITK, bool GEMM, int MODE, int AIN = 1>
__global__ __launch_bounds__(256) void conv_nhwc_pipelined_kernel(const int8_t* __restrict__ wpk, const int8_t* __restrict__ x, NhwcGeom g, ConvEpilogue epi,
                                                                   ConvFusion fusion, GemmTail gemm, int out_cp, int col_limit, int tiles_m, int tiles_n, int splits, int steps_per_split, unsigned magic_n, int32_t* __restrict__ partial, unsigned* __restrict__ counters,
                                                                   const float* __restrict__ a_scale, int a_cache_bytes)
{
    constexpr bool dense = MODE == 1;
    constexpr bool STAGED = AIN != 1;
    static_assert(!STAGED || (!GEMM && MODE != 2 && MODE != 3), "the quantising loader exists for convolutions on ordinary blobs");
    constexpr int TM = BM / 64, TN = BN / 64; // 32x32 blocks per wavefront along pixels / channels
    constexpr int LAR = BM / 64;              // 64-row groups of the activation tile
    constexpr int LA = STAGED ? 0 : LAR, LB = BN / 64; // direct-to-LDS loads per wavefront per stage
    static_assert(STAGES >= 2 && STAGES <= 7 && (STAGES - 2) * (LA + LB) < 64, "the vmcnt field counts to 63");
    constexpr int STAGE_BYTES = (BM + BN) * 64;
    constexpr int EPILOGUE_BYTES = 4 * 32 * (BN / 2 + 4) * 4; // per wavefront 32 pixels x (BN/2 + 4) floats
    constexpr int SMEM_BYTES = (!STAGED && STAGES * STAGE_BYTES > EPILOGUE_BYTES) ? STAGES * STAGE_BYTES : EPILOGUE_BYTES;
    __shared__ __attribute__((aligned(1024))) int8_t smem[SMEM_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    // ---- which tile: XCD x gets the x-th contiguous share of the tile list
    int b = blockIdx.x;
    {
        const int T = gridDim.x, xcd = b & 7, idx = b >> 3, rem = T & 7;
        b = xcd * (T >> 3) + (xcd < rem ? xcd : rem) + idx;
    }
    // b / tiles_n by multiplication: magic_n = 2^32/tiles_n + 1 is exact while b * tiles_n < 2^32 (checked at launch),
    // and stays on the scalar unit, where a division would be some twenty vector instructions per wavefront
    const int rest = tiles_n == 1 ? b : (int)__umulhi((unsigned)b, magic_n);
    const int tn = b - rest * tiles_n;
    const int split = SPLITK ? rest / tiles_m : 0;
    const int tm = rest - split * tiles_m;
    const int row0 = tm * BM, col0 = tn * BN;

    const int total_steps = g.K / 64;
    const int step_begin = SPLITK ? split * steps_per_split : 0;
    int step_end = SPLITK ? step_begin + steps_per_split : total_steps;
    if (step_end > total_steps) step_end = total_steps;
    const int nk = step_end - step_begin;
    const int tile_steps = SPLITK ? steps_per_split : total_steps; // K steps the quantising loader's LDS regions are sized for
    if (!SPLITK && nk <= 0) return; // (a split workgroup always has steps, and must reach the tile counter in any case)

    // ---- sources of this lane's loads.  Load i of a wavefront fills LDS rows i*64 + wave*16 .. +16 of the operand;
    // the lane's row is +lane/4 and it fetches source chunk (lane&3) ^ ((lane>>4)&3) into position lane&3.
    const int ld_row = wave * 16 + (lane >> 2);
    const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);
    const int8_t* zero = g_zero_line;

    const int8_t* a_base[LAR];
    int a_iy0[LAR], a_ix0[LAR];
    int a_img0[LAR]; // first pixel of the row's image, counted in input pixels over the whole batch (the quantising loader's cache)
#pragma unroll
    for (int i = 0; i < LAR; i++)
    {
        const int n = row0 + i * 64 + ld_row;
        const bool ok = n < g.npix;
        const int nn = ok ? n : 0;
        // dense: the launch presents a 1x1 stride-1 unpadded layer as one row of npix pixels, output pixel = input pixel
        int img = 0, oy = 0, ox = nn;
        if (!dense)
        {
            const int plane = g.outw * g.outh;
            if (g.npix < (1 << 20))
            {
                img = small_div(nn, plane);
                const int rem = nn - img * plane;
                oy = small_div(rem, g.outw);
                ox = rem - oy * g.outw;
            }
            else
            {
                img = nn / plane;
                const int rem = nn - img * plane;
                oy = rem / g.outw;
                ox = rem - oy * g.outw;
            }
        }
        // a pixel beyond the end gets coordinates that fail every bounds test
        a_iy0[i] = ok ? oy * g.sh - g.pad_top : -0x40000000;
        a_ix0[i] = ox * g.sw - g.pad_left;
        // dense: the pixel's own address, so that a stage's source is one 64-bit add away
        a_base[i] = dense ? x + (size_t)nn * g.Cp * AIN : x + (size_t)img * g.H * g.W * g.Cp * AIN;
        a_img0[i] = img * g.H * g.W;
    }
    const int8_t* b_ptr[LB];
#pragma unroll
    for (int i = 0; i < LB; i++)
    {
        int ch = col0 + i * 64 + ld_row;
        if (ch >= g.cout) ch = g.cout - 1; // a valid row; its products land in columns nobody stores
        b_ptr[i] = wpk + (size_t)ch * g.K + (size_t)step_begin * 64 + ld_chunk * 16;
    }
    // this lane's position in K: tap (ky,kx) and first channel q0 of its 16-byte chunk; +64 bytes per stage issued
    int q0, ky, kx, tap;
    {
        const int k = step_begin * 64 + ld_chunk * 16;
        if (dense)
        {
            // one tap; K beyond it is the round-up to 64, less than one tap's worth
            tap = k >= g.tapK ? 1 : 0;
            ky = tap;
            kx = 0;
        }
        else
        {
            if (g.K < (1 << 20)) // k < K
            {
                tap = small_div(k, g.tapK);
                ky = small_div(tap, g.kw);
            }
            else
            {
                tap = k / g.tapK;
                ky = tap / g.kw;
            }
            kx = tap - ky * g.kw;
        }
        q0 = k - tap * g.tapK;
    }
    const int first_q0 = q0, first_tap = tap, first_ky = ky, first_kx = kx; // where the quantising loader starts (issue() moves the others on)
    // MODE 3: the wavefront's position in K (the same in every lane) and, per lane, where the current tap's bytes of its
    // row are (or the line of zeros) and how far the next step moves on (64 bytes, or nothing on the line of zeros)
    int u_q0 = 0, u_tap = 0, u_ky = 0, u_kx = 0;
    bool u_new_tap = true;
    const int8_t* m3_src[LAR];
    int m3_step[LAR];
    if (MODE == 3)
    {
        const int k = step_begin * 64;
        u_tap = k / g.tapK;
        u_q0 = k - u_tap * g.tapK;
        u_ky = u_tap / g.kw;
        u_kx = u_tap - u_ky * g.kw;
#pragma unroll
        for (int i = 0; i < LAR; i++)
        {
            m3_src[i] = zero;
            m3_step[i] = 0;
        }
    }

    // issues the loads of the next stage in sequence (s = 0, 1, 2, ... relative to step_begin)
    extern __shared__ __attribute__((aligned(1024))) int8_t a_tile[]; // quantising loader: [K/64][BM][64] activations, then [K/64][BN][64] weights, then the input cache
    auto issue = [&](int s) {
        // quantising loader: every step has its own place (written once); the address below is that place minus the
        // activation part a ring stage would start with
        int8_t* stage = STAGED ? a_tile + tile_steps * (BM * 64) + s * (BN * 64) - BM * 64 + wave * 1024 : smem + (s % STAGES) * STAGE_BYTES + wave * 1024;
        if (dense)
        {
            // one tap, no border: the row's pixel exists or it does not (a_iy0 is 0 or hugely negative)
#pragma unroll
            for (int i = 0; i < LA; i++)
            {
                const bool in = tap == 0 && a_iy0[i] == 0;
                const int8_t* src = in ? a_base[i] + q0 : zero;
                __builtin_amdgcn_global_load_lds((const AS1 void*)src, (AS3 void*)(stage + i * 4096), 16, 0, 0);
            }
        }
        else if (MODE == 3)
        {
            if (u_new_tap) // (uniform)
            {
                const int dy = u_ky * g.dh, dx = u_kx * g.dw;
                const bool tap_ok = u_tap < g.ntaps;
#pragma unroll
                for (int i = 0; i < LA; i++)
                {
                    const int iy = a_iy0[i] + dy, ix = a_ix0[i] + dx;
                    const bool in = tap_ok && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                    m3_src[i] = in ? a_base[i] + ((size_t)iy * g.W + ix) * g.Cp + u_q0 + ld_chunk * 16 : zero;
                    m3_step[i] = in ? 64 : 0;
                }
            }
#pragma unroll
            for (int i = 0; i < LA; i++)
            {
                __builtin_amdgcn_global_load_lds((const AS1 void*)m3_src[i], (AS3 void*)(stage + i * 4096), 16, 0, 0);
                m3_src[i] += m3_step[i];
            }
        }
        else
        {
            const int dy = ky * g.dh, dx = kx * g.dw;
            const bool tap_ok = tap < g.ntaps;
#pragma unroll
            for (int i = 0; i < LA; i++)
            {
                const int iy = a_iy0[i] + dy, ix = a_ix0[i] + dx;
                const bool in = tap_ok && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                const int8_t* src = in ? a_base[i] + ((size_t)iy * g.W + ix) * g.Cp + q0 : zero;
                __builtin_amdgcn_global_load_lds((const AS1 void*)src, (AS3 void*)(stage + i * 4096), 16, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < LB; i++)
            __builtin_amdgcn_global_load_lds((const AS1 void*)(b_ptr[i] + (size_t)s * 64), (AS3 void*)(stage + BM * 64 + i * 4096), 16, 0, 0);
        // the lane's K position moves on by 64 bytes
        if (MODE == 1)
        {
            q0 += 64;
            if (q0 >= g.tapK) tap = 1; // past the only tap: the rest of K is the round-up, zero-filled
        }
        else if (MODE == 3)
        {
            u_q0 += 64;
            u_new_tap = u_q0 >= g.tapK;
            if (u_new_tap)
            {
                u_q0 = 0;
                u_tap++;
                if (++u_kx == g.kw)
                {
                    u_kx = 0;
                    u_ky++;
                }
            }
        }
        else if (MODE == 2)
        {
            // a whole number of taps per step; the offset inside the tap stays
            tap += g.tapK == 16 ? 4 : 2;
            ky = small_div(tap, g.kw);
            kx = tap - ky * g.kw;
        }
        else
        {
            q0 += 64;
            while (q0 >= g.tapK)
            {
                q0 -= g.tapK;
                tap++;
                if (++kx == g.kw)
                {
                    kx = 0;
                    ky++;
                }
            }
        }
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][c][r] = 0;

    // fragment read offsets inside a stage: row l32 of each 32-row block, K chunk ks*2 + lhi, swizzled
    const int sw = (l32 >> 2) & 3;
    const unsigned lds_base = (unsigned)(uintptr_t)(AS3 int8_t*)smem;
    const unsigned rd_a = (unsigned)((wm * (BM / 2) + l32) * 64);
    const unsigned rd_b = (unsigned)(BM * 64 + (wn * (BN / 2) + l32) * 64);
    const unsigned ch0 = (unsigned)(((0 + lhi) ^ sw) * 16), ch1 = (unsigned)(((2 + lhi) ^ sw) * 16);

    // The epilogue's per-channel tables are requested now, before the first stage, so that they arrive during the K
    // loop instead of costing a memory latency after it (a layer with a handful of K steps is little more than the
    // sum of its latencies).  Only the raw loads happen here, from clamped indices and always-valid pointers: a select
    // or a branch on the values would make the wavefront wait for them on the spot.
    float raw_s_in[BN / 64], raw_bias[BN / 64], raw_s_out[BN / 64];
    if (!GEMM)
    {
        const float* bias_src = epi.bias ? epi.bias : epi.scale_in;
        const float* s_out_src = epi.scale_out ? epi.scale_out : epi.scale_in;
#pragma unroll
        for (int c = 0; c < BN / 64; c++)
        {
            int ch = col0 + wn * (BN / 2) + c * 32 + l32;
            if (ch >= g.cout) ch = g.cout - 1;
            raw_s_in[c] = epi.scale_in[ch];
            raw_bias[c] = bias_src[ch];
            raw_s_out[c] = s_out_src[ch];
        }
    }

    if constexpr (STAGED)
        for (int s = 0; s < nk; s++) issue(s); // all the tile's weights at once (at most 48 loads per lane: the launch checks K)
    else
    {
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++)
            if (s < nk) issue(s);
    }

    // ---- the quantising loader: the whole activation tile, fp32 / fp16 -> int8, while the first weight stages arrive
    unsigned a_tile_lds = 0;
    if constexpr (STAGED)
    {
        a_tile_lds = (unsigned)(uintptr_t)(AS3 int8_t*)a_tile;
        const float sc = a_scale[0];
        int pq0 = first_q0, ptap = first_tap, pky = first_ky, pkx = first_kx;
        // The taps of neighbouring output pixels overlap: a 3x3 layer reads every input value nine times.  The input
        // pixels a tile touches form one contiguous run of the blob (counted over the whole batch, first tap of the
        // first row to last tap of the last row); when that run fits the cache region behind the tile, it is fetched
        // and quantised ONCE, fully coalesced and all loads in flight together, and the im2col tile is then gathered
        // from LDS.  Otherwise (and for 1x1 stride-1 layers, which read nothing twice) the tile is gathered from global
        // memory directly, three K steps at a time.
        bool cached = false;
        // (barriers in here wait for LDS traffic only: the weight stages requested above stay in flight)
        auto lds_barrier = [] {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        if (!dense && a_cache_bytes > 0)
        {
            // first and last input pixel of the tile: a wavefront reduction, then the four wavefronts' results through LDS
            __shared__ int run[4][2];
            int first = 0x7fffffff, last = -0x7fffffff;
            // taps this workgroup's K steps cover (all of them unless K is split); a tap's offset from the first one grows
            // with its index (the launch checks dh * W > (kw - 1) * dw), so the first and the last tap bound the run
            int tap_lo = 0, tap_hi = g.ntaps - 1;
            if (SPLITK)
            {
                tap_lo = (step_begin * 64) / g.tapK;
                const int t_hi = (step_end * 64 - 1) / g.tapK;
                tap_hi = t_hi < tap_hi ? t_hi : tap_hi;
                if (tap_lo > tap_hi) tap_lo = tap_hi; // a range that lies in the round-up of K: nothing is looked up
            }
            const int off_lo = (tap_lo / g.kw) * g.dh * g.W + (tap_lo % g.kw) * g.dw;
            const int off_hi = (tap_hi / g.kw) * g.dh * g.W + (tap_hi % g.kw) * g.dw;
#pragma unroll
            for (int i = 0; i < LAR; i++)
                if (a_iy0[i] > -0x40000000) // the row is a real output pixel
                {
                    const int f0 = a_img0[i] + a_iy0[i] * g.W + a_ix0[i];
                    const int f = f0 + off_lo, l = f0 + off_hi;
                    first = f < first ? f : first;
                    last = l > last ? l : last;
                }
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1)
            {
                const int of = __shfl_xor(first, d), ol = __shfl_xor(last, d);
                first = of < first ? of : first;
                last = ol > last ? ol : last;
            }
            if (lane == 0)
            {
                run[wave][0] = first;
                run[wave][1] = last;
            }
            lds_barrier();
#pragma unroll
            for (int w2 = 0; w2 < 4; w2++)
            {
                first = run[w2][0] < first ? run[w2][0] : first;
                last = run[w2][1] > last ? run[w2][1] : last;
            }
            // taps outside the image are never looked up, so the run may be cut to the blob
            const int in_pixels = epi.batch * g.H * g.W;
            const int lo = __builtin_amdgcn_readfirstlane(first > 0 ? first : 0);
            const int hi = __builtin_amdgcn_readfirstlane(last < in_pixels - 1 ? last : in_pixels - 1);
            const int count = hi - lo + 1;
            if (count > 0 && (long long)count * g.Cp <= (long long)a_cache_bytes)
            {
                cached = true;
                int8_t* cache = a_tile + tile_steps * ((BM + BN) * 64);
                // 4 values per lane and load: a wavefront instruction reads 1 KiB (fp32) or 512 B (fp16) of consecutive addresses
                const int nquad = count * (g.Cp >> 2);
                const int8_t* src0 = x + (size_t)lo * g.Cp * AIN;
                constexpr int INFL = 12; // loads in flight per lane
                for (int q0v = 0; q0v < nquad; q0v += 256 * INFL)
                {
                    v4f val[INFL];
#pragma unroll
                    for (int j = 0; j < INFL; j++)
                    {
                        int qi = q0v + j * 256 + (int)threadIdx.x;
                        if (qi >= nquad) qi = nquad - 1; // a valid address; the value is not stored
                        if constexpr (AIN == 4)
                            val[j] = *reinterpret_cast<const v4f*>(src0 + (size_t)qi * 16);
                        else
                        {
                            typedef unsigned v2u __attribute__((ext_vector_type(2)));
                            const v2u pair = *reinterpret_cast<const v2u*>(src0 + (size_t)qi * 8);
                            val[j][0] = (float)__builtin_bit_cast(_Float16, (unsigned short)(pair[0] & 0xffffu));
                            val[j][1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(pair[0] >> 16));
                            val[j][2] = (float)__builtin_bit_cast(_Float16, (unsigned short)(pair[1] & 0xffffu));
                            val[j][3] = (float)__builtin_bit_cast(_Float16, (unsigned short)(pair[1] >> 16));
                        }
                    }
#pragma unroll
                    for (int j = 0; j < INFL; j++)
                    {
                        const int qi = q0v + j * 256 + (int)threadIdx.x;
                        float v0 = mul_rn(val[j][0], sc), v1 = mul_rn(val[j][1], sc), v2 = mul_rn(val[j][2], sc), v3 = mul_rn(val[j][3], sc);
                        float2int8_as_float_x4(v0, v1, v2, v3);
                        const uint32_t word = pack4_quantised(v0, v1, v2, v3);
                        if (qi < nquad) *reinterpret_cast<uint32_t*>(cache + (size_t)qi * 4) = word;
                    }
                }
                lds_barrier();
                // the gather, LDS -> LDS: four K steps' reads in flight, then their writes
                constexpr int GATHER = 12;
                // the lane's first tap of its row, as a byte offset into the cache (may point outside: only looked up when the tap is inside the image)
                int row_byte0[LAR];
#pragma unroll
                for (int i = 0; i < LAR; i++) row_byte0[i] = (a_img0[i] + a_iy0[i] * g.W + a_ix0[i] - lo) * g.Cp;
                int8_t* const tile_lane = a_tile + wave * 1024 + lane * 16;
                if ((g.tapK & 63) == 0)
                {
                    // a K step lies inside one tap, the same for every lane: its position is wavefront-uniform arithmetic
                    const int chunk_byte = ld_chunk * 16;
                    // position of the workgroup's first K step
                    int stap = (step_begin * 64) / g.tapK;
                    int sq0 = step_begin * 64 - stap * g.tapK;
                    int sky = stap / g.kw;
                    int skx = stap - sky * g.kw;
                    for (int s0 = 0; s0 < nk; s0 += GATHER)
                    {
                        v4i piece[GATHER][LAR];
#pragma unroll
                        for (int u = 0; u < GATHER; u++)
                        {
                            const bool tap_ok = s0 + u < nk && stap < g.ntaps;
                            const int dy = sky * g.dh, dx = skx * g.dw;
                            const int step_byte = (dy * g.W + dx) * g.Cp + sq0 + chunk_byte;
#pragma unroll
                            for (int i = 0; i < LAR; i++)
                            {
                                const int iy = a_iy0[i] + dy, ix = a_ix0[i] + dx;
                                const bool in = tap_ok && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                                const v4i got = *reinterpret_cast<const v4i*>(cache + (in ? row_byte0[i] + step_byte : 0));
                                piece[u][i] = in ? got : v4i{0, 0, 0, 0}; // the border is zero bytes whatever the scale
                            }
                            sq0 += 64;
                            if (sq0 >= g.tapK)
                            {
                                sq0 = 0;
                                stap++;
                                if (++skx == g.kw)
                                {
                                    skx = 0;
                                    sky++;
                                }
                            }
                        }
#pragma unroll
                        for (int u = 0; u < GATHER; u++)
                            if (s0 + u < nk)
                            {
#pragma unroll
                                for (int i = 0; i < LAR; i++) *reinterpret_cast<v4i*>(tile_lane + (s0 + u) * (BM * 64) + i * 4096) = piece[u][i];
                            }
                    }
                }
                else
                    for (int s0 = 0; s0 < nk; s0 += GATHER)
                    {
                        v4i piece[GATHER][LAR];
#pragma unroll
                        for (int u = 0; u < GATHER; u++)
                        {
                            const bool tap_ok = s0 + u < nk && ptap < g.ntaps;
                            const int dy = pky * g.dh, dx = pkx * g.dw;
#pragma unroll
                            for (int i = 0; i < LAR; i++)
                            {
                                const int iy = a_iy0[i] + dy, ix = a_ix0[i] + dx;
                                const bool in = tap_ok && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                                const v4i got = *reinterpret_cast<const v4i*>(cache + (in ? row_byte0[i] + (dy * g.W + dx) * g.Cp + pq0 : 0));
                                piece[u][i] = in ? got : v4i{0, 0, 0, 0};
                            }
                            pq0 += 64;
                            while (pq0 >= g.tapK)
                            {
                                pq0 -= g.tapK;
                                ptap++;
                                if (++pkx == g.kw)
                                {
                                    pkx = 0;
                                    pky++;
                                }
                            }
                        }
#pragma unroll
                        for (int u = 0; u < GATHER; u++)
                            if (s0 + u < nk)
                            {
#pragma unroll
                                for (int i = 0; i < LAR; i++) *reinterpret_cast<v4i*>(tile_lane + (s0 + u) * (BM * 64) + i * 4096) = piece[u][i];
                            }
                    }
            }
        }
        constexpr int GRP = AIN == 4 ? 3 : 6; // K steps whose loads are in flight together (48 registers of raw values)
        constexpr int NLD = AIN == 4 ? 4 : 2; // 16-byte loads per 16 values
        for (int s0 = cached ? nk : 0; s0 < nk; s0 += GRP)
        {
            v4i raw[GRP][LAR][NLD];
            unsigned inside = 0; // bit u * LAR + i: the values are real (not border, not beyond K, not beyond the last pixel)
#pragma unroll
            for (int u = 0; u < GRP; u++)
            {
                const bool tap_ok = s0 + u < nk && (dense ? ptap == 0 : ptap < g.ntaps);
                const int dy = pky * g.dh, dx = pkx * g.dw;
#pragma unroll
                for (int i = 0; i < LAR; i++)
                {
                    bool in;
                    size_t off;
                    if (dense)
                    {
                        in = tap_ok && a_iy0[i] == 0;
                        off = (size_t)pq0;
                    }
                    else
                    {
                        const int iy = a_iy0[i] + dy, ix = a_ix0[i] + dx;
                        in = tap_ok && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                        off = ((size_t)iy * g.W + ix) * g.Cp + pq0;
                    }
                    const int8_t* src = in ? a_base[i] + off * AIN : zero;
                    inside |= in ? 1u << (u * LAR + i) : 0u;
#pragma unroll
                    for (int j = 0; j < NLD; j++) raw[u][i][j] = *reinterpret_cast<const v4i*>(src + 16 * j);
                }
                pq0 += 64;
                if (dense)
                {
                    if (pq0 >= g.tapK) ptap = 1;
                }
                else
                    while (pq0 >= g.tapK)
                    {
                        pq0 -= g.tapK;
                        ptap++;
                        if (++pkx == g.kw)
                        {
                            pkx = 0;
                            pky++;
                        }
                    }
            }
#pragma unroll
            for (int u = 0; u < GRP; u++)
            {
                if (s0 + u < nk)
                {
#pragma unroll
                    for (int i = 0; i < LAR; i++)
                    {
                        float v[16];
                        if constexpr (AIN == 4)
                        {
#pragma unroll
                            for (int j = 0; j < 4; j++)
#pragma unroll
                                for (int e = 0; e < 4; e++) v[j * 4 + e] = mul_rn(__int_as_float(raw[u][i][j][e]), sc);
                        }
                        else
                        {
#pragma unroll
                            for (int j = 0; j < 2; j++)
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                {
                                    const unsigned pair = (unsigned)raw[u][i][j][e]; // two halves, the first in the low 16 bits
                                    v[j * 8 + e * 2] = mul_rn((float)__builtin_bit_cast(_Float16, (unsigned short)(pair & 0xffffu)), sc);
                                    v[j * 8 + e * 2 + 1] = mul_rn((float)__builtin_bit_cast(_Float16, (unsigned short)(pair >> 16)), sc);
                                }
                        }
#pragma unroll
                        for (int e = 0; e < 16; e += 4) float2int8_as_float_x4(v[e], v[e + 1], v[e + 2], v[e + 3]);
                        v4i w;
                        uint32_t r0, r1, r2, r3;
                        pack16_quantised(v, r0, r1, r2, r3);
                        // the border is zero bytes whatever the scale (the reference pads after it quantises)
                        const bool real = (inside >> (u * LAR + i)) & 1u;
                        w[0] = real ? (int)r0 : 0;
                        w[1] = real ? (int)r1 : 0;
                        w[2] = real ? (int)r2 : 0;
                        w[3] = real ? (int)r3 : 0;
                        const unsigned dst = a_tile_lds + (unsigned)((s0 + u) * (BM * 64) + i * 4096 + wave * 1024 + lane * 16);
                        asm volatile("ds_write_b128 %0, %1" ::"v"(dst), "v"(w) : "memory");
                    }
                }
            }
        }
        // every wavefront's bytes, and the weights it asked for, are in place before anybody multiplies
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    }

    for (int t = 0; t < nk; t++)
    {
        if constexpr (!STAGED)
        {
            // this wavefront's loads of step t have landed (later stages may stay in flight) ...
            const int ahead = nk - 1 - t < STAGES - 2 ? nk - 1 - t : STAGES - 2;
            switch (ahead)
            {
            case 0: WAIT_VMCNT(0); break;
            case 1: WAIT_VMCNT(1 * (LA + LB)); break;
            case 2: WAIT_VMCNT(2 * (LA + LB)); break;
            case 3: WAIT_VMCNT(3 * (LA + LB)); break;
            case 4: WAIT_VMCNT(4 * (LA + LB)); break;
            default: WAIT_VMCNT(5 * (LA + LB)); break; // STAGES <= 7
            }
            // ... and everybody's: the barrier also says nobody still reads the stage refilled next
            __builtin_amdgcn_s_barrier();
        }
        // (quantising loader: step t's weights at their own place, see issue())
        const unsigned st = STAGED ? a_tile_lds + (unsigned)(tile_steps * (BM * 64) + t * (BN * 64) - BM * 64) : lds_base + (unsigned)((t % STAGES) * STAGE_BYTES);
        // fragment reads of both K halves go out first; the address arithmetic and the global loads of the stage
        // refilled next are issued while they are in flight
        v4i fa[2][TM], fb[2][TN];
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
        {
            const unsigned chunk = ks ? ch1 : ch0;
#pragma unroll
            for (int a = 0; a < TM; a++)
                asm volatile("ds_read_b128 %0, %1" : "=v"(fa[ks][a]) : "v"((STAGED ? a_tile_lds + (unsigned)(t * (BM * 64)) : st) + rd_a + chunk + (unsigned)(a * 32 * 64)));
#pragma unroll
            for (int c = 0; c < TN; c++) asm volatile("ds_read_b128 %0, %1" : "=v"(fb[ks][c]) : "v"(st + rd_b + chunk + (unsigned)(c * 32 * 64)));
        }
        if (!STAGED && t + STAGES - 1 < nk) issue(t + STAGES - 1);
        // the reads are asm, so the wait is too; passing each fragment through an (empty) volatile asm after it
        // keeps the MFMAs, which consume those values, below the wait
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
        {
#pragma unroll
            for (int a = 0; a < TM; a++) asm volatile("" : "+v"(fa[ks][a]));
#pragma unroll
            for (int c = 0; c < TN; c++) asm volatile("" : "+v"(fb[ks][c]));
        }
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int c = 0; c < TN; c++) acc[a][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks][a], fb[ks][c], acc[a][c], 0, 0, 0);
    }

    // ---- epilogue: lane = one output channel per 32-column block, registers = pixels
    if (SPLITK)
    {
        // Slice of this workgroup: [register][thread] int32.  The dump and its read-back are agent-scope atomic
        // stores / loads: they go to the coherence point of the whole device (the XCDs' L2s are not coherent with each
        // other inside a kernel) without the full L2 write-back and invalidate a fence would cost every workgroup.
        constexpr int NREG = TM * TN * 16;
        const int tile_id = tm * tiles_n + tn;
        __shared__ unsigned arrived;
        int* mine = partial + ((size_t)split * tiles_m * tiles_n + tile_id) * (size_t)(NREG * 256);
        // optimistic dump: the last workgroup would not need it, but it does not know yet that it is the last
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
            for (int c = 0; c < TN; c++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    __hip_atomic_store(mine + ((a * TN + c) * 16 + r) * 256 + threadIdx.x, acc[a][c][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        WAIT_VMCNT(0); // this wavefront's stores have reached the coherence point ...
        asm volatile("" ::: "memory");
        __syncthreads(); // ... and everybody else's in the workgroup, before the counter moves
        if (threadIdx.x == 0) arrived = atomicAdd(counters + tile_id, 1u);
        __syncthreads();
        if (arrived != (unsigned)(splits - 1)) return; // somebody else finishes this tile
        for (int s2 = 0; s2 < splits; s2++)
        {
            if (s2 == split) continue;
            const int* theirs = partial + ((size_t)s2 * tiles_m * tiles_n + tile_id) * (size_t)(NREG * 256);
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int c = 0; c < TN; c++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        acc[a][c][r] += __hip_atomic_load(theirs + ((a * TN + c) * 16 + r) * 256 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (threadIdx.x == 0) counters[tile_id] = 0u; // ready for the next launch
    }
    // Through LDS, so that global memory sees whole runs of channels: each wavefront stages 32 pixels x CW channels of
    // results as [pixel][channel] floats (the pipeline stages are free by now), then every lane takes 4 consecutive
    // channels of one pixel: a 16-byte residual load, a 16-byte fp32 store and a 4-byte int8 store, the wavefront
    // covering 64/(CW/4) pixel rows of CW contiguous channels per instruction.
    constexpr int CW = BN / 2;      // channels per wavefront
    constexpr int LD = CW + 4;      // row pitch in floats
    constexpr int G = CW / 4;       // 4-channel groups per row
    __syncthreads();                // nobody reads the operand stages any more
    float* tile = reinterpret_cast<float*>(smem) + wave * (32 * LD);
    const bool to_int8 = epi.scale_out != 0;

    float s_in[TN], bias[TN], s_out[TN];
    bool real[TN];
#pragma unroll
    for (int c = 0; c < TN; c++)
    {
        const int ch = col0 + wn * CW + c * 32 + l32;
        real[c] = ch < g.cout; // channels from cout up to out_cp are the blob's zero padding
        if (GEMM)
        {
            // s_in: 1/sB_j (one scale per column) ; bias: beta*C_j (C broadcast per column)
            s_in[c] = (real[c] && gemm.per_col) ? div_rn(1.f, gemm.b_scales[ch]) : 0.f;
            bias[c] = (real[c] && gemm.bt == 4) ? mul_rn(gemm.c[ch], gemm.beta) : 0.f;
            s_out[c] = 0.f;
        }
        else
        {
            s_in[c] = real[c] ? raw_s_in[c] : 0.f;
            // no bias: -0, the one value whose addition changes nothing (x + -0 = x for every x, -0 included)
            bias[c] = (real[c] && epi.bias) ? raw_bias[c] : -0.f;
            s_out[c] = (real[c] && to_int8) ? raw_s_out[c] : 0.f;
        }
    }
    if (GEMM)
    {
        const float sb0 = gemm.b_scales[0];
        const float c0 = gemm.bt == 0 ? mul_rn(gemm.c[0], gemm.beta) : 0.f;
#pragma unroll
        for (int a = 0; a < TM; a++)
        {
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int pl = 8 * (r >> 2) + 4 * lhi + (r & 3);
                int row = row0 + wm * (BM / 2) + a * 32 + pl;
                if (row >= g.npix) row = g.npix - 1; // rows beyond M are staged but never stored
                const float sa = gemm.a_scales[row];
                const float rowscale = gemm.per_col ? div_rn(1.f, sa) : div_rn(1.f, mul_rn(sa, sb0));
                const float crow = (gemm.bt == 1 || gemm.bt == 2) ? mul_rn(gemm.c[row], gemm.beta) : 0.f;
#pragma unroll
                for (int c = 0; c < TN; c++)
                {
                    float f = mul_rn((float)acc[a][c][r], rowscale);
                    if (gemm.per_col) f = mul_rn(f, s_in[c]);
                    if (gemm.bt == 4)
                        f = add_rn(f, bias[c]);
                    else if (gemm.bt == 0)
                        f = add_rn(f, c0);
                    else if (gemm.bt >= 0)
                        f = add_rn(f, crow);
                    f = mul_rn(f, gemm.alpha);
                    tile[pl * LD + c * 32 + l32] = f;
                }
            }
            __syncthreads();
#pragma unroll
            for (int it = 0; it < G / 2; it++)
            {
                const int idx = it * 64 + lane;
                const int p = idx / G, j = idx - p * G;
                const v4f v = *reinterpret_cast<const v4f*>(tile + p * LD + 4 * j);
                const int pix = row0 + wm * (BM / 2) + a * 32 + p;
                const int ch4 = col0 + wn * CW + 4 * j;
                if (pix < g.npix && ch4 < col_limit) *reinterpret_cast<v4f*>(static_cast<float*>(epi.out) + (size_t)pix * out_cp + ch4) = v;
            }
            if (a + 1 < TM) __syncthreads();
        }
        return;
    }

    // the activation type is uniform: branch on it once, outside the unrolled loops
    auto finish = [&](auto act_tag) {
        constexpr int ACT = decltype(act_tag)::value;
        float q_lo[TN], q_hi[TN]; // ACT 103 to int8: the clip's bounds in the output scale, inside [-127, 127]
#pragma unroll
        for (int c = 0; c < TN; c++)
        {
            q_lo[c] = __builtin_amdgcn_fmed3f(mul_rn(epi.act.p0, s_out[c]), -127.f, 127.f);
            q_hi[c] = __builtin_amdgcn_fmed3f(mul_rn(epi.act.p1, s_out[c]), -127.f, 127.f);
        }
#pragma unroll
        for (int a = 0; a < TM; a++)
        {
            // The residual this lane will add in the read-out below is requested now, so that it arrives while the
            // accumulators are being converted (clamped addresses, nothing selected: see the tables above).
            v4f resv[G / 2];
            const bool with_residual = !to_int8 && fusion.residual != 0;
            if (with_residual)
            {
#pragma unroll
                for (int it = 0; it < G / 2; it++)
                {
                    const int idx = it * 64 + lane;
                    const int p = idx / G, j = idx - p * G;
                    int pix = row0 + wm * (BM / 2) + a * 32 + p;
                    int ch4 = col0 + wn * CW + 4 * j;
                    if (pix >= g.npix) pix = g.npix - 1;
                    if (ch4 >= col_limit) ch4 = col_limit - 4;
                    resv[it] = *reinterpret_cast<const v4f*>(fusion.residual + (size_t)pix * out_cp + ch4);
                }
            }
#pragma unroll
            for (int c = 0; c < TN; c++)
            {
                if (col0 + wn * CW + c * 32 >= col_limit) continue; // a whole 32-channel block of tile padding (uniform per wavefront)
                float fr[16];
#pragma unroll
                for (int r = 0; r < 16; r++)
                {
                    float f = add_rn(mul_rn((float)acc[a][c][r], s_in[c]), bias[c]);
                    if (ACT == 1)
                        f = fmaxf(f, 0.f);
                    else if (ACT == 3)
                    {
                        if (f < epi.act.p0) f = epi.act.p0;
                        if (f > epi.act.p1) f = epi.act.p1;
                    }
                    else if (ACT == 103)
                    {
                        if (!to_int8) f = clip_not_nan(f, epi.act.p0, epi.act.p1); // (to int8: folded into the clamp below)
                    }
                    else if (ACT != 0)
                        f = apply_activation(f, epi.act);
                    fr[r] = to_int8 ? mul_rn(f, s_out[c]) : f;
                }
                if (to_int8)
                {
#pragma unroll
                    for (int r = 0; r < 16; r += 4)
                    {
                        if (ACT == 103)
                            float2int8_as_float_bounded_x4(fr[r], fr[r + 1], fr[r + 2], fr[r + 3], q_lo[c], q_hi[c]);
                        else
                            float2int8_as_float_x4(fr[r], fr[r + 1], fr[r + 2], fr[r + 3]);
                    }
                }
                // Pad channels carry zero scales and no bias: with no activation or ReLU they are zero already, and
                // behind the bounded clip a pad's (finite) value times its zero output scale rounds to zero too.
                const bool clear_pads = ACT != 0 && ACT != 1 && !(ACT == 103 && to_int8);
#pragma unroll
                for (int r = 0; r < 16; r++)
                {
                    if (clear_pads && !real[c]) fr[r] = 0.f;
                    tile[(8 * (r >> 2) + 4 * lhi + (r & 3)) * LD + c * 32 + l32] = fr[r];
                }
            }
            __syncthreads();
            if (to_int8)
            {
                // 16 channels of one pixel per lane: four LDS reads, one 16-byte store
                constexpr int G16 = CW / 16;
                constexpr int ITS = G16 / 2 > 0 ? G16 / 2 : 1;
#pragma unroll
                for (int it = 0; it < ITS; it++)
                {
                    const int idx = it * 64 + lane;
                    const int p = idx / G16, j = idx - p * G16;
                    const int pix = row0 + wm * (BM / 2) + a * 32 + p;
                    const int ch16 = col0 + wn * CW + 16 * j;
                    if (p < 32 && pix < g.npix && ch16 < col_limit)
                    {
                        float q[16];
#pragma unroll
                        for (int w4 = 0; w4 < 4; w4++)
                        {
                            const v4f t = *reinterpret_cast<const v4f*>(tile + p * LD + 16 * j + 4 * w4);
                            q[4 * w4] = t[0], q[4 * w4 + 1] = t[1], q[4 * w4 + 2] = t[2], q[4 * w4 + 3] = t[3];
                        }
                        uint32_t p0, p1, p2, p3;
                        pack16_quantised(q, p0, p1, p2, p3);
                        const v4i pk = {(int)p0, (int)p1, (int)p2, (int)p3};
                        *reinterpret_cast<v4i*>(static_cast<int8_t*>(epi.out) + (size_t)pix * out_cp + ch16) = pk;
                    }
                }
            }
            else
            {
#pragma unroll
            for (int it = 0; it < G / 2; it++)
            {
                const int idx = it * 64 + lane;
                const int p = idx / G, j = idx - p * G;
                v4f v = *reinterpret_cast<const v4f*>(tile + p * LD + 4 * j);
                const int pix = row0 + wm * (BM / 2) + a * 32 + p;
                const int ch4 = col0 + wn * CW + 4 * j;
                if (pix < g.npix && ch4 < col_limit)
                {
                    const size_t o = (size_t)pix * out_cp + ch4;
                    {
                        if (with_residual)
                        {
#pragma unroll
                            for (int e = 0; e < 4; e++) v[e] = add_rn(v[e], resv[it][e]);
                        }
                        if (fusion.relu_after)
                        {
#pragma unroll
                            for (int e = 0; e < 4; e++) v[e] = v[e] < 0.f ? 0.f : v[e]; // the ReLU LAYER's statement (src/layer/relu.cpp:36-37): a NaN stays, unlike fmaxf
                        }
                        *reinterpret_cast<v4f*>(static_cast<float*>(epi.out) + o) = v;
                        if (fusion.q8_out)
                        {
                            v4f q;
#pragma unroll
                            for (int e = 0; e < 4; e++) q[e] = mul_rn(v[e], fusion.q8_scale);
                            float q0 = q[0], q1 = q[1], q2 = q[2], q3 = q[3];
                            float2int8_as_float_x4(q0, q1, q2, q3);
                            *reinterpret_cast<uint32_t*>(fusion.q8_out + o) = pack4(v4f{q0, q1, q2, q3});
                        }
                    }
                }
            }
            }
            if (a + 1 < TM) __syncthreads();
        }
    };
    if (epi.act.type == 0)
        finish(std::integral_constant<int, 0>{});
    else if (epi.act.type == 1)
        finish(std::integral_constant<int, 1>{});
    else if (epi.act.type == 3)
    {
        // Tame tables: every accumulator comes out of scale and bias finite (|acc| <= 2^31, so 2^90 and 2^120 leave
        // room), so the clip is max-then-min; the clipped value times the output scale stays below 2^31, so float2int8
        // needs no out-of-range branch; and the clip folds into the requantising clamp.
        const float clip_abs = fmaxf(fabsf(epi.act.p0), fabsf(epi.act.p1));
        bool tame = fabsf(epi.act.p0) < INFINITY && fabsf(epi.act.p1) < INFINITY;
#pragma unroll
        for (int c = 0; c < TN; c++)
            tame = tame && fabsf(s_in[c]) < 0x1p90f && fabsf(bias[c]) < 0x1p120f && mul_rn(clip_abs, fabsf(s_out[c])) < 2147483648.f
                   && clip_folds_into_requantise(epi.act.p0, epi.act.p1, s_out[c]);
        if (__all(tame))
            finish(std::integral_constant<int, 103>{});
        else
            finish(std::integral_constant<int, 3>{});
    }
    else
        finish(std::integral_constant<int, -1>{});
}

struct PipePlan
{
    int bm, bn, tiles_m, tiles_n, splits, steps_per_split;
};

// tile shape and K split for a problem of cout channels, npix pixels and `steps` 64-byte K steps
PipePlan plan_pipelined(int cout, long long npix, int steps);

// multiplier that turns b / tiles_n into a high multiply, exact for b * tiles_n < 2^32 (tiles_n == 1 is special-cased)
static inline unsigned tile_magic(int tiles_n)
{
    return tiles_n > 1 ? (unsigned)((1ull << 32) / (unsigned)tiles_n + 1) : 0u;
}

// The launches of conv_nhwc_pipelined_split.hip.  launch_pipe_split: the convolution kernel with K split over workgroups
// (modes 0, 1 and 3; the grid, the partial sums and the counters come from the caller's plan).
int launch_pipe_split(const PipePlan& p, int mode, const int8_t* wpk, const int8_t* x, const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion,
                      int out_cp, int col_limit, int32_t* partial, unsigned* counters, hipStream_t stream);

} // namespace ncnnhip

#endif // NCNNHIP_CONV_NHWC_PIPELINED_KERNEL_H
