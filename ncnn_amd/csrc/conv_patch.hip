// int8 Convolution (group 1, zero border) on channels-last blobs for layers with FEW output pixels, where the
// 64-pixel tiles of the pipelined kernel leave most of the chip idle and a layer is the sum of its latencies.
//
// One workgroup (4 wavefronts) owns a two-dimensional tile of 32 output pixels (32x1, 16x2, 8x4, ... whichever covers
// the output plane with the fewest tiles) and 64 output channels.  A 2-D tile keeps the halo small: 8x4 outputs of a
// 3x3 layer read 10x6 input pixels, where 32 consecutive outputs of a 56-wide image read a run of 146.
//   1. The input patch -- patch rows x patch columns x Cp channels -- is requested first, 16 bytes per lane and load (it is
//      what the workgroup waits for: load, quantise, LDS, barrier), then every lane requests its share of the weights
//      straight into registers (a lane's B operand of v_mfma_i32_32x32x32_i8 is 16 consecutive K bytes of one channel
//      row: no staging, nothing shared).
//   2. The patch is quantised on the way when the blob is still fp32 / fp16 (Quantize::forward,
//      src/layer/quantize.cpp:48-111, one scale) and written to LDS as [row][column][Cp] int8 with ZEROS wherever it
//      leaves the image: the convolution's border (src/layer/convolution.cpp:383-508 pads after it quantises, with zero bytes).
//   3. The K loop touches LDS and registers only and has no bounds tests (its LDS reads all go out before the first
//      product): the A operand of output pixel (ty, tx) and tap (ky, kx) is 16 bytes at ((ty*sh + ky*dh) * patch columns + tx*sw + kx*dw) * Cp + channel -- a per-lane base plus a
//      wavefront-uniform offset.  The four wavefronts are 2 channel halves x 2 K halves (even / odd 32-byte steps).
//   4. The two K halves exchange half of their accumulators through LDS (integer addition: exact in any order), so each
//      wavefront finishes 16 pixels x 32 channels; results go through LDS once more so that global memory sees whole
//      runs of channels, as in the pipelined kernel, with the same epilogue arithmetic and the same fused tail.
// Weights are the pipelined kernel's: [cout][K], K = (tap, channel) rounded up to 64 bytes.
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "conv_nhwc.h"
#include "mfma_tile.h"

namespace ncnnhip {

typedef float v4f __attribute__((ext_vector_type(4)));

struct PatchPlan
{
    int twl;                       // tile = (1 << twl) x (32 >> twl) output pixels
    int tiles_x, tiles_y, tiles_n; // tiles across, down, and 64-channel tiles
    int pr, pc;                    // patch rows / columns in input pixels
    int nsteps;                    // 32-byte K steps that carry taps: ntaps * tapK / 32
    int batch;
};

// AIN: bytes per activation value (1: the blob is int8; 4 / 2: fp32 / fp16, quantised here).  MAXS: 32-byte K steps a
// wavefront can hold the weights of (its registers: 4 per step).
template<int AIN, int MAXS>
__global__ __launch_bounds__(256) void conv_patch_kernel(const int8_t* __restrict__ wpk, const int8_t* __restrict__ x, NhwcGeom g, ConvEpilogue epi, ConvFusion fusion,
                                                         int out_cp, PatchPlan pl, const float* __restrict__ a_scale)
{
    extern __shared__ __attribute__((aligned(16))) int8_t patch[];
    __shared__ int red[4][8][64];
    constexpr int LD = 68; // row pitch of the result staging in floats
    __shared__ __attribute__((aligned(16))) float stage[32 * LD];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 1, wk = wave >> 1;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int twl = pl.twl, tw_mask = (1 << twl) - 1;

    // Workgroup ids are dealt round-robin to the 8 XCDs; they are remapped so that an XCD works on consecutive tiles
    // (channel tiles of one pixel tile, then the tiles of one row of tiles, then the rows): neighbours share their
    // patches' borders in that XCD's L2.
    int b = blockIdx.x;
    {
        const int T = gridDim.x, xcd = b & 7, idx = b >> 3, rem = T & 7;
        b = xcd * (T >> 3) + (xcd < rem ? xcd : rem) + idx;
    }
    b = __builtin_amdgcn_readfirstlane(b);
    int tn = 0, txi, tyi, img;
    {
        int t = b;
        if (pl.tiles_n > 1)
        {
            const int q = t / pl.tiles_n;
            tn = t - q * pl.tiles_n;
            t = q;
        }
        const int row = t / pl.tiles_x;
        txi = t - row * pl.tiles_x;
        img = row / pl.tiles_y;
        tyi = row - img * pl.tiles_y;
    }
    const int col0 = tn * 64;
    const int oy0 = tyi * (32 >> twl), ox0 = txi << twl;
    const int iy0 = oy0 * g.sh - g.pad_top, ix0 = ox0 * g.sw - g.pad_left;

    // ---- 1. the input patch, 16 bytes of the blob per lane and load: the first round of requests goes out before anything
    // else (the patch is what the workgroup waits for first: load, quantise, LDS, barrier); the weights follow
    constexpr int VPI = 16 / AIN;          // values per load
    constexpr int INFL = 8;                // loads in flight per lane
    const int ipp = g.Cp / VPI;            // loads per pixel
    const int rowitems = pl.pc * ipp;      // per patch row
    const int nitems = pl.pr * rowitems;
    const int8_t* img_base = x + (size_t)img * g.H * g.W * g.Cp * AIN;
    auto patch_request = [&](int base, v4i (&raw)[INFL], unsigned& inside) {
        inside = 0;
#pragma unroll
        for (int j = 0; j < INFL; j++)
        {
            if (base + j * 256 >= nitems) break; // (uniform) nobody has a j-th item
            int qi = base + j * 256 + (int)threadIdx.x;
            if (qi >= nitems) qi = nitems - 1;
            const int row = small_div(qi, rowitems);
            const int rem = qi - row * rowitems;
            const int col = small_div(rem, ipp);
            const int c = rem - col * ipp;
            const int iy = iy0 + row, ix = ix0 + col;
            const bool in = (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
            const size_t off = in ? ((size_t)(iy * g.W + ix) * g.Cp + c * VPI) * AIN : 0;
            raw[j] = *reinterpret_cast<const v4i*>(img_base + off);
            inside |= in ? 1u << j : 0u;
        }
    };
    auto patch_store = [&](int base, const v4i (&raw)[INFL], unsigned inside, float sc) {
#pragma unroll
        for (int j = 0; j < INFL; j++)
        {
            if (base + j * 256 >= nitems) break;
            const int qi = base + j * 256 + (int)threadIdx.x;
            const bool in = (inside >> j) & 1u;
            if constexpr (AIN == 1)
            {
                const v4i w = in ? raw[j] : v4i{0, 0, 0, 0};
                if (qi < nitems) *reinterpret_cast<v4i*>(patch + (size_t)qi * 16) = w;
            }
            else if constexpr (AIN == 4)
            {
                float v0 = mul_rn(__int_as_float(raw[j][0]), sc), v1 = mul_rn(__int_as_float(raw[j][1]), sc);
                float v2 = mul_rn(__int_as_float(raw[j][2]), sc), v3 = mul_rn(__int_as_float(raw[j][3]), sc);
                float2int8_as_float_x4(v0, v1, v2, v3);
                const uint32_t word = pack4_quantised(v0, v1, v2, v3);
                if (qi < nitems) *reinterpret_cast<uint32_t*>(patch + (size_t)qi * 4) = in ? word : 0u;
            }
            else
            {
                float v[8];
#pragma unroll
                for (int e = 0; e < 4; e++)
                {
                    const unsigned pair = (unsigned)raw[j][e]; // two halves, the first in the low 16 bits
                    v[2 * e] = mul_rn((float)__builtin_bit_cast(_Float16, (unsigned short)(pair & 0xffffu)), sc);
                    v[2 * e + 1] = mul_rn((float)__builtin_bit_cast(_Float16, (unsigned short)(pair >> 16)), sc);
                }
                float2int8_as_float_x4(v[0], v[1], v[2], v[3]);
                float2int8_as_float_x4(v[4], v[5], v[6], v[7]);
                typedef unsigned v2u __attribute__((ext_vector_type(2)));
                v2u w = {pack4_quantised(v[0], v[1], v[2], v[3]), pack4_quantised(v[4], v[5], v[6], v[7])};
                if (!in) w = v2u{0u, 0u};
                if (qi < nitems) *reinterpret_cast<v2u*>(patch + (size_t)qi * 8) = w;
            }
        }
    };
    v4i raw0[INFL];
    unsigned inside0;
    patch_request(0, raw0, inside0);
    float sc = 0.f;
    if constexpr (AIN != 1) sc = a_scale[0];

    // ---- 2. this lane's weights: channel row col0 + wn*32 + l32, K bytes (2i + wk)*32 + lhi*16 .. +16 for its i-th step
    const int ch = col0 + wn * 32 + l32;
    const int chc = ch < g.cout ? ch : g.cout - 1; // a valid row; its products land in columns nobody stores
    const int my_steps = (pl.nsteps - wk + 1) >> 1;
    v4i bw[MAXS];
    {
        const int8_t* bsrc = wpk + (size_t)chc * g.K + wk * 32 + lhi * 16;
#pragma unroll
        for (int i = 0; i < MAXS; i++)
            if (i < my_steps) bw[i] = *reinterpret_cast<const v4i*>(bsrc + i * 64);
    }
    // the epilogue's per-channel tables, requested now so that they arrive under everything else (bare loads from
    // always-valid addresses; nothing is selected until the values are used)
    const float raw_s_in = epi.scale_in[chc];
    const float raw_bias = (epi.bias ? epi.bias : epi.scale_in)[chc];
    const float raw_s_out = (epi.scale_out ? epi.scale_out : epi.scale_in)[chc];

    // ---- the patch -> LDS (quantised on the way when the blob is fp32 / fp16); further rounds for a patch of more than 2048 loads
    patch_store(0, raw0, inside0, sc);
    for (int base = 256 * INFL; base < nitems; base += 256 * INFL)
    {
        v4i raw[INFL];
        unsigned inside;
        patch_request(base, raw, inside);
        patch_store(base, raw, inside, sc);
    }
    __syncthreads();

    // ---- 3. the K loop: LDS and registers only
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    {
        const int tx = l32 & tw_mask, ty = l32 >> twl;
        const int8_t* a_lane = patch + ((ty * g.sh) * pl.pc + tx * g.sw) * g.Cp + lhi * 16;
        // position of this wavefront's step in K: offset q inside tap (ky, kx); wavefront-uniform
        int q = wk * 32, kx = 0, ky = 0;
        while (q >= g.tapK)
        {
            q -= g.tapK;
            if (++kx == g.kw)
            {
                kx = 0;
                ky++;
            }
        }
        // every A operand is requested before the first product (a step beyond this wavefront's share reads the first one again)
        v4i fa[MAXS];
#pragma unroll
        for (int i = 0; i < MAXS; i++)
        {
            const int off = i < my_steps ? ((ky * g.dh) * pl.pc + kx * g.dw) * g.Cp + q : 0;
            fa[i] = *reinterpret_cast<const v4i*>(a_lane + off);
            q += 64;
            while (q >= g.tapK)
            {
                q -= g.tapK;
                if (++kx == g.kw)
                {
                    kx = 0;
                    ky++;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MAXS; i++)
            if (i < my_steps) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], bw[i], acc, 0, 0, 0);
    }

    // ---- 4. epilogue
    const bool to_int8 = epi.scale_out != 0;
    const bool with_residual = !to_int8 && fusion.residual != 0;
    // read-out items of the fp32 form: 4 consecutive channels of one pixel, two per lane; the residual they will add is
    // requested now (clamped addresses, nothing selected)
    v4f resv[2];
    if (with_residual)
    {
#pragma unroll
        for (int it = 0; it < 2; it++)
        {
            const int idx = it * 256 + (int)threadIdx.x;
            const int p = idx >> 4, j = idx & 15;
            int oy = oy0 + (p >> twl), ox = ox0 + (p & tw_mask);
            if (oy >= g.outh) oy = g.outh - 1;
            if (ox >= g.outw) ox = g.outw - 1;
            int ch4 = col0 + 4 * j;
            if (ch4 >= out_cp) ch4 = out_cp - 4;
            resv[it] = *reinterpret_cast<const v4f*>(fusion.residual + ((size_t)(img * g.outh + oy) * g.outw + ox) * out_cp + ch4);
        }
    }

    // accumulator register r of lane (l32, lhi) is pixel 8*(r/4) + 4*lhi + r%4 of the tile: registers 0-7 are pixels
    // 0-15, registers 8-15 pixels 16-31.  K half 0 finishes the first sixteen pixels, K half 1 the others.
    int mine[8];
#pragma unroll
    for (int r = 0; r < 8; r++)
    {
        mine[r] = wk ? acc[8 + r] : acc[r];
        red[wave][r][lane] = wk ? acc[r] : acc[8 + r];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; r++) mine[r] += red[wave ^ 2][r][lane];

    const bool real = ch < g.cout; // channels from cout up to out_cp are the blob's zero padding
    const float s_in = real ? raw_s_in : 0.f;
    // no bias: -0, the one value whose addition changes nothing (x + -0 = x for every x, -0 included)
    const float bias = (real && epi.bias) ? raw_bias : -0.f;
    const float s_out = (real && to_int8) ? raw_s_out : 0.f;

    auto convert = [&](auto act_tag) {
        constexpr int ACT = decltype(act_tag)::value;
        float fr[8];
#pragma unroll
        for (int r = 0; r < 8; r++)
        {
            float f = add_rn(mul_rn((float)mine[r], s_in), bias);
            if (ACT == 1)
                f = fmaxf(f, 0.f);
            else if (ACT == 3)
            {
                if (f < epi.act.p0) f = epi.act.p0;
                if (f > epi.act.p1) f = epi.act.p1;
            }
            else if (ACT != 0)
                f = apply_activation(f, epi.act);
            fr[r] = to_int8 ? mul_rn(f, s_out) : f;
        }
        if (to_int8)
        {
            float2int8_as_float_x4(fr[0], fr[1], fr[2], fr[3]);
            float2int8_as_float_x4(fr[4], fr[5], fr[6], fr[7]);
        }
        // pad channels carry zero scales and no bias: with no activation or ReLU they are zero already
        const bool clear_pads = ACT != 0 && ACT != 1;
#pragma unroll
        for (int r = 0; r < 8; r++)
        {
            if (clear_pads && !real) fr[r] = 0.f;
            stage[(16 * wk + 8 * (r >> 2) + 4 * lhi + (r & 3)) * LD + wn * 32 + l32] = fr[r];
        }
    };
    if (epi.act.type == 0)
        convert(std::integral_constant<int, 0>{});
    else if (epi.act.type == 1)
        convert(std::integral_constant<int, 1>{});
    else if (epi.act.type == 3)
        convert(std::integral_constant<int, 3>{});
    else
        convert(std::integral_constant<int, -1>{});
    __syncthreads();

    if (to_int8)
    {
        // 16 channels of one pixel per lane: four LDS reads, one 16-byte store
        if (threadIdx.x < 128)
        {
            const int p = (int)threadIdx.x >> 2, j = (int)threadIdx.x & 3;
            const int oy = oy0 + (p >> twl), ox = ox0 + (p & tw_mask);
            const int ch16 = col0 + 16 * j;
            if (oy < g.outh && ox < g.outw && ch16 < out_cp)
            {
                float qv[16];
#pragma unroll
                for (int w4 = 0; w4 < 4; w4++)
                {
                    const v4f t = *reinterpret_cast<const v4f*>(stage + p * LD + 16 * j + 4 * w4);
                    qv[4 * w4] = t[0], qv[4 * w4 + 1] = t[1], qv[4 * w4 + 2] = t[2], qv[4 * w4 + 3] = t[3];
                }
                uint32_t p0, p1, p2, p3;
                pack16_quantised(qv, p0, p1, p2, p3);
                const v4i pk = {(int)p0, (int)p1, (int)p2, (int)p3};
                *reinterpret_cast<v4i*>(static_cast<int8_t*>(epi.out) + ((size_t)(img * g.outh + oy) * g.outw + ox) * out_cp + ch16) = pk;
            }
        }
        return;
    }
#pragma unroll
    for (int it = 0; it < 2; it++)
    {
        const int idx = it * 256 + (int)threadIdx.x;
        const int p = idx >> 4, j = idx & 15;
        const int oy = oy0 + (p >> twl), ox = ox0 + (p & tw_mask);
        const int ch4 = col0 + 4 * j;
        if (oy < g.outh && ox < g.outw && ch4 < out_cp)
        {
            v4f v = *reinterpret_cast<const v4f*>(stage + p * LD + 4 * j);
            const size_t o = ((size_t)(img * g.outh + oy) * g.outw + ox) * out_cp + ch4;
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
                float q0 = mul_rn(v[0], fusion.q8_scale), q1 = mul_rn(v[1], fusion.q8_scale), q2 = mul_rn(v[2], fusion.q8_scale), q3 = mul_rn(v[3], fusion.q8_scale);
                float2int8_as_float_x4(q0, q1, q2, q3);
                *reinterpret_cast<uint32_t*>(fusion.q8_out + o) = pack4_quantised(q0, q1, q2, q3);
            }
        }
    }
}

static const size_t PATCH_LDS_LIMIT = 64u << 10; // bytes of LDS for the input patch
static const int PATCH_MAX_STEPS = 36;           // 32-byte K steps per wavefront (K up to 2304 bytes of taps)

static bool patch_plan(const NhwcGeom& g, int batch, PatchPlan& pl)
{
    if (g.pad_word != 0 || g.tapK != g.Cp || g.tapK % 32 != 0 || g.ntaps != g.kw * g.kh || batch < 1) return false;
    pl.nsteps = g.ntaps * (g.tapK / 32);
    if ((pl.nsteps + 1) / 2 > PATCH_MAX_STEPS) return false;
    long long best_tiles = -1, best_patch = 0;
    for (int twl = 5; twl >= 0; twl--)
    {
        const int tw = 1 << twl, th = 32 >> twl;
        const long long tiles = (long long)ceil_div(g.outw, tw) * ceil_div(g.outh, th);
        const long long pr = (long long)(th - 1) * g.sh + (long long)(g.kh - 1) * g.dh + 1, pc = (long long)(tw - 1) * g.sw + (long long)(g.kw - 1) * g.dw + 1;
        const long long patch = pr * pc;
        if (patch * g.Cp > (long long)PATCH_LDS_LIMIT) continue;
        if (best_tiles < 0 || tiles < best_tiles || (tiles == best_tiles && patch < best_patch))
        {
            best_tiles = tiles;
            best_patch = patch;
            pl.twl = twl;
            pl.pr = (int)pr;
            pl.pc = (int)pc;
        }
    }
    if (best_tiles < 0) return false;
    pl.tiles_x = ceil_div(g.outw, 1 << pl.twl);
    pl.tiles_y = ceil_div(g.outh, 32 >> pl.twl);
    pl.tiles_n = ceil_div(g.cout, 64);
    pl.batch = batch;
    return (long long)pl.tiles_x * pl.tiles_y * pl.tiles_n * batch < (1ll << 31);
}

bool conv_patch_supported(const NhwcGeom& g, int batch)
{
    PatchPlan pl;
    return patch_plan(g, batch, pl);
}

bool conv_patch_pays(const NhwcGeom& g, int batch, int x_elemsize)
{
    PatchPlan pl;
    if (!patch_plan(g, batch, pl)) return false;
    const char* e = getenv("NCNNHIP_PATCH"); // 0: never, 1: whenever the layer fits (tests walk shapes the rule below would not send here)
    if (e && e[0] == '0') return false;
    if (e && e[0] == '1') return true;
    // Measured on ResNet-50's layers at batch 1 against the pipelined kernel (which splits K over workgroups there): ahead
    // where 64-pixel tiles would cover less than half the chip and K is short -- from an fp32 blob 3x3 64 -> 64 on 56 x 56
    // 8.5 -> 6.3 us; from an int8 blob the same layer 6.0 -> 5.4, 3x3 128 -> 128 on 28 x 28 7.2 -> 6.9 -- and behind with
    // longer K (3x3 256 -> 256 on 14 x 14 8.4 -> 11.7: 36 dependent steps per wavefront) and on int8 1x1 layers (nothing
    // to share, 4.5 -> 5.7).
    const long long tiles64 = (long long)ceil_div(g.npix, 64) * ceil_div(g.cout, 64);
    return tiles64 < 128 && (pl.nsteps + 1) / 2 <= 18 && (x_elemsize != 1 || g.ntaps > 1);
}

int launch_conv_patch(const NhwcGeom& g, const int8_t* wpk, const void* x, int x_elemsize, const float* x_scale, const ConvEpilogue& epi, const ConvFusion& fusion,
                      int out_cp, hipStream_t stream)
{
    PatchPlan pl;
    NCNNHIP_REQUIRE(x_elemsize == 4 || x_elemsize == 2 || x_elemsize == 1, "convolution: activations of %d bytes per value", x_elemsize);
    NCNNHIP_REQUIRE(x_elemsize == 1 || x_scale, "convolution: the input scale is missing");
    NCNNHIP_REQUIRE(patch_plan(g, epi.batch, pl), "convolution: this layer does not fit the small-tile kernel");
    NCNNHIP_REQUIRE(epi.batch >= 1 && (long long)epi.batch * g.outw * g.outh == (long long)g.npix, "convolution: pixel count and batch disagree");
    const size_t patch_bytes = (size_t)pl.pr * pl.pc * g.Cp;
    dim3 grid((unsigned)((long long)pl.tiles_x * pl.tiles_y * pl.tiles_n * pl.batch)), block(256);
    const int8_t* xb = static_cast<const int8_t*>(x);
    const int per_wave = (pl.nsteps + 1) / 2;
#define LAUNCH_PATCH(AIN_, MAXS_)                                                                                                                            \
    do                                                                                                                                                       \
    {                                                                                                                                                        \
        auto kernel = conv_patch_kernel<AIN_, MAXS_>;                                                                                                        \
        static std::once_flag once;                                                                                                                          \
        static hipError_t attr = hipSuccess;                                                                                                                 \
        std::call_once(once, [&]() { attr = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)PATCH_LDS_LIMIT); });   \
        NCNNHIP_CHECK(attr);                                                                                                                                 \
        hipLaunchKernelGGL(kernel, grid, block, patch_bytes, stream, wpk, xb, g, epi, fusion, out_cp, pl, x_scale);                                          \
    } while (0)
#define LAUNCH_PATCH_IN(MAXS_)          \
    do                                  \
    {                                   \
        if (x_elemsize == 4)            \
            LAUNCH_PATCH(4, MAXS_);     \
        else if (x_elemsize == 2)       \
            LAUNCH_PATCH(2, MAXS_);     \
        else                            \
            LAUNCH_PATCH(1, MAXS_);     \
    } while (0)
    if (per_wave <= 9)
        LAUNCH_PATCH_IN(9);
    else if (per_wave <= 18)
        LAUNCH_PATCH_IN(18);
    else
        LAUNCH_PATCH_IN(36);
#undef LAUNCH_PATCH_IN
#undef LAUNCH_PATCH
    return launch_status("conv_patch_kernel");
}

} // namespace ncnnhip
