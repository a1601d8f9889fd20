// Launches of the pipelined channels-last convolution kernel with K split over workgroups (few output tiles, long K:
// the partial sums meet in a workspace, the last workgroup of a tile to finish runs the epilogue), and the kernel's Gemm
// form.  The kernel itself is in conv_nhwc_pipelined_kernel.h.
#include "conv_nhwc_pipelined_kernel.h"

namespace ncnnhip {

int launch_pipe_split(const PipePlan& p, int mode, const int8_t* wpk, const int8_t* x, const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion,
                      int out_cp, int col_limit, int32_t* partial, unsigned* counters, hipStream_t stream)
{
    NCNNHIP_REQUIRE(p.splits > 1 && partial && counters && (mode == 0 || mode == 1 || mode == 3), "convolution: K split without its workspace");
    dim3 grid((unsigned)((long long)p.tiles_m * p.tiles_n * p.splits)), block(256);
    const GemmTail no_gemm = {0, 0, 0, 0, -1, 1.f, 1.f};
#define LAUNCH_SPLIT_MODE(BM_, BN_, MODE_)                                                                                                              \
    hipLaunchKernelGGL((conv_nhwc_pipelined_kernel<BM_, BN_, PIPE_RING, true, false, MODE_>), grid, block, 0, stream, wpk, x, g, epi, fusion, no_gemm, out_cp, \
                       col_limit, p.tiles_m, p.tiles_n, p.splits, p.steps_per_split, tile_magic(p.tiles_n), partial, counters, (const float*)0, 0)
#define LAUNCH_SPLIT(BM_, BN_)                  \
    do                                          \
    {                                           \
        if (mode == 1)                          \
            LAUNCH_SPLIT_MODE(BM_, BN_, 1);     \
        else if (mode == 3)                     \
            LAUNCH_SPLIT_MODE(BM_, BN_, 3);     \
        else                                    \
            LAUNCH_SPLIT_MODE(BM_, BN_, 0);     \
    } while (0)
    if (p.bm == 128 && p.bn == 256)
        LAUNCH_SPLIT(128, 256);
    else if (p.bm == 128 && p.bn == 128)
        LAUNCH_SPLIT(128, 128);
    else if (p.bm == 128)
        LAUNCH_SPLIT(128, 64);
    else if (p.bn == 256)
        LAUNCH_SPLIT(64, 256);
    else if (p.bn == 128)
        LAUNCH_SPLIT(64, 128);
    else
        LAUNCH_SPLIT(64, 64);
#undef LAUNCH_SPLIT
#undef LAUNCH_SPLIT_MODE
    return launch_status("conv_nhwc_pipelined_kernel (K split)");
}

int launch_gemm_via_conv_pipelined(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K, const GemmTail& tail,
                                   float* out, size_t out_stride, hipStream_t stream, bool* handled)
{
    *handled = false;
    const bool aligned = ((reinterpret_cast<uintptr_t>(aq) | reinterpret_cast<uintptr_t>(bq) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (K % 64 || N % 4 || aq_stride % 16 || bq_stride != (size_t)K || out_stride % 4 || !aligned || tail.bt == 3) return NCNNHIP_OK;
    if ((long long)M * (long long)aq_stride >= (1ll << 31)) return NCNNHIP_OK;
    *handled = true;

    NhwcGeom g;
    g.H = 1;
    g.W = M;
    g.Cp = (int)aq_stride; // one "pixel" per row of A, its channels the K bytes of that row
    g.tapK = g.Cp;
    g.kw = g.kh = g.dw = g.dh = g.sw = g.sh = 1;
    g.pad_top = g.pad_left = 0;
    g.outw = M;
    g.outh = 1;
    g.npix = M;
    g.ntaps = 1;
    g.K = K;
    g.cout = N;
    g.pad_word = 0;
    ConvEpilogue epi;
    epi.scale_in = epi.bias = epi.scale_out = 0;
    epi.act.type = 0;
    epi.act.p0 = epi.act.p1 = 0.f;
    epi.out = out;
    epi.out_cstep = epi.out_nstep = 0;
    epi.pix_per_img = M;
    epi.batch = 1;
    epi.out_channel0 = 0;
    epi.num_output = N;
    epi.acc_out = 0;
    const ConvFusion no_fusion = {0, 0, 0, 0.f};

    // tiles as for a convolution, never split (Gemm's K loops are long enough to pipeline)
    PipePlan p = plan_pipelined(N, M, K / 64);
    p.splits = 1;
    p.steps_per_split = K / 64;
    const long long blocks = (long long)p.tiles_m * p.tiles_n;
    NCNNHIP_REQUIRE(blocks < (1ll << 31) && blocks * p.tiles_n < (1ll << 32), "gemm: too many tiles");
    dim3 grid((unsigned)blocks), block(256);
#define LAUNCH_GEMM(BM_, BN_)                                                                                                                        \
    hipLaunchKernelGGL((conv_nhwc_pipelined_kernel<BM_, BN_, PIPE_RING, false, true, 1>), grid, block, 0, stream, bq, aq, g, epi, no_fusion, tail, (int)out_stride, N, \
                       p.tiles_m, p.tiles_n, 1, p.steps_per_split, tile_magic(p.tiles_n), (int32_t*)0, (unsigned*)0, (const float*)0, 0)
    if (p.bm == 128 && p.bn == 256)
        LAUNCH_GEMM(128, 256);
    else if (p.bm == 128 && p.bn == 128)
        LAUNCH_GEMM(128, 128);
    else if (p.bm == 128)
        LAUNCH_GEMM(128, 64);
    else if (p.bn == 256)
        LAUNCH_GEMM(64, 256);
    else if (p.bn == 128)
        LAUNCH_GEMM(64, 128);
    else
        LAUNCH_GEMM(64, 64);
#undef LAUNCH_GEMM
    return launch_status("conv_nhwc_pipelined_kernel<gemm>");
}

} // namespace ncnnhip
