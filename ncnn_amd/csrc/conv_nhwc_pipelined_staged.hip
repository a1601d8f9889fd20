// One launch for a convolution whose input blob is still fp32 / fp16: the pipelined kernel with its quantising loader
// (template argument AIN = 4 / 2).  The kernel itself is in conv_nhwc_pipelined_kernel.h.
#include "conv_nhwc_pipelined_kernel.h"

namespace ncnnhip {

// ---- one launch for a layer whose input is still fp32 / fp16: the kernel's quantising loader (AIN = 4 / 2)
static const size_t STAGED_TILE_LIMIT = 96u << 10; // bytes of LDS for the tile's operands: (64 pixels + BN channels) x K
static const size_t STAGED_LDS_LIMIT = 124u << 10; // operands + input cache (the epilogue staging takes up to 34 KiB more)

static bool staged_plan(const NhwcGeom& g_in, NhwcGeom& g, PipePlan& p, int& mode)
{
    g = g_in;
    const int dense = g.kw == 1 && g.kh == 1 && g.sw == 1 && g.sh == 1 && g.pad_top == 0 && g.pad_left == 0 && g.outw == g.W && g.outh == g.H && g.tapK == g.Cp;
    if (dense)
    {
        g.H = g.outh = 1;
        g.W = g.outw = g.npix;
    }
    const int steps = g.K / 64;
    p = plan_pipelined(g.cout, g.npix, steps);
    mode = dense ? 1 : 0;
    // (K is split over workgroups exactly where the plan splits it for an int8 blob.  Splitting shorter K loops as well
    // -- three steps per workgroup for a 3x3 64 -> 64 layer on 56x56, 147 workgroups instead of 49 -- was measured: the
    // hand-off through memory costs more than the shorter loader saves, 10.7 us against 8.6.)
    const int wg_steps = p.splits > 1 ? p.steps_per_split : steps;
    // 64-pixel tiles; the workgroup's share of both operands in LDS; at most 48 weight loads in flight per lane (the
    // counter holds 63); zero border; tap offsets that grow with the tap index (the cached run is bounded by the first and last tap)
    return p.bm == 64 && p.bn <= 128 && (size_t)wg_steps * 64 * (64 + p.bn) <= STAGED_TILE_LIMIT && wg_steps * (p.bn / 64) <= 48 && g.pad_word == 0 &&
           g.tapK == g.Cp && (dense || (long long)g.dh * g.W > (long long)(g.kw - 1) * g.dw) &&
           (long long)p.tiles_m * p.tiles_n * p.splits * p.tiles_n < (1ll << 32);
}

bool conv_nhwc_staged_supported(const NhwcGeom& g_in)
{
    NhwcGeom g;
    PipePlan p;
    int mode;
    return staged_plan(g_in, g, p, mode);
}

size_t conv_nhwc_staged_workspace_bytes(const NhwcGeom& g_in)
{
    NhwcGeom g;
    PipePlan p;
    int mode;
    if (!staged_plan(g_in, g, p, mode) || p.splits <= 1) return 0;
    return SPLIT_COUNTER_BYTES + (size_t)p.splits * p.tiles_m * p.tiles_n * p.bm * p.bn * sizeof(int32_t);
}

int launch_conv_nhwc_staged(const NhwcGeom& g_in, const int8_t* wpk, const void* x, int x_elemsize, const float* x_scale, const ConvEpilogue& epi,
                            const ConvFusion& fusion, int out_cp, void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    NhwcGeom g;
    PipePlan p;
    int mode;
    NCNNHIP_REQUIRE(x_elemsize == 4 || x_elemsize == 2, "convolution: activations of %d bytes per value", x_elemsize);
    NCNNHIP_REQUIRE(staged_plan(g_in, g, p, mode), "convolution: this layer does not fit the one-launch form (ask ncnnhip_conv_from_float_supported first)");
    const int wg_steps = p.splits > 1 ? p.steps_per_split : g.K / 64;
    const size_t tile_bytes = (size_t)wg_steps * 64 * (64 + p.bn);
    int32_t* partial = 0;
    unsigned* counters = 0;
    if (p.splits > 1)
    {
        const size_t need = SPLIT_COUNTER_BYTES + (size_t)p.splits * p.tiles_m * p.tiles_n * p.bm * p.bn * sizeof(int32_t);
        NCNNHIP_REQUIRE(workspace && workspace_bytes >= need, "convolution: workspace of %zu bytes required", need);
        counters = (unsigned*)workspace; // zero on entry (the caller cleared the workspace once), zero again on exit
        partial = (int32_t*)((char*)workspace + SPLIT_COUNTER_BYTES);
    }
    // Behind the operands, a cache for the run of input pixels a tile touches (quantised once instead of once per tap): 64
    // consecutive output pixels span at most (63 / outw + 2) output rows, one more image-to-image gap of at most
    // (H + pad) rows, and the kernel's own extent.  An estimate only: the kernel measures each tile's run and gathers
    // from global memory when it does not fit.
    size_t cache_bytes = 0;
    if (mode == 0 && (long long)epi.batch * g.H * g.W < (1ll << 30))
    {
        const long long rows = (63 / g.outw + 2) * (long long)g.sh + (long long)(g.kh - 1) * g.dh + g.H - (long long)(g.outh - 1) * g.sh + 2;
        const long long pixels = rows * g.W + (long long)(g.kw - 1) * g.dw + 64ll * g.sw;
        const size_t room = STAGED_LDS_LIMIT - tile_bytes;
        cache_bytes = (size_t)std::min<long long>(pixels * g.Cp, (long long)room) & ~(size_t)15;
    }
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n * p.splits)), block(256);
    const GemmTail no_gemm = {0, 0, 0, 0, -1, 1.f, 1.f};
    const int8_t* xb = static_cast<const int8_t*>(x);
#define LAUNCH_STAGED(BN_, SPLIT_, MODE_, AIN_)                                                                                                              \
    do                                                                                                                                                       \
    {                                                                                                                                                        \
        auto kernel = conv_nhwc_pipelined_kernel<64, BN_, PIPE_RING, SPLIT_, false, MODE_, AIN_>;                                                                    \
        static std::once_flag once;                                                                                                                          \
        static hipError_t attr = hipSuccess;                                                                                                                 \
        std::call_once(once, [&]() { attr = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)STAGED_LDS_LIMIT); });  \
        NCNNHIP_CHECK(attr);                                                                                                                                 \
        hipLaunchKernelGGL(kernel, grid, block, tile_bytes + cache_bytes, stream, wpk, xb, g, epi, fusion, no_gemm, out_cp, out_cp, p.tiles_m, p.tiles_n, \
                           p.splits, p.steps_per_split, tile_magic(p.tiles_n), partial, counters, x_scale, (int)cache_bytes);                               \
    } while (0)
#define LAUNCH_STAGED_IN(BN_, MODE_)                 \
    do                                               \
    {                                                \
        if (x_elemsize == 4 && p.splits > 1)         \
            LAUNCH_STAGED(BN_, true, MODE_, 4);      \
        else if (x_elemsize == 4)                    \
            LAUNCH_STAGED(BN_, false, MODE_, 4);     \
        else if (p.splits > 1)                       \
            LAUNCH_STAGED(BN_, true, MODE_, 2);      \
        else                                         \
            LAUNCH_STAGED(BN_, false, MODE_, 2);     \
    } while (0)
    if (p.bn == 128 && mode == 1)
        LAUNCH_STAGED_IN(128, 1);
    else if (p.bn == 128)
        LAUNCH_STAGED_IN(128, 0);
    else if (mode == 1)
        LAUNCH_STAGED_IN(64, 1);
    else
        LAUNCH_STAGED_IN(64, 0);
#undef LAUNCH_STAGED_IN
#undef LAUNCH_STAGED
    return launch_status("conv_nhwc_pipelined_kernel (quantising loader)");
}

} // namespace ncnnhip
