// The pipelined channels-last convolution kernel's launches with one workgroup per output tile: Convolution (every
// addressing mode) and InnerProduct, the planner they share with the other forms, and the InnerProduct entry that
// allocates nothing.  The kernel itself is in conv_nhwc_pipelined_kernel.h.
#include "conv_nhwc_pipelined_kernel.h"

namespace ncnnhip {

constexpr int SPLIT_MIN_STEPS = 12;

PipePlan plan_pipelined(int cout, long long npix, int steps)
{
    PipePlan p;
    // channel tile: the width that pads the channel count least (padded channels cost matrix-core time and unbalance the
    // wavefronts' epilogues: 144 channels in one 256-wide tile ran 34 us, in three 64-wide tiles 21), the wider on a tie
    p.bn = 64;
    for (int bn = 128; bn <= 256; bn *= 2)
        if (ceil_div(cout, bn) * bn <= ceil_div(cout, p.bn) * p.bn) p.bn = bn;
    p.bm = 128;
    auto tiles = [&]() { return (long long)ceil_div(npix, p.bm) * ceil_div(cout, p.bn); };
    // measured over the ResNet-50 / MobileNetV2 layers: more, smaller workgroups win until there are a few
    // thousand of them (these layers are latency bound, not matrix-core bound)
    if (tiles() < 100000) p.bm = 64;
    if (tiles() < 1024 && p.bn == 256) p.bn = 128;
    if (tiles() < 512 && p.bn == 128 && cout > 64) p.bn = 64;
    p.tiles_m = ceil_div(npix, p.bm);
    p.tiles_n = ceil_div(cout, p.bn);
    p.splits = 1;
    const long long t = tiles();
    if (t < 256 && t <= SPLIT_MAX_TILES && steps >= 2 * SPLIT_MIN_STEPS)
    {
        // fewer tiles than CUs: split K until there is about one workgroup per CU (two splits from 128 tiles up; with the
        // limit at 128 tiles the 196-tile 3x3 layers of ResNet-50's fourth stage at batch 16 ran unsplit on 196 of the 256
        // CUs), at least 12 steps each.  A split costs about 2 us (partial sums through memory, the last workgroup of a
        // tile adds them up): with 8 steps each, the 16-step 1x1 layers 1024 -> 256 of ResNet-50 ran 8.6 us in two halves
        // and 6.8 whole at batch 16, the 18-step 3x3 layers 128 -> 128 9.6 and 7.5 at batch 8; summed over a pass the
        // kernels take 350 / 355 / 362 / 385 us at batch 1 with at least 8 / 12 / 16 / 24 steps, 404 / 389 / 395 / 414
        // at batch 4, 459 / 449 / 446 / 466 at batch 8, 568 / 555 / 556 / 565 at batch 16 (MobileNetV2: no difference)
        const int want = (int)((256 + t - 1) / t);
        const int max_splits = steps / SPLIT_MIN_STEPS;
        p.splits = want < max_splits ? want : max_splits;
        if (p.splits < 1) p.splits = 1;
    }
    p.steps_per_split = ceil_div(steps, p.splits);
    p.splits = ceil_div(steps, p.steps_per_split);
    return p;
}

size_t conv_nhwc_pipelined_workspace_words(int cout, long long npix, int steps)
{
    const PipePlan p = plan_pipelined(cout, npix, steps);
    if (p.splits <= 1) return 0;
    return SPLIT_COUNTER_BYTES / sizeof(int32_t) + (size_t)p.splits * p.tiles_m * p.tiles_n * p.bm * p.bn;
}

int launch_conv_nhwc_pipelined(const NhwcGeom& g_in, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp,
                               void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    if (conv_pointwise_fits(g_in, epi, fusion, out_cp) || conv_pointwise_stem_fits(g_in, epi, fusion, out_cp)) return launch_conv_pointwise(g_in, wpk, x, epi, out_cp, stream);
    if (conv_resident_fits(g_in, epi, fusion, out_cp)) return launch_conv_resident(g_in, wpk, x, epi, fusion, out_cp, stream);
    NhwcGeom g = g_in;
    // A 1x1, stride-1, unpadded layer reads input pixel n for output pixel n, whatever the image shape: present it as
    // one row of npix pixels, and the kernel skips the pixel -> (image, y, x) divisions.
    const int dense = g.kw == 1 && g.kh == 1 && g.sw == 1 && g.sh == 1 && g.pad_top == 0 && g.pad_left == 0 && g.outw == g.W && g.outh == g.H && g.tapK == g.Cp;
    if (dense)
    {
        g.H = g.outh = 1;
        g.W = g.outw = g.npix;
    }
    PipePlan p = plan_pipelined(g.cout, g.npix, g.K / 64);
    // the narrow-input first layer has four K steps at most: from a million output pixels up, 128-pixel tiles halve the number of
    // workgroup prologues (ResNet-50's 7 x 7 first layer at batch 128: the pass 2.22 -> 2.20 ms; at batch 16, 0.2 M pixels, no gain)
    if ((g.tapK == 16 || g.tapK == 32) && p.splits == 1 && p.bm == 64 && g.npix >= (1 << 20))
    {
        p.bm = 128;
        p.tiles_m = ceil_div(g.npix, 128);
    }
    const long long blocks = (long long)p.tiles_m * p.tiles_n * p.splits;
    NCNNHIP_REQUIRE(blocks < (1ll << 31) && blocks * p.tiles_n < (1ll << 32), "convolution: too many tiles");
    int32_t* partial = 0;
    unsigned* counters = 0;
    if (p.splits > 1)
    {
        const size_t need = SPLIT_COUNTER_BYTES + (size_t)p.splits * p.tiles_m * p.tiles_n * p.bm * p.bn * sizeof(int32_t);
        NCNNHIP_REQUIRE(workspace && workspace_bytes >= need, "convolution: workspace of %zu bytes required", need);
        counters = (unsigned*)workspace; // zero on entry (the caller cleared the workspace once), zero again on exit
        partial = (int32_t*)((char*)workspace + SPLIT_COUNTER_BYTES);
    }
    dim3 grid((unsigned)blocks), block(256);
    const GemmTail no_gemm = {0, 0, 0, 0, -1, 1.f, 1.f};
    // addressing mode (the kernel's MODE); the K-split kernels exist for modes 0, 1 and 3 only (a narrow-input layer has
    // too few K steps to be split)
    const int mode = dense ? 1 : ((g.tapK == 16 || g.tapK == 32) && p.splits == 1) ? 2 : (g.tapK % 64 == 0 && g.tapK == g.Cp) ? 3 : 0;
    if (p.splits > 1) return launch_pipe_split(p, mode, wpk, x, g, epi, fusion, out_cp, out_cp, partial, counters, stream);
#define LAUNCH_PIPE_MODE(BM_, BN_, MODE_)                                                                                                                \
    hipLaunchKernelGGL((conv_nhwc_pipelined_kernel<BM_, BN_, PIPE_RING, false, false, MODE_>), grid, block, 0, stream, wpk, x, g, epi, fusion, no_gemm, out_cp, \
                       out_cp, p.tiles_m, p.tiles_n, p.splits, p.steps_per_split, tile_magic(p.tiles_n), partial, counters, (const float*)0, 0)
#define LAUNCH_PIPE(BM_, BN_)                  \
    do                                         \
    {                                          \
        if (mode == 1)                         \
            LAUNCH_PIPE_MODE(BM_, BN_, 1);     \
        else if (mode == 2)                    \
            LAUNCH_PIPE_MODE(BM_, BN_, 2);     \
        else if (mode == 3)                    \
            LAUNCH_PIPE_MODE(BM_, BN_, 3);     \
        else                                   \
            LAUNCH_PIPE_MODE(BM_, BN_, 0);     \
    } while (0)
    if (p.bm == 128 && p.bn == 256)
        LAUNCH_PIPE(128, 256);
    else if (p.bm == 128 && p.bn == 128)
        LAUNCH_PIPE(128, 128);
    else if (p.bm == 128)
        LAUNCH_PIPE(128, 64);
    else if (p.bn == 256)
        LAUNCH_PIPE(64, 256);
    else if (p.bn == 128)
        LAUNCH_PIPE(64, 128);
    else
        LAUNCH_PIPE(64, 64);
#undef LAUNCH_PIPE
#undef LAUNCH_PIPE_MODE
    return launch_status("conv_nhwc_pipelined_kernel");
}

int launch_fc_via_conv_pipelined(const int8_t* x, size_t x_stride, int rows, int K, int num_output, const int8_t* weight, const ConvEpilogue& epi,
                                 size_t out_stride, void* workspace, size_t workspace_bytes, hipStream_t stream, bool* handled)
{
    *handled = false;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(epi.out)) & 15) == 0;
    if (K % 64 || num_output % 4 || x_stride % 16 || out_stride % 4 || !aligned || epi.scale_out || epi.acc_out) return NCNNHIP_OK;
    if ((long long)rows * (long long)x_stride >= (1ll << 31)) return NCNNHIP_OK;
    const size_t need = conv_nhwc_pipelined_workspace_words(num_output, rows, K / 64) * sizeof(int32_t);
    if (need > workspace_bytes || (need && !workspace)) return NCNNHIP_OK;
    *handled = true;

    NhwcGeom g;
    g.H = 1;
    g.W = rows;
    g.Cp = (int)x_stride;
    g.tapK = g.Cp;
    g.kw = g.kh = g.dw = g.dh = g.sw = g.sh = 1;
    g.pad_top = g.pad_left = 0;
    g.outw = rows;
    g.outh = 1;
    g.npix = rows;
    g.ntaps = 1;
    g.K = K;
    g.cout = num_output;
    g.pad_word = 0;
    const ConvFusion no_fusion = {0, 0, 0, 0.f};
    const GemmTail no_gemm = {0, 0, 0, 0, -1, 1.f, 1.f};
    const PipePlan p = plan_pipelined(num_output, rows, K / 64);
    int32_t* partial = 0;
    unsigned* counters = 0;
    if (p.splits > 1)
    {
        counters = (unsigned*)workspace;
        partial = (int32_t*)((char*)workspace + SPLIT_COUNTER_BYTES);
    }
    NCNNHIP_REQUIRE((long long)p.tiles_m * p.tiles_n * p.splits * p.tiles_n < (1ll << 32), "innerproduct: too many tiles");
    dim3 grid((unsigned)((long long)p.tiles_m * p.tiles_n * p.splits)), block(256);
    // rows are few: only the 64-pixel tiles occur
    if (p.bm != 64)
    {
        *handled = false;
        return NCNNHIP_OK;
    }
    if (p.splits > 1) return launch_pipe_split(p, 1, weight, x, g, epi, no_fusion, (int)out_stride, num_output, partial, counters, stream);
#define LAUNCH_FC(BN_)                                                                                                                                \
    hipLaunchKernelGGL((conv_nhwc_pipelined_kernel<64, BN_, PIPE_RING, false, false, 1>), grid, block, 0, stream, weight, x, g, epi, no_fusion, no_gemm, \
                       (int)out_stride, num_output, p.tiles_m, p.tiles_n, p.splits, p.steps_per_split, tile_magic(p.tiles_n), partial, counters, (const float*)0, 0)
    if (p.bn == 256)
        LAUNCH_FC(256);
    else if (p.bn == 128)
        LAUNCH_FC(128);
    else
        LAUNCH_FC(64);
#undef LAUNCH_FC
    return launch_status("conv_nhwc_pipelined_kernel<fc>");
}

// ---- InnerProduct through the K-split kernel on a scratch buffer the library holds itself, for callers that cannot
// allocate (under stream capture, in a serving loop that must not touch the allocator).  The array below is the
// workspace launch_fc_via_conv_pipelined otherwise gets from its caller; every device the library runs on holds its own
// copy of it, at its own address, until the process ends.
constexpr size_t STATIC_SCRATCH_PARTIAL_BYTES = 4u << 20;
constexpr size_t STATIC_SCRATCH_BYTES = SPLIT_COUNTER_BYTES + STATIC_SCRATCH_PARTIAL_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int STATIC_SCRATCH_MAX_DEVICES = 64;
static void* g_scratch_ptr[STATIC_SCRATCH_MAX_DEVICES]; // device address of `scratch` on each device, 0 = not looked up yet
static std::mutex g_scratch_mutex;

// The array's name is only a handle on the host; its address on the CURRENT device comes from the runtime, once per device.
int static_scratch_for_current_device(void** ptr)
{
    int dev = 0;
    NCNNHIP_CHECK(hipGetDevice(&dev));
    NCNNHIP_REQUIRE(dev >= 0 && dev < STATIC_SCRATCH_MAX_DEVICES, "device %d beyond the %d the static scratch table covers", dev, STATIC_SCRATCH_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev])
    {
        void* p = 0;
        NCNNHIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        NCNNHIP_REQUIRE(p, "hipGetSymbolAddress returned a null address for the static scratch");
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return NCNNHIP_OK;
}

// one workgroup: the arrival counters at the head of the scratch start every call at zero, whatever the last call left
__global__ __launch_bounds__(256) void clear_split_counters_kernel(unsigned* __restrict__ counters)
{
    for (int i = threadIdx.x; i < SPLIT_MAX_TILES; i += 256) counters[i] = 0u;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" int ncnnhip_innerproduct_int8_noalloc(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output, const int8_t* weight_dev,
                                                 const float* scale_in_dev, const float* bias_dev, ncnnhip_activation act, float* out_dev, size_t out_stride,
                                                 void* stream)
{
    NCNNHIP_REQUIRE(x_dev && weight_dev && scale_in_dev && out_dev, "ncnnhip_innerproduct_int8_noalloc: null pointer");
    NCNNHIP_REQUIRE(rows >= 1 && num_input >= 1 && num_output >= 1, "ncnnhip_innerproduct_int8_noalloc: bad shape");
    NCNNHIP_REQUIRE(x_stride >= (size_t)num_input && out_stride >= (size_t)num_output, "ncnnhip_innerproduct_int8_noalloc: stride too small");
    void* ptr = 0;
    int ret = static_scratch_for_current_device(&ptr);
    if (ret != NCNNHIP_OK) return ret;
    // few rows: the kernel that needs no scratch (and so no ordering between calls that share it)
    const bool aligned = ((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(weight_dev)) & 15) == 0 && x_stride % 16 == 0;
    if (aligned && fc_skinny_takes(rows, num_input, num_output))
        return ncnnhip_innerproduct_int8(x_dev, x_stride, rows, num_input, num_output, weight_dev, scale_in_dev, bias_dev, act, out_dev, out_stride, 0, stream);
    if (rows >= 8 && num_input % 64 == 0)
    {
        const size_t need = conv_nhwc_pipelined_workspace_words(num_output, rows, num_input / 64) * sizeof(int32_t);
        NCNNHIP_REQUIRE(need <= STATIC_SCRATCH_BYTES,
                        "ncnnhip_innerproduct_int8_noalloc: %d x %d -> %d needs %zu bytes of scratch, the library holds %zu; use ncnnhip_innerproduct_int8_ws",
                        rows, num_input, num_output, need, (size_t)STATIC_SCRATCH_BYTES);
        ConvEpilogue epi;
        epi.scale_in = scale_in_dev;
        epi.bias = bias_dev;
        epi.scale_out = 0;
        epi.act = act;
        epi.out = out_dev;
        epi.out_cstep = epi.out_nstep = 0;
        epi.pix_per_img = rows;
        epi.batch = 1;
        epi.out_channel0 = 0;
        epi.num_output = num_output;
        epi.acc_out = 0;
        if (need)
        {
            hipLaunchKernelGGL(clear_split_counters_kernel, dim3(1), dim3(256), 0, as_stream(stream), (unsigned*)ptr);
            ret = launch_status("clear_split_counters_kernel");
            if (ret != NCNNHIP_OK) return ret;
        }
        bool handled = false;
        ret = launch_fc_via_conv_pipelined(x_dev, x_stride, rows, num_input, num_output, weight_dev, epi, out_stride, ptr, STATIC_SCRATCH_BYTES,
                                           as_stream(stream), &handled);
        if (handled) return ret;
    }
    // shapes the matrix-core kernel does not take run on the kernel that needs no scratch at all
    return ncnnhip_innerproduct_int8(x_dev, x_stride, rows, num_input, num_output, weight_dev, scale_in_dev, bias_dev, act, out_dev, out_stride, 0, stream);
}
