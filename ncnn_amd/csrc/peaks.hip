// Measured ceilings of the chip the kernels run on, for the roofline lines of the benchmark: what the matrix pipe
// sustains on int8 operands with nothing else going on, and what a kernel that does nothing but read gets out of HBM.
// The published peaks (5.0 POP/s int8, 8 TB/s) assume the top clock and a full pipe; these two kernels say what this
// part reaches at the clock it actually holds under that load.
#include "common.h"

namespace ncnnhip {

typedef int v4i_pk __attribute__((ext_vector_type(4)));
typedef int v16i_pk __attribute__((ext_vector_type(16)));

// One wavefront per SIMD (one workgroup of 256 per compute unit), eight independent accumulator chains of
// v_mfma_i32_32x32x32_i8 back to back from registers: no memory, no LDS, no dependent issue.  Operands: all zero (hardly a
// bit toggles: the pipe's rate at the top clock) or pseudo-random bytes (the data the benchmark multiplies: power, and so
// the clock, is what differs).  Workgroup 0 reports the shader cycles and the 100 MHz wall ticks its loop took.
__global__ __launch_bounds__(256) void peak_mfma_i8_kernel(int iters, int random_operands, long long* __restrict__ clocks, int* __restrict__ sink)
{
    const unsigned x = random_operands ? (threadIdx.x + 1 + blockIdx.x * 256u) * 2654435761u : 0u;
    v4i_pk a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
    {
        a[i] = v4i_pk{(int)(x * (3u + i)), (int)(x * (7u + 2 * i)), (int)(x * (13u + 4 * i)), (int)(x * (29u + 6 * i))};
        b[i] = v4i_pk{(int)(x * (31u + i)), (int)(x * (37u + 2 * i)), (int)(x * (41u + 4 * i)), (int)(x * (43u + 6 * i))};
    }
    v16i_pk acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int t = 0; t < iters; t++)
    {
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 1], b[(i >> 1) & 1], acc[i], 0, 0, 0);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += acc[i][r];
    if (s == 0x7fffffff) sink[0] = s; // never true for these operands; keeps the chains alive
    if (threadIdx.x == 0 && blockIdx.x == 0)
    {
        clocks[0] = c1 - c0;
        clocks[1] = w1 - w0;
    }
}

// Reads `nvec` 16-byte words once, non-temporal, and folds them; nothing is written.  A workgroup owns U * 4 KB of
// consecutive memory, a wavefront's load covers 1 KB of it, and a lane issues all U loads before it looks at the first
// one: the whole share of a workgroup is in flight at once, which is what a bandwidth kernel on this chip needs.
template<int U>
__global__ __launch_bounds__(256) void peak_hbm_read_kernel(const v4i_pk* __restrict__ src, size_t nvec, int* __restrict__ sink)
{
    const size_t base = (size_t)blockIdx.x * (256 * U) + threadIdx.x;
    v4i_pk t[U];
#pragma unroll
    for (int u = 0; u < U; u++)
    {
        size_t i = base + (size_t)u * 256;
        if (i >= nvec) i = nvec - 1;
        t[u] = __builtin_nontemporal_load(src + i);
    }
    v4i_pk acc = {0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < U; u++) acc += t[u];
    const int s = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (s == 0x12345679) sink[0] = s; // practically never; keeps the loads alive without a store per lane
}

// one wavefront; each launch reads what the launch before it wrote, as the layers of a net do
__global__ void __launch_bounds__(64) peak_launch_chain_kernel(int* counter)
{
    if (threadIdx.x == 0) counter[0] = counter[0] + 1;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_peak_mfma_i8(int iters, int random_operands, void* scratch_dev, void* stream)
{
    NCNNHIP_REQUIRE(iters >= 1 && scratch_dev, "ncnnhip_peak_mfma_i8: bad argument");
    int dev = 0;
    NCNNHIP_CHECK(hipGetDevice(&dev));
    int cus = 0;
    NCNNHIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    long long* clocks = static_cast<long long*>(scratch_dev);
    hipLaunchKernelGGL(peak_mfma_i8_kernel, dim3(cus), dim3(256), 0, as_stream(stream), iters, random_operands, clocks, reinterpret_cast<int*>(clocks + 2));
    return launch_status("peak_mfma_i8_kernel");
}

int ncnnhip_peak_hbm_read(const void* src_dev, size_t bytes, int loads_per_lane, void* scratch_dev, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && scratch_dev && bytes >= 16 && bytes % 16 == 0, "ncnnhip_peak_hbm_read: %zu bytes (a multiple of 16)", bytes);
    NCNNHIP_REQUIRE((reinterpret_cast<uintptr_t>(src_dev) & 15) == 0, "ncnnhip_peak_hbm_read: source must be 16-byte aligned");
    const size_t nvec = bytes / 16;
    const v4i_pk* src = static_cast<const v4i_pk*>(src_dev);
    int* sink = static_cast<int*>(scratch_dev);
#define LAUNCH_READ(U_)                                                                                                    \
    do                                                                                                                     \
    {                                                                                                                      \
        const size_t groups = (nvec + 256 * U_ - 1) / (256 * U_);                                                          \
        NCNNHIP_REQUIRE(groups < (1ull << 31), "ncnnhip_peak_hbm_read: too many workgroups");                            \
        hipLaunchKernelGGL(peak_hbm_read_kernel<U_>, dim3((unsigned)groups), dim3(256), 0, as_stream(stream), src, nvec, sink); \
    } while (0)
    switch (loads_per_lane)
    {
    case 4: LAUNCH_READ(4); break;
    case 8: LAUNCH_READ(8); break;
    case 16: LAUNCH_READ(16); break;
    case 32: LAUNCH_READ(32); break;
    default: NCNNHIP_REQUIRE(false, "ncnnhip_peak_hbm_read: loads_per_lane %d (4, 8, 16 or 32)", loads_per_lane);
    }
#undef LAUNCH_READ
    return launch_status("peak_hbm_read_kernel");
}

int ncnnhip_peak_launch_chain(int launches, void* scratch_dev, void* stream)
{
    NCNNHIP_REQUIRE(launches >= 1 && scratch_dev, "ncnnhip_peak_launch_chain: bad argument");
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(peak_launch_chain_kernel, dim3(1), dim3(64), 0, as_stream(stream), static_cast<int*>(scratch_dev));
    return launch_status("peak_launch_chain_kernel");
}

} // extern "C"
