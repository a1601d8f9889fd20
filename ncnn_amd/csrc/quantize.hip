// fp32 -> int8 quantisation kernels and the small layout helpers Gemm needs.
// All of them are HBM-bound streaming kernels: 16-byte loads, 4-byte packed int8 stores.
#include "common.h"

namespace ncnnhip {

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d)
{
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}

// y[b][r][i] = float2int8(x[b][r][i] * scale_r)
template<bool VEC>
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x, size_t xs, size_t xn, int8_t* __restrict__ y,
                                                        size_t ys, size_t yn, int cols, const float* __restrict__ scales, int nscales)
{
    const int r = blockIdx.y;
    const int b = blockIdx.z;
    const float s = nscales == 1 ? scales[0] : scales[r];
    const float* xr = x + (size_t)b * xn + (size_t)r * xs;
    int8_t* yr = y + (size_t)b * yn + (size_t)r * ys;
    const int i0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i0 >= cols) return;
    if (VEC && i0 + 4 <= cols)
    {
        const float4 v = *reinterpret_cast<const float4*>(xr + i0);
        *reinterpret_cast<uint32_t*>(yr + i0) = pack4(float2int8(mul_rn(v.x, s)), float2int8(mul_rn(v.y, s)),
                                                       float2int8(mul_rn(v.z, s)), float2int8(mul_rn(v.w, s)));
    }
    else
    {
        for (int i = i0; i < i0 + 4 && i < cols; i++) yr[i] = (int8_t)float2int8(mul_rn(xr[i], s));
    }
}

__device__ __forceinline__ float block_max_256(float v, float* red)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return v;
}

// One workgroup per row: absmax, scale = 127/absmax (1 if the row is all zero), then quantise.
// The second sweep re-reads the row, which is still resident in L2.
template<bool VEC>
__global__ __launch_bounds__(256) void quantize_rows_dynamic_kernel(const float* __restrict__ a, size_t as, int cols,
                                                                     int8_t* __restrict__ aq, size_t aqs, float* __restrict__ scales)
{
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* ar = a + (size_t)r * as;
    int8_t* qr = aq + (size_t)r * aqs;

    float m = 0.f;
    if (VEC)
    {
        const int n4 = cols >> 2;
        for (int i = threadIdx.x; i < n4; i += 256)
        {
            const float4 v = reinterpret_cast<const float4*>(ar)[i];
            m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
        for (int i = (n4 << 2) + threadIdx.x; i < cols; i += 256) m = fmaxf(m, fabsf(ar[i]));
    }
    else
    {
        for (int i = threadIdx.x; i < cols; i += 256) m = fmaxf(m, fabsf(ar[i]));
    }
    m = block_max_256(m, red);
    const float s = m == 0.f ? 1.f : div_rn(127.f, m);
    if (threadIdx.x == 0) scales[r] = s;

    if (VEC)
    {
        const int n4 = cols >> 2;
        for (int i = threadIdx.x; i < n4; i += 256)
        {
            const float4 v = reinterpret_cast<const float4*>(ar)[i];
            reinterpret_cast<uint32_t*>(qr)[i] = pack4(float2int8(mul_rn(v.x, s)), float2int8(mul_rn(v.y, s)),
                                                       float2int8(mul_rn(v.z, s)), float2int8(mul_rn(v.w, s)));
        }
        for (int i = (n4 << 2) + threadIdx.x; i < cols; i += 256) qr[i] = (int8_t)float2int8(mul_rn(ar[i], s));
    }
    else
    {
        for (int i = threadIdx.x; i < cols; i += 256) qr[i] = (int8_t)float2int8(mul_rn(ar[i], s));
    }
}

// Rows of up to 8192 aligned floats: the row is read ONCE into registers (NV float4 per thread), reduced, and quantised
// from the registers -- 5 bytes of traffic per element instead of 9.
// NT: the fp32 source is larger than the chip's last-level cache can hold on to, so it is read with non-temporal loads and
// leaves the cache to the int8 rows the Gemm is about to read (8192 x 8192: 88 -> 57 us; smaller sources are re-read from
// the cache by the next pass over the same buffer and lose 1 us this way).
template<int NV, bool NT>
__global__ __launch_bounds__(256) void quantize_rows_dynamic_reg_kernel(const float* __restrict__ a, size_t as, int cols,
                                                                         int8_t* __restrict__ aq, size_t aqs, float* __restrict__ scales, int tiled)
{
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float4* ar = reinterpret_cast<const float4*>(a + (size_t)r * as);
    // tiled: the 256x256 Gemm kernel's operand layout, [r / 256][k / 64][r % 256][k % 64]; word i of the row (bytes 4i .. 4i+3)
    // is word i % 16 of K step i / 16
    uint32_t* qr = tiled ? reinterpret_cast<uint32_t*>(aq + ((size_t)(r >> 8) * (cols >> 6) * 256 + (r & 255)) * 64) : reinterpret_cast<uint32_t*>(aq + (size_t)r * aqs);
    const int n4 = cols >> 2; // cols % 4 == 0 here
    float4 v[NV];
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < NV; j++)
    {
        const int i = threadIdx.x + j * 256;
        if (NT)
        {
            typedef float v4f_nt __attribute__((ext_vector_type(4)));
            const v4f_nt t = i < n4 ? __builtin_nontemporal_load(reinterpret_cast<const v4f_nt*>(ar) + i) : v4f_nt{0.f, 0.f, 0.f, 0.f};
            v[j] = float4{t[0], t[1], t[2], t[3]};
        }
        else
            v[j] = i < n4 ? ar[i] : float4{0.f, 0.f, 0.f, 0.f};
        m = fmaxf(m, fmaxf(fmaxf(fabsf(v[j].x), fabsf(v[j].y)), fmaxf(fabsf(v[j].z), fabsf(v[j].w))));
    }
    m = block_max_256(m, red);
    const float s = m == 0.f ? 1.f : div_rn(127.f, m);
    if (threadIdx.x == 0) scales[r] = s;
#pragma unroll
    for (int j = 0; j < NV; j++)
    {
        const int i = threadIdx.x + j * 256;
        if (i < n4)
        {
            const uint32_t q4 = pack4((int)float2int8_as_float(mul_rn(v[j].x, s)), (int)float2int8_as_float(mul_rn(v[j].y, s)),
                                      (int)float2int8_as_float(mul_rn(v[j].z, s)), (int)float2int8_as_float(mul_rn(v[j].w, s)));
            uint32_t* dst = qr + (tiled ? (size_t)(i >> 4) * 4096 + (i & 15) : (size_t)i);
            *dst = q4;
        }
    }
}

// whole-tensor absmax: non-negative floats order like their bit patterns, so an integer atomic max works
__global__ void zero_word_kernel(uint32_t* p)
{
    *p = 0u;
}

__global__ __launch_bounds__(256) void tensor_absmax_kernel(const float* __restrict__ b, size_t bs, int cols, uint32_t* out_bits)
{
    __shared__ float red[4];
    const float* br = b + (size_t)blockIdx.x * bs;
    float m = 0.f;
    for (int i = threadIdx.x; i < cols; i += 256) m = fmaxf(m, fabsf(br[i]));
    m = block_max_256(m, red);
    if (threadIdx.x == 0) atomicMax(out_bits, __float_as_uint(m));
}

__global__ void absmax_to_scale_kernel(float* p)
{
    const float m = *p;
    *p = m == 0.f ? 1.f : div_rn(127.f, m);
}

template<typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ src, size_t ss, int rows, int cols, T* __restrict__ dst, size_t ds)
{
    __shared__ T tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
#pragma unroll
    for (int k = 0; k < 32; k += 8)
    {
        const int r = r0 + ty + k, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + k][tx] = src[(size_t)r * ss + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 32; k += 8)
    {
        const int c = c0 + ty + k, r = r0 + tx; // dst[c][r]
        if (r < rows && c < cols) dst[(size_t)c * ds + r] = tile[tx][ty + k];
    }
}

// two transposes of the same shape and strides in one launch (the key and the value columns of an attention layer's cache)
__global__ __launch_bounds__(256) void transpose_pair_kernel(const float* __restrict__ src_a, const float* __restrict__ src_b, size_t ss, int rows, int cols,
                                                             float* __restrict__ dst_a, float* __restrict__ dst_b, size_t ds)
{
    __shared__ float tile[32][33];
    const float* __restrict__ src = blockIdx.z ? src_b : src_a;
    float* __restrict__ dst = blockIdx.z ? dst_b : dst_a;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
#pragma unroll
    for (int k = 0; k < 32; k += 8)
    {
        const int r = r0 + ty + k, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + k][tx] = src[(size_t)r * ss + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 32; k += 8)
    {
        const int c = c0 + ty + k, r = r0 + tx; // dst[c][r]
        if (r < rows && c < cols) dst[(size_t)c * ds + r] = tile[tx][ty + k];
    }
}

static inline bool aligned(const void* p, size_t a)
{
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_quantize(const float* x_dev, size_t x_stride, size_t x_nstep, int8_t* y_dev, size_t y_stride, size_t y_nstep,
                     int rows, int cols, int batch, const float* scales_dev, int nscales, void* stream)
{
    NCNNHIP_REQUIRE(x_dev && y_dev && scales_dev, "ncnnhip_quantize: null pointer");
    NCNNHIP_REQUIRE(rows >= 0 && cols >= 0 && batch >= 1, "ncnnhip_quantize: bad extent %d x %d x %d", rows, cols, batch);
    NCNNHIP_REQUIRE(nscales == 1 || nscales == rows, "ncnnhip_quantize: %d scales for %d rows", nscales, rows);
    NCNNHIP_REQUIRE(rows <= 65535 && batch <= 65535, "ncnnhip_quantize: rows/batch above 65535");
    if (rows == 0 || cols == 0) return NCNNHIP_OK;
    const bool vec = aligned(x_dev, 16) && aligned(y_dev, 4) && x_stride % 4 == 0 && x_nstep % 4 == 0 && y_stride % 4 == 0 && y_nstep % 4 == 0;
    dim3 grid(ceil_div(cols, 1024), rows, batch);
    if (vec)
        hipLaunchKernelGGL(quantize_kernel<true>, grid, dim3(256), 0, as_stream(stream), x_dev, x_stride, x_nstep, y_dev, y_stride, y_nstep, cols, scales_dev, nscales);
    else
        hipLaunchKernelGGL(quantize_kernel<false>, grid, dim3(256), 0, as_stream(stream), x_dev, x_stride, x_nstep, y_dev, y_stride, y_nstep, cols, scales_dev, nscales);
    return launch_status("quantize_kernel");
}

static int quantize_rows_impl(const float* a_dev, size_t a_stride, int rows, int cols, int8_t* aq_dev, size_t aq_stride, float* scales_dev,
                              int tiled, void* stream)
{
    const bool vec = aligned(a_dev, 16) && aligned(aq_dev, 4) && a_stride % 4 == 0 && aq_stride % 4 == 0;
    NCNNHIP_REQUIRE(!tiled || (vec && cols <= 8192), "ncnnhip_gemm_quantize_rows_tiled: needs 16-byte aligned rows of at most 8192 values");
    if (vec && cols % 4 == 0 && cols <= 8192)
    {
        const int nv = ceil_div(cols, 1024);
        const bool nt = (size_t)rows * cols * sizeof(float) > ((size_t)128 << 20);
#define LAUNCH_REG(NV_)                                                                                                                          \
    do                                                                                                                                           \
    {                                                                                                                                            \
        if (nt)                                                                                                                                  \
            hipLaunchKernelGGL((quantize_rows_dynamic_reg_kernel<NV_, true>), dim3(rows), dim3(256), 0, as_stream(stream), a_dev, a_stride, cols, \
                               aq_dev, aq_stride, scales_dev, tiled);                                                                            \
        else                                                                                                                                     \
            hipLaunchKernelGGL((quantize_rows_dynamic_reg_kernel<NV_, false>), dim3(rows), dim3(256), 0, as_stream(stream), a_dev, a_stride,     \
                               cols, aq_dev, aq_stride, scales_dev, tiled);                                                                      \
    } while (0)
        if (nv <= 1)
            LAUNCH_REG(1);
        else if (nv <= 2)
            LAUNCH_REG(2);
        else if (nv <= 4)
            LAUNCH_REG(4);
        else
            LAUNCH_REG(8);
#undef LAUNCH_REG
    }
    else if (vec)
        hipLaunchKernelGGL(quantize_rows_dynamic_kernel<true>, dim3(rows), dim3(256), 0, as_stream(stream), a_dev, a_stride, cols, aq_dev, aq_stride, scales_dev);
    else
        hipLaunchKernelGGL(quantize_rows_dynamic_kernel<false>, dim3(rows), dim3(256), 0, as_stream(stream), a_dev, a_stride, cols, aq_dev, aq_stride, scales_dev);
    return launch_status("quantize_rows_dynamic_kernel");
}

int ncnnhip_gemm_quantize_rows(const float* a_dev, size_t a_stride, int rows, int cols, int8_t* aq_dev, size_t aq_stride,
                               float* scales_dev, void* stream)
{
    NCNNHIP_REQUIRE(a_dev && aq_dev && scales_dev, "ncnnhip_gemm_quantize_rows: null pointer");
    NCNNHIP_REQUIRE(rows >= 0 && cols >= 0, "ncnnhip_gemm_quantize_rows: bad extent");
    NCNNHIP_REQUIRE(a_stride >= (size_t)cols && aq_stride >= (size_t)cols, "ncnnhip_gemm_quantize_rows: stride below cols");
    if (rows == 0) return NCNNHIP_OK;
    return quantize_rows_impl(a_dev, a_stride, rows, cols, aq_dev, aq_stride, scales_dev, 0, stream);
}

int ncnnhip_gemm_quantize_rows_tiled(const float* a_dev, size_t a_stride, int rows, int cols, int8_t* aq_tiled_dev, float* scales_dev, void* stream)
{
    NCNNHIP_REQUIRE(a_dev && aq_tiled_dev && scales_dev, "ncnnhip_gemm_quantize_rows_tiled: null pointer");
    NCNNHIP_REQUIRE(rows >= 256 && rows % 256 == 0 && cols >= 64 && cols % 64 == 0,
                    "ncnnhip_gemm_quantize_rows_tiled: %d rows of %d (multiples of 256 and 64 only)", rows, cols);
    NCNNHIP_REQUIRE(a_stride >= (size_t)cols, "ncnnhip_gemm_quantize_rows_tiled: stride below cols");
    return quantize_rows_impl(a_dev, a_stride, rows, cols, aq_tiled_dev, (size_t)cols, scales_dev, 1, stream);
}

int ncnnhip_gemm_quantize_tensor(const float* b_dev, size_t b_stride, int rows, int cols, int8_t* bq_dev, size_t bq_stride,
                                 float* scale_dev, void* stream)
{
    NCNNHIP_REQUIRE(b_dev && bq_dev && scale_dev, "ncnnhip_gemm_quantize_tensor: null pointer");
    NCNNHIP_REQUIRE(rows >= 1 && cols >= 1 && rows <= 65535, "ncnnhip_gemm_quantize_tensor: bad extent");
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(zero_word_kernel, dim3(1), dim3(1), 0, s, reinterpret_cast<uint32_t*>(scale_dev));
    hipLaunchKernelGGL(tensor_absmax_kernel, dim3(rows), dim3(256), 0, s, b_dev, b_stride, cols, reinterpret_cast<uint32_t*>(scale_dev));
    hipLaunchKernelGGL(absmax_to_scale_kernel, dim3(1), dim3(1), 0, s, scale_dev);
    int ret = launch_status("tensor_absmax_kernel");
    if (ret) return ret;
    return ncnnhip_quantize(b_dev, b_stride, 0, bq_dev, bq_stride, 0, rows, cols, 1, scale_dev, 1, stream);
}

int ncnnhip_transpose_f32(const float* src_dev, size_t src_stride, int rows, int cols, float* dst_dev, size_t dst_stride, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && rows >= 1 && cols >= 1, "ncnnhip_transpose_f32: bad argument");
    dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32));
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_transpose_f32: too many rows");
    hipLaunchKernelGGL(transpose_kernel<float>, grid, dim3(256), 0, as_stream(stream), src_dev, src_stride, rows, cols, dst_dev, dst_stride);
    return launch_status("transpose_kernel<float>");
}

int ncnnhip_transpose_pair_f32(const float* src_a_dev, const float* src_b_dev, size_t src_stride, int rows, int cols, float* dst_a_dev, float* dst_b_dev,
                               size_t dst_stride, void* stream)
{
    NCNNHIP_REQUIRE(src_a_dev && src_b_dev && dst_a_dev && dst_b_dev && rows >= 1 && cols >= 1, "ncnnhip_transpose_pair_f32: bad argument");
    dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32), 2);
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_transpose_pair_f32: too many rows");
    hipLaunchKernelGGL(transpose_pair_kernel, grid, dim3(256), 0, as_stream(stream), src_a_dev, src_b_dev, src_stride, rows, cols, dst_a_dev, dst_b_dev, dst_stride);
    return launch_status("transpose_pair_kernel");
}

int ncnnhip_transpose_s8(const int8_t* src_dev, size_t src_stride, int rows, int cols, int8_t* dst_dev, size_t dst_stride, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev && rows >= 1 && cols >= 1, "ncnnhip_transpose_s8: bad argument");
    dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32));
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_transpose_s8: too many rows");
    hipLaunchKernelGGL(transpose_kernel<int8_t>, grid, dim3(256), 0, as_stream(stream), src_dev, src_stride, rows, cols, dst_dev, dst_stride);
    return launch_status("transpose_kernel<int8_t>");
}

} // extern "C"
