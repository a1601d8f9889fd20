// Weight-only block-quantised Gemm: out[i][j] = alpha*(beta*C + sum_k a[i][k]*s_in[k] * (q[j][k] * (1/scale[j][k/block]))).
// The weights are streamed from HBM exactly once; this is a bandwidth kernel (no matrix cores):
// one wavefront owns one weight row, every lane pulls 16 weight bytes per step, partial sums are
// combined with cross-lane adds.  Products are formed as a*(q*descale) like the reference; the
// order of the fp32 additions differs from the reference's single sequential sum, which is why
// this output is compared with a relative tolerance and not bit-for-bit.
#include <hip/hip_fp16.h>

#include "common.h"

namespace ncnnhip {

typedef int v4i_bq __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = add_rn(v, __shfl_xor(v, o, 64));
    return v;
}

__device__ __forceinline__ float load_c(const float* c, int bt, int i, int j, int N)
{
    if (bt == 0) return c[0];
    if (bt == 1 || bt == 2) return c[i];
    if (bt == 3) return c[(size_t)i * N + j];
    return c[j];
}

__device__ __forceinline__ float to_f32(float v)
{
    return v;
}
__device__ __forceinline__ float to_f32(__half v)
{
    return __half2float(v);
}

// ---- 8-bit weights, K % 16 == 0, 16-byte aligned rows ------------------------------------
template<typename AT, int MB>
__global__ __launch_bounds__(256) void blockquant8_kernel(const AT* __restrict__ a, size_t a_stride, int M, int N, int K,
                                                           const int8_t* __restrict__ b, int block_shift, int nblk,
                                                           const float* __restrict__ scales, const float* __restrict__ in_scales,
                                                           const float* __restrict__ c, int bt, float alpha, float beta,
                                                           float* __restrict__ out, size_t out_stride)
{
    const int lane = threadIdx.x & 63;
    const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (j >= N) return;
    const int8_t* br = b + (size_t)j * K;
    const float* sr = scales + (size_t)j * nblk;

    for (int i0 = 0; i0 < M; i0 += MB)
    {
        float sum[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) sum[m] = 0.f;

        for (int k = lane * 16; k < K; k += 64 * 16)
        {
            const v4i_bq wv = *reinterpret_cast<const v4i_bq*>(br + k);
            const float descale = div_rn(1.f, sr[k >> block_shift]);
            float wf[16];
#pragma unroll
            for (int t = 0; t < 16; t++) wf[t] = mul_rn((float)(int)(int8_t)(wv[t >> 2] >> ((t & 3) * 8)), descale);
#pragma unroll
            for (int m = 0; m < MB; m++)
            {
                if (i0 + m < M)
                {
                    const AT* ar = a + (size_t)(i0 + m) * a_stride + k;
#pragma unroll
                    for (int t = 0; t < 16; t++)
                    {
                        float v = to_f32(ar[t]);
                        if (in_scales) v = mul_rn(v, in_scales[k + t]);
                        sum[m] = add_rn(sum[m], mul_rn(v, wf[t]));
                    }
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MB; m++)
        {
            const float total = wave_sum(sum[m]);
            if (lane == 0 && i0 + m < M)
            {
                float f = total;
                if (bt >= 0) f = add_rn(mul_rn(load_c(c, bt, i0 + m, j, N), beta), f);
                out[(size_t)(i0 + m) * out_stride + j] = mul_rn(f, alpha);
            }
        }
    }
}

// ---- any bits / block / alignment --------------------------------------------------------
__device__ __forceinline__ int unpack_field(const uint8_t* row, int k, int bits, int packed_k_bytes)
{
    const int bit = k * bits;
    const int byte = bit >> 3;
    unsigned v = row[byte];
    if (byte + 1 < packed_k_bytes) v |= (unsigned)row[byte + 1] << 8;
    const int field = (int)((v >> (bit & 7)) & ((1u << bits) - 1u));
    const int sign = 1 << (bits - 1);
    return (field ^ sign) - sign;
}

__global__ __launch_bounds__(256) void blockquant_generic_kernel(const float* __restrict__ a, size_t a_stride, int M, int N, int K,
                                                                  const uint8_t* __restrict__ b, int bits, int block, int packed_k_bytes,
                                                                  int nblk, const float* __restrict__ scales,
                                                                  const float* __restrict__ in_scales, const float* __restrict__ c, int bt,
                                                                  float alpha, float beta, float* __restrict__ out, size_t out_stride)
{
    const int lane = threadIdx.x & 63;
    const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (j >= N) return;
    const uint8_t* br = b + (size_t)j * packed_k_bytes;
    const float* sr = scales + (size_t)j * nblk;
    for (int i = 0; i < M; i++)
    {
        const float* ar = a + (size_t)i * a_stride;
        float sum = 0.f;
        for (int k = lane; k < K; k += 64)
        {
            const float descale = div_rn(1.f, sr[k / block]);
            const int q = unpack_field(br, k, bits, packed_k_bytes);
            float v = ar[k];
            if (in_scales) v = mul_rn(v, in_scales[k]);
            sum = add_rn(sum, mul_rn(v, mul_rn((float)q, descale)));
        }
        const float total = wave_sum(sum);
        if (lane == 0)
        {
            float f = total;
            if (bt >= 0) f = add_rn(mul_rn(load_c(c, bt, i, j, N), beta), f);
            out[(size_t)i * out_stride + j] = mul_rn(f, alpha);
        }
    }
}

static int check_blockquant(const void* a, const void* b, const void* scales, const void* out, int M, int N, int K, int bits, int block,
                            const void* c, int bt)
{
    NCNNHIP_REQUIRE(a && b && scales && out, "ncnnhip_gemm_blockquant: null pointer");
    NCNNHIP_REQUIRE(M >= 1 && N >= 1 && K >= 1, "ncnnhip_gemm_blockquant: bad shape %d %d %d", M, N, K);
    NCNNHIP_REQUIRE(bits == 4 || bits == 6 || bits == 8, "ncnnhip_gemm_blockquant: weight bits %d", bits);
    NCNNHIP_REQUIRE(block == 32 || block == 64 || block == 128, "ncnnhip_gemm_blockquant: block size %d", block);
    NCNNHIP_REQUIRE(bt >= -1 && bt <= 4 && (bt < 0 || c), "ncnnhip_gemm_blockquant: C broadcast %d", bt);
    return NCNNHIP_OK;
}

static inline bool al16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_gemm_blockquant(const float* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* b_dev, int bits, int block,
                            const float* scales_dev, const float* in_scales_dev, const float* c_dev, int broadcast_type_c,
                            float alpha, float beta, float* out_dev, size_t out_stride, void* stream)
{
    const int bt = c_dev ? broadcast_type_c : -1;
    int ret = check_blockquant(a_dev, b_dev, scales_dev, out_dev, M, N, K, bits, block, c_dev, bt);
    if (ret) return ret;
    NCNNHIP_REQUIRE(a_stride >= (size_t)K && out_stride >= (size_t)N, "ncnnhip_gemm_blockquant: stride too small");
    const int nblk = (K + block - 1) / block;
    dim3 grid(ceil_div(N, 4));
    if (bits == 8 && K % 16 == 0 && al16(b_dev))
    {
        const int shift = block == 32 ? 5 : block == 64 ? 6 : 7;
        const int8_t* b8 = reinterpret_cast<const int8_t*>(b_dev);
        if (M == 1)
            hipLaunchKernelGGL((blockquant8_kernel<float, 1>), grid, dim3(256), 0, as_stream(stream), a_dev, a_stride, M, N, K, b8, shift, nblk,
                               scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride);
        else
            hipLaunchKernelGGL((blockquant8_kernel<float, 4>), grid, dim3(256), 0, as_stream(stream), a_dev, a_stride, M, N, K, b8, shift, nblk,
                               scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride);
        return launch_status("blockquant8_kernel");
    }
    const int packed = (int)(((size_t)K * bits + 7) / 8);
    hipLaunchKernelGGL(blockquant_generic_kernel, grid, dim3(256), 0, as_stream(stream), a_dev, a_stride, M, N, K, b_dev, bits, block, packed,
                       nblk, scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride);
    return launch_status("blockquant_generic_kernel");
}

int ncnnhip_gemm_blockquant_f16a(const uint16_t* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* b_dev, int bits,
                                 int block, const float* scales_dev, float* out_dev, size_t out_stride, void* stream)
{
    int ret = check_blockquant(a_dev, b_dev, scales_dev, out_dev, M, N, K, bits, block, 0, -1);
    if (ret) return ret;
    NCNNHIP_REQUIRE(bits == 8 && K % 16 == 0 && al16(b_dev), "ncnnhip_gemm_blockquant_f16a: needs 8-bit weights, K %% 16 == 0, aligned rows");
    NCNNHIP_REQUIRE(a_stride >= (size_t)K && out_stride >= (size_t)N, "ncnnhip_gemm_blockquant_f16a: stride too small");
    const int nblk = (K + block - 1) / block;
    const int shift = block == 32 ? 5 : block == 64 ? 6 : 7;
    dim3 grid(ceil_div(N, 4));
    const __half* ah = reinterpret_cast<const __half*>(a_dev);
    const int8_t* b8 = reinterpret_cast<const int8_t*>(b_dev);
    if (M == 1)
        hipLaunchKernelGGL((blockquant8_kernel<__half, 1>), grid, dim3(256), 0, as_stream(stream), ah, a_stride, M, N, K, b8, shift, nblk, scales_dev,
                           (const float*)0, (const float*)0, -1, 1.f, 1.f, out_dev, out_stride);
    else
        hipLaunchKernelGGL((blockquant8_kernel<__half, 4>), grid, dim3(256), 0, as_stream(stream), ah, a_stride, M, N, K, b8, shift, nblk, scales_dev,
                           (const float*)0, (const float*)0, -1, 1.f, 1.f, out_dev, out_stride);
    return launch_status("blockquant8_kernel<half>");
}

} // extern "C"
