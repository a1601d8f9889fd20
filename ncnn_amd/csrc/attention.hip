// The attention core of MultiHeadAttention (src/layer/multiheadattention.cpp:776-866 in the block-quantised forward):
// per head  out = softmax(q k^T + mask) v  in fp32.  The four projections around it are block-quantised Gemms.
//
// Layouts: q and out are [sequence][embed_dim] (row = token); keys and values are [embed_dim][dst_seqlen], one row per
// channel over time, which is the layout the reference layer hands out and takes back as its cache.
//
// One workgroup = up to 4 query rows of one head.
//   scores : thread j owns key j, walks the head's channels in order (the reference's summation order, no FMA) reading
//            k[channel][j] coalesced; the 4 queries reuse every key value loaded
//   softmax: one wavefront per query row (max, exp, sum by shuffles), probabilities stay in LDS
//   p v    : a wavefront takes channels w, w+4, ...; lanes stride over time reading v[channel][k] coalesced, then a
//            shuffle reduction (so the sum over k is a tree, not the reference's sequence: fp32 tolerance)
#include <float.h>

#include "common.h"

namespace ncnnhip {

static constexpr int ATT_TQ = 4;

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = add_rn(v, __shfl_xor(v, o));
    return v;
}

__global__ __launch_bounds__(256) void attention_f32_kernel(const float* __restrict__ q, const float* __restrict__ kt, const float* __restrict__ vt,
                                                            const float* __restrict__ mask, int mask_heads, int head_dim, int embed_dim, int src, int dst,
                                                            size_t kv_stride, float* __restrict__ out)
{
    extern __shared__ float smem[];
    float* qs = smem;                     // [ATT_TQ][head_dim]
    float* sc = smem + ATT_TQ * head_dim; // [ATT_TQ][dst]
    const int h = blockIdx.y;
    const int i0 = blockIdx.x * ATT_TQ;
    const int rows = src - i0 < ATT_TQ ? src - i0 : ATT_TQ;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    for (int e = tid; e < ATT_TQ * head_dim; e += 256)
    {
        const int t = e / head_dim, l = e - t * head_dim;
        qs[e] = t < rows ? q[(size_t)(i0 + t) * embed_dim + h * head_dim + l] : 0.f;
    }
    __syncthreads();

    // ---- scores
    const float* kh = kt + (size_t)h * head_dim * kv_stride;
    for (int j = tid; j < dst; j += 256)
    {
        float acc[ATT_TQ];
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++) acc[t] = 0.f;
        for (int l = 0; l < head_dim; l++)
        {
            const float kv = kh[(size_t)l * kv_stride + j];
#pragma unroll
            for (int t = 0; t < ATT_TQ; t++) acc[t] = add_rn(acc[t], mul_rn(qs[t * head_dim + l], kv));
        }
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++)
        {
            float s = acc[t];
            if (mask && t < rows) s = add_rn(s, mask[((size_t)(mask_heads > 1 ? h : 0) * src + i0 + t) * dst + j]);
            sc[t * dst + j] = s;
        }
    }
    __syncthreads();

    // ---- softmax, wavefront `wave` owns query row `wave`
    {
        float* row = sc + wave * dst;
        float mx = -FLT_MAX;
        for (int j = lane; j < dst; j += 64) mx = fmaxf(mx, row[j]);
        mx = wave_max(mx);
        float total = 0.f;
        for (int j = lane; j < dst; j += 64)
        {
            const float e = expf(add_rn(row[j], -mx));
            row[j] = e;
            total = add_rn(total, e);
        }
        total = wave_sum(total);
        for (int j = lane; j < dst; j += 64) row[j] = div_rn(row[j], total);
    }
    __syncthreads();

    // ---- probabilities times values
    const float* vh = vt + (size_t)h * head_dim * kv_stride;
    for (int l = wave; l < head_dim; l += 4)
    {
        const float* vr = vh + (size_t)l * kv_stride;
        float acc[ATT_TQ];
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++) acc[t] = 0.f;
        for (int k = lane; k < dst; k += 64)
        {
            const float v = vr[k];
#pragma unroll
            for (int t = 0; t < ATT_TQ; t++) acc[t] = add_rn(acc[t], mul_rn(sc[t * dst + k], v));
        }
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++)
        {
            const float s = wave_sum(acc[t]);
            if (lane == 0 && t < rows) out[(size_t)(i0 + t) * embed_dim + h * head_dim + l] = s;
        }
    }
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_attention_f32(const float* q_dev, const float* kt_dev, const float* vt_dev, size_t kv_stride, const float* mask_dev, int mask_heads,
                          int num_heads, int head_dim, int src_seqlen, int dst_seqlen, float* out_dev, void* stream)
{
    NCNNHIP_REQUIRE(q_dev && kt_dev && vt_dev && out_dev, "ncnnhip_attention_f32: null pointer");
    NCNNHIP_REQUIRE(num_heads >= 1 && head_dim >= 1 && src_seqlen >= 1 && dst_seqlen >= 1, "ncnnhip_attention_f32: bad shape");
    NCNNHIP_REQUIRE(num_heads <= 65535, "ncnnhip_attention_f32: more than 65535 heads");
    NCNNHIP_REQUIRE(kv_stride >= (size_t)dst_seqlen, "ncnnhip_attention_f32: key/value row stride below dst_seqlen");
    NCNNHIP_REQUIRE(!mask_dev || mask_heads == 1 || mask_heads == num_heads, "ncnnhip_attention_f32: the mask is shared (1) or one per head");
    const size_t lds = (size_t)ATT_TQ * ((size_t)head_dim + (size_t)dst_seqlen) * sizeof(float);
    NCNNHIP_REQUIRE(lds <= 65536, "ncnnhip_attention_f32: head_dim + dst_seqlen = %d exceeds the 4096 this kernel keeps in LDS", head_dim + dst_seqlen);
    dim3 grid((unsigned)((src_seqlen + ATT_TQ - 1) / ATT_TQ), (unsigned)num_heads);
    hipLaunchKernelGGL(attention_f32_kernel, grid, dim3(256), lds, as_stream(stream), q_dev, kt_dev, vt_dev, mask_dev, mask_dev ? mask_heads : 0, head_dim,
                       num_heads * head_dim, src_seqlen, dst_seqlen, kv_stride, out_dev);
    return launch_status("attention_f32_kernel");
}

} // extern "C"
