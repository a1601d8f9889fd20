// Weight-only block-quantised Gemm: out[i][j] = alpha*(beta*C + sum_k a[i][k]*s_in[k] * (q[j][k] * (1/scale[j][k/block]))).
// The weights are streamed from HBM exactly once; this is a bandwidth kernel (no matrix cores):
// one wavefront owns one weight row, every lane pulls 16 weight bytes per step, partial sums are
// combined with cross-lane adds.  Products are formed as a*(q*descale) like the reference; the
// order of the fp32 additions differs from the reference's single sequential sum, which is why
// this output is compared with a relative tolerance and not bit-for-bit.
#include <hip/hip_fp16.h>
#include <string.h>

#include <atomic>

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
// Streaming kernel for up to MT activation rows at a time.
//   * the activations (times the optional input scales) are staged once per workgroup in LDS as
//     fp32, in K tiles of KT = 8192 / MT values;
//   * every wavefront owns R consecutive weight rows; per row each lane fetches 16-byte chunks
//     lane, lane+64, ... of the K tile, U chunks per batch, and all R*U 16-byte loads of a batch
//     are issued before the first one is consumed, which is what keeps enough bytes in flight to
//     cover HBM latency;
//   * a chunk never straddles a quantisation block (block >= 32), so the 16 products of a chunk
//     are summed first and the block's 1/scale is applied once per chunk.
// BITS = 4 / 6 / 8: a chunk is always 16 weights, i.e. 8 / 12 / 16 bytes of the LSB-first field stream
// (src/layer/gemm.cpp:318-336); a field is pulled out of its dword pair with one funnel shift + one signed bit-field extract.
#ifndef BQ_R
#define BQ_R 2
#endif
#ifndef BQ_U
#define BQ_U 2 // chunks per row and batch; with 32 KB of LDS this keeps three workgroups on a CU (measured over R 1..4, U 1..4, 16/32/64 KB)
#endif
#ifndef BQ_KT
#define BQ_KT 8192
#endif
template<int BITS>
__device__ __forceinline__ v4i_bq load_chunk(const uint8_t* p)
{
    v4i_bq w = {0, 0, 0, 0};
    // non-temporal: the weights are read once per Gemm
    if (BITS == 8)
        w = __builtin_nontemporal_load(reinterpret_cast<const v4i_bq*>(p));
    else if (BITS == 6)
    {
        const int* q = reinterpret_cast<const int*>(p);
        w[0] = __builtin_nontemporal_load(q);
        w[1] = __builtin_nontemporal_load(q + 1);
        w[2] = __builtin_nontemporal_load(q + 2);
    }
    else
    {
        typedef int v2i_bq __attribute__((ext_vector_type(2)));
        const v2i_bq t = __builtin_nontemporal_load(reinterpret_cast<const v2i_bq*>(p));
        w[0] = t[0];
        w[1] = t[1];
    }
    return w;
}
template<int BITS>
__device__ __forceinline__ float chunk_field(const v4i_bq& w, int t)
{
    const int bit = t * BITS, d = bit >> 5, sh = bit & 31;
    unsigned lo = (unsigned)w[d];
    if (sh + BITS > 32) lo = __funnelshift_r(lo, (unsigned)w[d + 1], sh); // the field straddles two dwords (6-bit only)
    const int v = sh + BITS > 32 ? (int)lo : (int)(lo >> sh);
    return (float)((v << (32 - BITS)) >> (32 - BITS));
}

template<typename AT, int MT, int R, int U, int BITS>
__global__ __launch_bounds__(256) void blockquant8_stream_kernel(const AT* __restrict__ a, size_t a_stride, int m0, int M, int N, int K,
                                                                  const uint8_t* __restrict__ b, int block_shift, int nblk,
                                                                  const float* __restrict__ scales, const float* __restrict__ in_scales,
                                                                  const float* __restrict__ c, int bt, float alpha, float beta,
                                                                  float* __restrict__ out, size_t out_stride)
{
    constexpr int KT = BQ_KT / MT; // activation tile in LDS: BQ_KT floats
    __shared__ __attribute__((aligned(16))) float lds_a[MT * KT];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j0 = (blockIdx.x * 4 + wave) * R;
    const int mcount = M - m0 < MT ? M - m0 : MT;
    const size_t row_bytes = (size_t)K * BITS / 8; // K % 16 == 0

    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MT; m++) acc[r][m] = 0.f;

    // A "batch" is R*U chunks per lane: rows j0..j0+R-1, chunks c0 + u*64 + lane of K tile kt0.
    // Weight batches do not depend on LDS, so batch n+1 is always requested before batch n is
    // multiplied, and the very first batch is requested before the activations are staged.
    auto load_batch = [&](int kt0, int c0, v4i_bq (&w)[R][U], float (&d)[R][U]) {
        const int kt = K - kt0 < KT ? K - kt0 : KT;
        const int nch = kt >> 4;
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                // unconditional loads from clamped addresses, zeros selected afterwards: a guarded load becomes a branch,
                // and past a branch the compiler waits for every load in flight
                const int ch = c0 + u * 64 + lane;
                const int j = j0 + r;
                const bool ok = ch < nch && j < N;
                const size_t jc = (size_t)(j < N ? j : N - 1);
                const size_t koff = (size_t)kt0 + ((size_t)(ch < nch ? ch : 0) << 4);
                v4i_bq wv = load_chunk<BITS>(b + jc * row_bytes + koff * BITS / 8);
                if (!ok) wv = v4i_bq{0, 0, 0, 0};
                w[r][u] = wv;
                d[r][u] = scales[jc * nblk + (koff >> block_shift)];
            }
    };
    auto compute_batch = [&](int kt0, int c0, const v4i_bq (&w)[R][U], const float (&d)[R][U]) {
        const int kt = K - kt0 < KT ? K - kt0 : KT;
        const int nch = kt >> 4;
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const int ch = c0 + u * 64 + lane;
            if (ch < nch)
            {
                float av[MT][16];
#pragma unroll
                for (int m = 0; m < MT; m++)
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++)
                    {
                        const float4 t4 = *reinterpret_cast<const float4*>(&lds_a[m * KT + (ch << 4) + q4 * 4]);
                        av[m][q4 * 4 + 0] = t4.x;
                        av[m][q4 * 4 + 1] = t4.y;
                        av[m][q4 * 4 + 2] = t4.z;
                        av[m][q4 * 4 + 3] = t4.w;
                    }
#pragma unroll
                for (int r = 0; r < R; r++)
                {
                    float part[MT];
#pragma unroll
                    for (int m = 0; m < MT; m++) part[m] = 0.f;
#pragma unroll
                    for (int t = 0; t < 16; t++)
                    {
                        const float q = chunk_field<BITS>(w[r][u], t);
#pragma unroll
                        for (int m = 0; m < MT; m++) part[m] = fmaf(av[m][t], q, part[m]);
                    }
                    const float descale = div_rn(1.f, d[r][u]);
#pragma unroll
                    for (int m = 0; m < MT; m++) acc[r][m] = fmaf(part[m], descale, acc[r][m]);
                }
            }
        }
    };
    auto stage_tile = [&](int kt0) {
        const int kt = K - kt0 < KT ? K - kt0 : KT;
        for (int m = 0; m < MT; m++)
        {
            const bool live = m < mcount;
            const AT* arow = a + (size_t)(m0 + (live ? m : 0)) * a_stride + kt0;
            constexpr int VEC = 16 / (int)sizeof(AT);
            const bool vec_ok = (reinterpret_cast<uintptr_t>(arow) & 15) == 0;
            if (vec_ok)
            {
                const int nvec = kt / VEC; // kt % 16 == 0
#pragma unroll 4
                for (int v = threadIdx.x; v < nvec; v += 256)
                {
                    float tmp[VEC];
                    if (live)
                    {
                        const v4i_bq raw = *reinterpret_cast<const v4i_bq*>(arow + v * VEC);
                        if (sizeof(AT) == 4)
                        {
#pragma unroll
                            for (int e = 0; e < 4; e++) tmp[e] = __int_as_float(raw[e]);
                        }
                        else
                        {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                            {
                                tmp[(2 * e) % VEC] = __half2float(__ushort_as_half((unsigned short)(raw[e] & 0xffff)));
                                tmp[(2 * e + 1) % VEC] = __half2float(__ushort_as_half((unsigned short)((unsigned)raw[e] >> 16)));
                            }
                        }
                        if (in_scales)
                        {
#pragma unroll
                            for (int e = 0; e < VEC; e++) tmp[e] = mul_rn(tmp[e], in_scales[kt0 + v * VEC + e]);
                        }
                    }
                    else
                    {
#pragma unroll
                        for (int e = 0; e < VEC; e++) tmp[e] = 0.f;
                    }
#pragma unroll
                    for (int e = 0; e < VEC; e += 4)
                        *reinterpret_cast<float4*>(&lds_a[m * KT + v * VEC + e]) = make_float4(tmp[e], tmp[e + 1], tmp[e + 2], tmp[e + 3]);
                }
            }
            else
            {
                for (int k = threadIdx.x; k < kt; k += 256)
                {
                    float v = 0.f;
                    if (live)
                    {
                        v = to_f32(arow[k]);
                        if (in_scales) v = mul_rn(v, in_scales[kt0 + k]);
                    }
                    lds_a[m * KT + k] = v;
                }
            }
        }
    };

    v4i_bq w0[R][U], w1[R][U];
    float d0[R][U], d1[R][U];
    load_batch(0, 0, w0, d0);
    for (int kt0 = 0; kt0 < K; kt0 += KT)
    {
        const int kt = K - kt0 < KT ? K - kt0 : KT;
        const int nch = kt >> 4;
        if (kt0) __syncthreads(); // everyone is done with the previous activation tile
        stage_tile(kt0);
        __syncthreads();
        // batches of this tile, two per trip so the two register sets alternate statically
        for (int c0 = 0; c0 < nch; c0 += 2 * 64 * U)
        {
            const int c1 = c0 + 64 * U;
            const int c2 = c1 + 64 * U;
            if (c1 < nch)
                load_batch(kt0, c1, w1, d1);
            else if (kt0 + KT < K)
                load_batch(kt0 + KT, 0, w1, d1);
            compute_batch(kt0, c0, w0, d0);
            if (c1 < nch)
            {
                if (c2 < nch)
                    load_batch(kt0, c2, w0, d0);
                else if (kt0 + KT < K)
                    load_batch(kt0 + KT, 0, w0, d0);
                compute_batch(kt0, c1, w1, d1);
            }
            else if (kt0 + KT < K)
            {
                // the prefetched first batch of the next tile sits in set 1: move it to set 0
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int u = 0; u < U; u++)
                    {
                        w0[r][u] = w1[r][u];
                        d0[r][u] = d1[r][u];
                    }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MT; m++)
        {
            const float total = wave_sum(acc[r][m]);
            const int j = j0 + r;
            if (lane == 0 && j < N && m < mcount)
            {
                float f = total;
                if (bt >= 0) f = add_rn(mul_rn(load_c(c, bt, m0 + m, j, N), beta), f);
                out[(size_t)(m0 + m) * out_stride + j] = mul_rn(f, alpha);
            }
        }
}

template<typename AT, int BITS = 8>
static int launch_blockquant8(const AT* a, size_t a_stride, int M, int N, int K, const uint8_t* b8, int block, const float* scales,
                              const float* in_scales, const float* c, int bt, float alpha, float beta, float* out, size_t out_stride,
                              hipStream_t stream)
{
    const int shift = block == 32 ? 5 : block == 64 ? 6 : 7;
    const int nblk = (K + block - 1) / block;
    constexpr int R = BQ_R, U = BQ_U;
    dim3 grid(ceil_div(N, 4 * R));
    for (int m0 = 0; m0 < M;)
    {
        const int left = M - m0;
        if (left >= 4)
        {
            hipLaunchKernelGGL((blockquant8_stream_kernel<AT, 4, R, U, BITS>), grid, dim3(256), 0, stream, a, a_stride, m0, M, N, K, b8, shift, nblk, scales,
                               in_scales, c, bt, alpha, beta, out, out_stride);
            m0 += 4;
        }
        else if (left >= 2)
        {
            hipLaunchKernelGGL((blockquant8_stream_kernel<AT, 2, R, U, BITS>), grid, dim3(256), 0, stream, a, a_stride, m0, M, N, K, b8, shift, nblk, scales,
                               in_scales, c, bt, alpha, beta, out, out_stride);
            m0 += 2;
        }
        else
        {
            hipLaunchKernelGGL((blockquant8_stream_kernel<AT, 1, R, U, BITS>), grid, dim3(256), 0, stream, a, a_stride, m0, M, N, K, b8, shift, nblk, scales,
                               in_scales, c, bt, alpha, beta, out, out_stride);
            m0 += 1;
        }
    }
    return launch_status("blockquant8_stream_kernel");
}

// ---- 8-bit weights, many activation rows: fp32 matrix cores -----------------------------------
// From 32 rows up streaming the weights once per 4 rows is the wrong shape; this kernel tiles 64 activation rows by 64
// weight rows per workgroup (4 wavefronts, 32x32 each) and multiplies on v_mfma_f32_32x32x2_f32.  The B operand is the
// weight as the reference forms it, (float)q * (1/scale), so every product is the reference's fp32 product; only the
// order of the fp32 additions differs.  K in tiles of 32 through two LDS buffers (row stride 33 floats: a column of 32
// rows hits 32 banks); the next tile's global loads are issued before the current tile's MFMAs.
typedef float v16f_bq __attribute__((ext_vector_type(16)));
typedef float v4f_bq __attribute__((ext_vector_type(4)));

template<int BITS>
__global__ __launch_bounds__(256) void blockquant8_f32_mfma_kernel(const float* __restrict__ a, size_t a_stride, int M, int N, int K,
                                                                   const uint8_t* __restrict__ b, int block_shift, int nblk, const float* __restrict__ scales,
                                                                   const float* __restrict__ in_scales, const float* __restrict__ c, int bt, float alpha,
                                                                   float beta, float* __restrict__ out, size_t out_stride)
{
    constexpr int LD = 33;
    __shared__ float sa[2][64 * LD];
    __shared__ float sb[2][64 * LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int row0 = blockIdx.y * 64, col0 = blockIdx.x * 64;

    // loader role: row tid/4 of the tile, 8 consecutive k starting at (tid%4)*8
    const int lr = tid >> 2, lk = (tid & 3) * 8;
    const int arow = row0 + lr < M ? row0 + lr : M - 1; // rows past the end repeat the last one; their results are not stored
    const int brow = col0 + lr < N ? col0 + lr : N - 1;
    const float* ap = a + (size_t)arow * a_stride + lk;
    // the loader's 8 weights are BITS bytes of the field stream (2-byte aligned for 6-bit: three halfword loads)
    const uint8_t* bp = b + (size_t)brow * ((size_t)K * BITS / 8) + (size_t)lk * BITS / 8;
    const float* sp = scales + (size_t)brow * nblk;

    v4f_bq a0, a1;
    unsigned long long bq;
    float descale;
    auto fetch = [&](int k0) {
        a0 = *reinterpret_cast<const v4f_bq*>(ap + k0);
        a1 = *reinterpret_cast<const v4f_bq*>(ap + k0 + 4);
        const uint8_t* wp = bp + (size_t)k0 * BITS / 8;
        if (BITS == 8)
        {
            const uint2 t = *reinterpret_cast<const uint2*>(wp);
            bq = (unsigned long long)t.x | ((unsigned long long)t.y << 32);
        }
        else if (BITS == 6)
        {
            const unsigned short* hp = reinterpret_cast<const unsigned short*>(wp);
            bq = (unsigned long long)hp[0] | ((unsigned long long)hp[1] << 16) | ((unsigned long long)hp[2] << 32);
        }
        else
            bq = *reinterpret_cast<const unsigned*>(wp);
        descale = div_rn(1.f, sp[(k0 + lk) >> block_shift]);
        if (in_scales)
        {
            const v4f_bq s0 = *reinterpret_cast<const v4f_bq*>(in_scales + k0 + lk), s1 = *reinterpret_cast<const v4f_bq*>(in_scales + k0 + lk + 4);
#pragma unroll
            for (int e = 0; e < 4; e++)
            {
                a0[e] = mul_rn(a0[e], s0[e]);
                a1[e] = mul_rn(a1[e], s1[e]);
            }
        }
    };
    auto stage = [&](int buf) {
        float* pa = &sa[buf][lr * LD + lk];
        float* pb = &sb[buf][lr * LD + lk];
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            pa[e] = a0[e];
            pa[4 + e] = a1[e];
            pb[e] = mul_rn((float)(((int)(unsigned)(bq >> (BITS * e)) << (32 - BITS)) >> (32 - BITS)), descale);
            pb[4 + e] = mul_rn((float)(((int)(unsigned)(bq >> (BITS * (4 + e))) << (32 - BITS)) >> (32 - BITS)), descale);
        }
    };

    v16f_bq acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;

    const int ntiles = K / 32;
    fetch(0);
    stage(0);
    __syncthreads();
    const int l32 = lane & 31, lhi = lane >> 5;
    for (int t = 0; t < ntiles; t++)
    {
        const int buf = t & 1;
        if (t + 1 < ntiles) fetch((t + 1) * 32);
        const float* pa = &sa[buf][(wm * 32 + l32) * LD + lhi];
        const float* pb = &sb[buf][(wn * 32 + l32) * LD + lhi];
#pragma unroll
        for (int kk = 0; kk < 16; kk++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[2 * kk], pb[2 * kk], acc, 0, 0, 0);
        if (t + 1 < ntiles) stage(buf ^ 1); // the other buffer: its readers finished before the barrier that ended tile t-1
        __syncthreads();
    }

    // accumulator register r of lane l: activation row 8*(r/4) + 4*(l/32) + r%4, weight row l%32
    const int j = col0 + wn * 32 + l32;
#pragma unroll
    for (int r = 0; r < 16; r++)
    {
        const int i = row0 + wm * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
        if (i < M && j < N)
        {
            float v = acc[r];
            if (bt >= 0) v = add_rn(mul_rn(load_c(c, bt, i, j, N), beta), v);
            out[(size_t)i * out_stride + j] = mul_rn(v, alpha);
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

// ---- matrix-core streaming kernel for packed 8-bit weights, up to 16 activation rows -------
// Packed layout (made once when the weights are uploaded):
//   weights   [ceil(N/16)][ceil(K/64)][64 lanes][16 bytes]: lane l of a tile holds row l%16,
//             K offsets (l/16)*16 .. +15 of the 64-wide K block, each byte stored as q+128;
//   descales  [ceil(N/16)][ceil(K/64)][16] fp32 = 1/scale of that row for that K block.
// A workgroup owns 16 weight rows; its 4 wavefronts split K.  Per K block a lane issues one
// 16-byte weight load, one 16-byte descale load and two 16-byte activation loads (fp16, straight
// from L2), turns the 16 bytes into 16 halves with byte permutes (0x6400|u is the half 1024+u,
// minus 1152 gives q exactly), and runs two v_mfma_f32_16x16x32_f16: rows = weight rows,
// columns = activation rows.  Integer-valued q times an fp16 activation is exact in fp32, so the
// only roundings are the fp32 accumulation and the one multiply by 1/scale per K block.
#ifndef BQ_MFMA_U
#define BQ_MFMA_U 1 // NS x U = 4 x 1: ~100 VGPRs, four wavefronts per SIMD (measured best of 2..8 x 1..4; see the load_batch comment)
#endif
#ifndef BQ_MFMA_NS
#define BQ_MFMA_NS 4
#endif
#ifndef BQ_MFMA_NS_LDS
#define BQ_MFMA_NS_LDS 4 // ring depth when the activations are staged in LDS (4..12 measured)
#endif
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

__device__ __forceinline__ v8h bytes_to_halves(int lo, int hi)
{
    // lo, hi: 8 bytes u0..u7 (u = q + 128).  Build halves 0x6400|u = 1024+u, then subtract 1152.
    union
    {
        int i[4];
        v2h h2[4];
        v8h h8;
    } t;
    t.i[0] = __builtin_amdgcn_perm(0x64646464, lo, 0x04010400);
    t.i[1] = __builtin_amdgcn_perm(0x64646464, lo, 0x04030402);
    t.i[2] = __builtin_amdgcn_perm(0x64646464, hi, 0x04010400);
    t.i[3] = __builtin_amdgcn_perm(0x64646464, hi, 0x04030402);
    const v2h off = {(_Float16)1152.f, (_Float16)1152.f};
#pragma unroll
    for (int e = 0; e < 4; e++) t.h2[e] = t.h2[e] - off;
    return t.h8;
}

// 8 nibbles u = q + 8; nibbles p and p + 4 of the dword are the two halves of pair p, so one mask serves both.
__device__ __forceinline__ v8h nibbles_to_halves(unsigned w)
{
    union
    {
        unsigned i[4];
        v2h h2[4];
        v8h h8;
    } t;
#pragma unroll
    for (int p = 0; p < 4; p++) t.i[p] = ((w >> (4 * p)) & 0x000F000Fu) | 0x64006400u; // halves 1024 + u
    const v2h off = {(_Float16)1032.f, (_Float16)1032.f};
#pragma unroll
    for (int e = 0; e < 4; e++) t.h2[e] = t.h2[e] - off;
    return t.h8;
}

// 16 six-bit fields u = q + 32 in three dwords.  A dword carries two whole pairs (the low-half field at bit 0 or 6,
// the high-half field 16 bits above) and, in bits 12-15 / 28-31, a third of a pair: pairs 6 and 7 have their low four
// bits in dword 0 / dword 1 and their high two bits side by side in dword 2.
__device__ __forceinline__ void sixbit_to_halves(unsigned d0, unsigned d1, unsigned d2, v8h& wa, v8h& wb)
{
    union
    {
        unsigned i[4];
        v2h h2[4];
        v8h h8;
    } a, b;
    const unsigned magic = 0x64006400u;
    a.i[0] = (d0 & 0x003F003Fu) | magic;
    a.i[1] = ((d0 >> 6) & 0x003F003Fu) | magic;
    a.i[2] = (d1 & 0x003F003Fu) | magic;
    a.i[3] = ((d1 >> 6) & 0x003F003Fu) | magic;
    b.i[0] = (d2 & 0x003F003Fu) | magic;
    b.i[1] = ((d2 >> 6) & 0x003F003Fu) | magic;
    b.i[2] = ((d0 >> 12) & 0x000F000Fu) | (((d2 >> 8) & 0x00300030u) | magic);
    b.i[3] = ((d1 >> 12) & 0x000F000Fu) | (((d2 >> 10) & 0x00300030u) | magic);
    const v2h off = {(_Float16)1056.f, (_Float16)1056.f};
#pragma unroll
    for (int e = 0; e < 4; e++)
    {
        a.h2[e] = a.h2[e] - off;
        b.h2[e] = b.h2[e] - off;
    }
    wa = a.h8;
    wb = b.h8;
}

// LDSA: the (few) activation rows are staged once per workgroup in LDS, zero-filled to a multiple of 64, instead of
// travelling with every batch in registers: a batch is then 4 VGPRs per block and the ring can be twice as deep at the same
// occupancy.  Used while M rows of K halves fit in 32 KB (decoding: M = 1..4 at K = 4096) and there are many tiles.
template<int NS, int U, bool LDSA>
__global__ __launch_bounds__(256) void blockquant8_mfma_kernel(const __half* __restrict__ a, size_t a_stride, int M, int N, int K, int kblocks,
                                                                const v4i_bq* __restrict__ wpk, const float4* __restrict__ dpk,
                                                                const float* __restrict__ c, int bt, float alpha, float beta,
                                                                float* __restrict__ out, size_t out_stride)
{
    extern __shared__ __attribute__((aligned(16))) float4 lds_d[]; // descales of this tile: [kblocks][4] float4
    __shared__ float red[4][64][4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tile = blockIdx.x;
    const int m = lane & 15;
    const int kg = lane >> 4; // K group of this lane inside a 64-wide block

    // K blocks of this wave
    const int per_wave = (kblocks + 3) >> 2;
    const int kb_begin = wave * per_wave;
    const int kb_end = kb_begin + per_wave < kblocks ? kb_begin + per_wave : kblocks;
    const int nkb = kb_end > kb_begin ? kb_end - kb_begin : 0;
    auto block_of = [&](int i) { return kb_begin + i; }; // i-th block this wave processes (callers pass i < nkb, else block 0)

    const v4i_bq* wt = wpk + ((size_t)tile * kblocks) * 64 + lane;
    const __half* arow = a + (size_t)(m < M ? m : 0) * a_stride + kg * 16;

    // Requests are issued in the order their data is consumed (loads return in order): the tile's
    // descales, then per batch the activations (L2) followed by the weights (the HBM stream).  NS
    // batches of U blocks are in flight in a ring of register sets, so the arithmetic of one small
    // batch runs while the following ones are still arriving and little work is left once the last
    // bytes land.
    struct Batch
    {
        v4i_bq w[U], a0[LDSA ? 1 : U], a1[LDSA ? 1 : U];
    };
    const int Kp = kblocks * 64;
    const __half* lds_act = reinterpret_cast<const __half*>(lds_d + (size_t)kblocks * 4) + (size_t)(m < M ? m : 0) * Kp + kg * 16;
    // Every load is unconditional (a guarded load becomes a branch, and after a branch the compiler waits for ALL loads in
    // flight, which empties the ring every step): a batch beyond the range re-reads the wave's first block and is cancelled
    // by a zero descale; a lane whose 16-half chunk lies beyond K (only when K % 64 != 0) reads chunk 0 and selects zeros;
    // lanes of activation rows >= M read row 0 and their results are never stored.
    auto load_batch = [&](int kb0, Batch& bt_) {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const bool live = kb0 + u < nkb;
            const int kb = live ? block_of(kb0 + u) : 0;
            if (LDSA) continue; // activations wait in LDS
            const bool aok = kb * 64 + kg * 16 < K; // K % 16 == 0: a 16-half chunk is all in or all out
            const __half* ap = arow + (aok ? (size_t)kb * 64 : (size_t)0) - (aok ? 0 : kg * 16);
            bt_.a0[LDSA ? 0 : u] = *reinterpret_cast<const v4i_bq*>(ap);
            bt_.a1[LDSA ? 0 : u] = *reinterpret_cast<const v4i_bq*>(ap + 8);
            if (K & 63)
            {
#pragma unroll
                for (int e = 0; e < 4; e++)
                {
                    bt_.a0[LDSA ? 0 : u][e] = aok ? bt_.a0[LDSA ? 0 : u][e] : 0;
                    bt_.a1[LDSA ? 0 : u][e] = aok ? bt_.a1[LDSA ? 0 : u][e] : 0;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const bool live = kb0 + u < nkb;
            const int kb = live ? block_of(kb0 + u) : 0;
            bt_.w[u] = __builtin_nontemporal_load(wt + (size_t)kb * 64); // read once: no need to keep the line (4-5 % faster)
        }
    };
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](int kb0, const Batch& bt_) {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const bool live = kb0 + u < nkb;
            const int kb = live ? block_of(kb0 + u) : 0;
            const v8h wa = bytes_to_halves(bt_.w[u][0], bt_.w[u][1]);
            const v8h wb = bytes_to_halves(bt_.w[u][2], bt_.w[u][3]);
            union
            {
                v4i_bq i;
                v8h h;
            } xa, xb;
            if (LDSA)
            {
                xa.i = *reinterpret_cast<const v4i_bq*>(lds_act + (size_t)kb * 64);
                xb.i = *reinterpret_cast<const v4i_bq*>(lds_act + (size_t)kb * 64 + 8);
            }
            else
            {
                xa.i = bt_.a0[LDSA ? 0 : u];
                xb.i = bt_.a1[LDSA ? 0 : u];
            }
            v4f t = {0.f, 0.f, 0.f, 0.f};
            t = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, xa.h, t, 0, 0, 0);
            t = __builtin_amdgcn_mfma_f32_16x16x32_f16(wb, xb.h, t, 0, 0, 0);
            float4 d = lds_d[kb * 4 + kg];
            if (!live) d = make_float4(0.f, 0.f, 0.f, 0.f); // a select, not a branch
            acc[0] = fmaf(t[0], d.x, acc[0]);
            acc[1] = fmaf(t[1], d.y, acc[1]);
            acc[2] = fmaf(t[2], d.z, acc[2]);
            acc[3] = fmaf(t[3], d.w, acc[3]);
        }
    };

    // descales of the whole tile: requested first, written to LDS once they are here
    const float4* dt = dpk + (size_t)tile * kblocks * 4;
    const int nd = kblocks * 4;
    float4 dreg[4];
#pragma unroll
    for (int i = 0; i < 4; i++) dreg[i] = threadIdx.x + i * 256 < nd ? dt[threadIdx.x + i * 256] : make_float4(0.f, 0.f, 0.f, 0.f);
    Batch sets[NS];
#pragma unroll
    for (int q = 0; q < NS; q++) load_batch(q * U, sets[q]);
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (threadIdx.x + i * 256 < nd) lds_d[threadIdx.x + i * 256] = dreg[i];
    for (int i = threadIdx.x + 1024; i < nd; i += 256) lds_d[i] = dt[i]; // K beyond 16384
    if (LDSA)
    {
        // M rows of Kp halves, 16 bytes per thread and step; beyond K zeros (K % 16 == 0: a vector is all in or all out)
        v4i_bq* la = reinterpret_cast<v4i_bq*>(lds_d + (size_t)kblocks * 4);
        const int vec_per_row = Kp / 8;
        for (int i = threadIdx.x; i < M * vec_per_row; i += 256)
        {
            const int row = i / vec_per_row, v = i - row * vec_per_row;
            la[i] = v * 8 < K ? *reinterpret_cast<const v4i_bq*>(a + (size_t)row * a_stride + v * 8) : v4i_bq{0, 0, 0, 0};
        }
    }
    __syncthreads();
    for (int kb0 = 0; kb0 < nkb; kb0 += NS * U)
    {
#pragma unroll
        for (int q = 0; q < NS; q++)
        {
            compute(kb0 + q * U, sets[q]);                 // batch indices count from 0 inside this wave's range
            load_batch(kb0 + (q + NS) * U, sets[q]);       // requests beyond the range are masked off
        }
    }

    // combine the four K splits; accumulator r of lane l is (weight row (l/16)*4 + r, activation row l%16)
#pragma unroll
    for (int r = 0; r < 4; r++) red[wave][lane][r] = acc[r];
    __syncthreads();
    if (wave == 0 && m < M)
    {
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int j = tile * 16 + kg * 4 + r;
            if (j < N)
            {
                float f = add_rn(add_rn(red[0][lane][r], red[1][lane][r]), add_rn(red[2][lane][r], red[3][lane][r]));
                if (bt >= 0) f = add_rn(mul_rn(load_c(c, bt, m, j, N), beta), f);
                out[(size_t)m * out_stride + j] = mul_rn(f, alpha);
            }
        }
    }
}

// ---- the same contraction with every weight byte of a wavefront requested before the first one is used ----
// A bandwidth kernel on this chip is paced by the bytes it has in flight: 8 TB/s times a microsecond of memory latency is
// 8 MB, 32 KB per compute unit, and a matrix of 4096 rows is only 64 KB per compute unit in all.  So a workgroup still owns
// one tile of 16 weight rows, but its K blocks are dealt to as many wavefronts as it takes for each to hold ALL its blocks
// in registers (NB of them, 4 VGPRs each): a wavefront issues its whole share of the weight stream in one go, then
// multiplies block after block as the bytes arrive, and what is left to do when the last byte lands is one block.
// Requests go out in the order their data is needed (loads return in order; the compiler's scheduler, left alone, issues
// them in reverse, hence the scheduling barriers).  Activations and descales are parked in a piece of LDS that belongs to
// the wavefront alone, so no workgroup barrier stands between the loads and the arithmetic (a barrier would first wait
// for every load in flight).
//   ACT_LDS (decoding, up to MT <= 4 activation rows): the rows' K range of this wavefront goes through that LDS piece
//   once, ahead of the weights.
//   otherwise (up to 16 rows): each block's 16 rows x 64 halves ride in registers (8 VGPRs per block), requested right
//   behind the block's weights with a COALESCED lane mapping (8 lanes = one row's 128 bytes; in the matrix core's own
//   operand mapping a 16-lane group touches 16 rows, 16 cache lines for 256 bytes, and the loads took four times the
//   weight stream's share of the L1 pipe), and are turned into the operand mapping through 2.25 KB of LDS per wavefront
//   when the block is multiplied.
// BITS / HALVES: the packed layouts of ncnnhip_blockquant_pack.  HALVES = false is the 8-bit layout for quantisation
// blocks of 64 or 128 (a lane's 16 weights are 16 consecutive K, one descale per 64).  HALVES = true serves 4- and 6-bit
// fields and blocks of 32: the first matrix-core instruction of a 64-wide step covers K 0..31 and the second K 32..63
// (a lane holds K (l/16)*8..+7 of either half), each with a descale of its own (`split` = 1: blocks of 32; 0: the same
// descale twice).  A lane's share of a step is 2 * BITS bytes: one 16-byte load, one 8-byte load, or 8 + 4 bytes.
// AIN = 4: fp32 activations (times the optional input scales, INSC), the layer's own contract.  The matrix cores take no fp32
// operand of this shape, so a value is split into three bf16 numbers hi + mid + lo that add up to it EXACTLY (each takes the
// next 8 significant bits, by truncation, so every remainder is exact), when it is staged in LDS: three planes, which
// enter the matrix cores as three COLUMNS per activation row (up to 5 rows in the 16 columns), the weights converted to
// bf16 (integers up to 128 are exact there).  Every
// product is then the exact q * a of the reference and only the order of the fp32 additions differs, as with fp16
// activations.  (A remainder below 2^-126 is a denormal and may be dropped by the matrix core: |a| < 2^-110 or so.)
typedef int v2i_bq __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

__device__ __forceinline__ void split_bf16x3(float v, unsigned& hi, unsigned& mid, unsigned& lo) // each in the upper half of its dword
{
    const unsigned b = __float_as_uint(v);
    hi = b & 0xFFFF0000u;
    const bool finite = (b & 0x7F800000u) != 0x7F800000u; // infinities and NaNs travel in hi alone
    const float r1 = finite ? v - __uint_as_float(hi) : 0.f;
    mid = __float_as_uint(r1) & 0xFFFF0000u;
    const float r2 = r1 - __uint_as_float(mid);
    lo = __float_as_uint(r2) & 0xFFFF0000u; // at most 8 significant bits are left
}

__device__ __forceinline__ unsigned bf16_pair(float even, float odd) // both exactly representable: truncation loses nothing
{
    return (__float_as_uint(even) >> 16) | (__float_as_uint(odd) & 0xFFFF0000u);
}

// the 8 fields that bytes_to_halves / nibbles_to_halves / sixbit_to_halves turn into halves, as bf16
__device__ __forceinline__ v8bf bytes_to_bf16(unsigned lo, unsigned hi)
{
    union
    {
        unsigned i[4];
        v8bf h;
    } t;
    const unsigned slo = lo ^ 0x80808080u, shi = hi ^ 0x80808080u; // q + 128 -> q as a signed byte
#pragma unroll
    for (int p = 0; p < 2; p++)
    {
        t.i[p] = bf16_pair((float)(signed char)(slo >> (16 * p)), (float)(signed char)(slo >> (16 * p + 8)));
        t.i[2 + p] = bf16_pair((float)(signed char)(shi >> (16 * p)), (float)(signed char)(shi >> (16 * p + 8)));
    }
    return t.h;
}
__device__ __forceinline__ v8bf nibbles_to_bf16(unsigned w)
{
    union
    {
        unsigned i[4];
        v8bf h;
    } t;
    const unsigned x = w ^ 0x88888888u; // q + 8 -> q as a two's complement nibble: one signed bit-field extract each
#pragma unroll
    for (int p = 0; p < 4; p++) t.i[p] = bf16_pair((float)((int)(x << (28 - 4 * p)) >> 28), (float)((int)(x << (12 - 4 * p)) >> 28));
    return t.h;
}
__device__ __forceinline__ void sixbit_to_bf16(unsigned d0, unsigned d1, unsigned d2, v8bf& wa, v8bf& wb)
{
    union
    {
        unsigned i[4];
        v8bf h;
    } a, b;
    // q + 32 -> q in two's complement: flip bit 5 of every field (for pairs 6 and 7 that bit sits in dword 2's top nibbles)
    const unsigned d[3] = {d0 ^ 0x08200820u, d1 ^ 0x08200820u, d2 ^ 0xA820A820u};
#pragma unroll
    for (int P = 0; P < 8; P++)
    {
        float f[2];
#pragma unroll
        for (int h = 0; h < 2; h++)
        {
            int q;
            if (P < 6)
                q = (int)(d[P >> 1] << (26 - 6 * (P & 1) - 16 * h)) >> 26; // a signed bit-field extract
            else
            {
                const unsigned u = ((d[P - 6] >> (12 + 16 * h)) & 15u) | (((d[2] >> (12 + 2 * (P - 6) + 16 * h)) & 3u) << 4);
                q = (int)(u << 26) >> 26;
            }
            f[h] = (float)q;
        }
        (P < 4 ? a.i[P & 3] : b.i[P & 3]) = bf16_pair(f[0], f[1]);
    }
    wa = a.h;
    wb = b.h;
}

// Several weight matrices that share the activation rows, K and the field format in ONE launch (the gate and up projections of a
// decoder layer, q / k / v of an attention layer): the tiles of matrix i follow those of matrix i - 1 in the grid, and a workgroup
// finds its matrix by comparing its index with the running tile counts.  A launch of 17.8 or 45.8 MB is paced by its ramp and its
// tail, not by bandwidth; two or three of them in one launch are one ramp and one tail.  count == 0: the kernel's own arguments
// describe the one matrix.
constexpr int BQ_MULTI_MAX = 8;
struct BqMulti
{
    int count;
    int tile_end[BQ_MULTI_MAX]; // first tile (of the whole launch) that no longer belongs to matrix i
    int N[BQ_MULTI_MAX];
    int bt[BQ_MULTI_MAX];
    float alpha[BQ_MULTI_MAX], beta[BQ_MULTI_MAX];
    const unsigned char* wpk[BQ_MULTI_MAX];
    const float4* dpk[BQ_MULTI_MAX];
    const float* c[BQ_MULTI_MAX];
    float* out[BQ_MULTI_MAX];
    size_t out_stride[BQ_MULTI_MAX];
};

template<int BITS, bool HALVES, int NB, int MAXW, int MT, bool ACT_LDS, int AIN = 2, bool INSC = false>
__global__ __launch_bounds__(MAXW * 64) void blockquant8_upfront_kernel(const void* __restrict__ a_, size_t a_stride, int M, int N_, int K, int kblocks,
                                                                        const unsigned char* __restrict__ wpk_, const float4* __restrict__ dpk_, int split,
                                                                        const float* __restrict__ in_scales, const float* __restrict__ c_, int bt_, float alpha_,
                                                                        float beta_, float* __restrict__ out_, size_t out_stride_, BqMulti multi)
{
    // which matrix, which of its tiles (all wavefront-uniform: scalar loads from the argument block)
    int tile = blockIdx.x;
    int N = N_, bt = bt_;
    float alpha = alpha_, beta = beta_;
    const unsigned char* wpk = wpk_;
    const float4* dpk = dpk_;
    const float* c = c_;
    float* out = out_;
    size_t out_stride = out_stride_;
    if (multi.count)
    {
        int mi = 0;
#pragma unroll
        for (int i = 0; i < BQ_MULTI_MAX - 1; i++) mi += (i + 1 < multi.count && tile >= multi.tile_end[i]) ? 1 : 0;
        tile -= mi ? multi.tile_end[mi - 1] : 0;
        N = multi.N[mi], bt = multi.bt[mi], alpha = multi.alpha[mi], beta = multi.beta[mi];
        wpk = multi.wpk[mi], dpk = multi.dpk[mi], c = multi.c[mi], out = multi.out[mi], out_stride = multi.out_stride[mi];
    }
    static_assert(HALVES || BITS == 8, "4- and 6-bit fields come in the halves layout");
    static_assert(AIN == 2 || (AIN == 4 && ACT_LDS), "fp32 activations are staged in LDS");
    static_assert(AIN == 4 || !INSC, "input scales come with fp32 activations");
    constexpr bool F32 = AIN == 4;
    const __half* a = static_cast<const __half*>(a_);
    const float* af = static_cast<const float*>(a_);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_up[];
    constexpr int ACT_PITCH = NB * 128 + 128;                               // ACT_LDS: bytes from one staged activation row to the next (off the bank stride)
    constexpr int AV = ACT_LDS ? (MT * NB * 8 + 63) / 64 : 1;               // ACT_LDS: vectors of 8 activations per lane
    // rows the staging stores touch (>= MT: every lane stores, no branch); fp32: exactly MT, spare lanes store into row 0's padding
    constexpr int AROWS = ACT_LDS ? (F32 ? MT : (AV * 64 + NB * 8 - 1) / (NB * 8)) : 0;
    constexpr int PLANE_BYTES = AROWS * ACT_PITCH;                          // fp32: the hi, mid and lo planes follow one another
    constexpr int TR_PITCH = 144;                                           // !ACT_LDS: one row of a block (128 bytes) + 16: 16 rows land on 16 different bank groups
    const int D_BYTES = HALVES ? 1024 << split : 1024;                      // 64 (128 with blocks of 32) float4 of descales: NB * 4 (* 2) used
    const int WAVE_BYTES = D_BYTES + (ACT_LDS ? (F32 ? 3 : 1) * PLANE_BYTES : 16 * TR_PITCH); // descales, then the activations
    constexpr int STEP_BYTES = 128 * BITS;                                  // one tile's weights for a 64-wide K step
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int m = lane & 15;
    const int kg = lane >> 4;

    // K blocks of this wavefront: NB each, the last one what is left (possibly none: it then re-reads block 0 and adds zeros)
    const int kb_begin = wave * NB;
    int nkb = kblocks - kb_begin;
    nkb = nkb > NB ? NB : nkb;
    nkb = nkb < 0 ? 0 : nkb;
    const int kb_base = nkb > 0 ? kb_begin : 0;

    unsigned char* mine = lds_up + wave * WAVE_BYTES;
    float4* my_d = reinterpret_cast<float4*>(mine);
    unsigned char* my_a = mine + D_BYTES;

    // (1) ACT_LDS: the activations of the wavefront's K range.  Every load is unconditional, from a clamped address, and
    // masked afterwards (a guarded load becomes a branch, and the compiler waits for every load in flight past a branch).
    v4i_bq areg[AV];
    v4i_bq areg2[F32 ? AV : 1];                // fp32: the vector's second 16 bytes
    v4i_bq sreg[INSC ? AV : 1], sreg2[INSC ? AV : 1]; // its input scales
    if (ACT_LDS)
    {
#pragma unroll
        for (int q = 0; q < AV; q++)
        {
            const int idx = q * 64 + lane;
            const int r = idx / (NB * 8), v = idx - r * (NB * 8);
            const int k = kb_base * 64 + v * 8;
            const bool ok = v < nkb * 8 && k < K; // K % 16 == 0: a vector of 8 activations is all in or all out
            const int rr = r < M ? r : 0;
            if (F32)
            {
                const float* p = af + (size_t)rr * a_stride + (ok ? k : 0);
                areg[q] = *reinterpret_cast<const v4i_bq*>(p);
                areg2[F32 ? q : 0] = *reinterpret_cast<const v4i_bq*>(p + 4);
                if (INSC)
                {
                    sreg[INSC ? q : 0] = *reinterpret_cast<const v4i_bq*>(in_scales + (ok ? k : 0));
                    sreg2[INSC ? q : 0] = *reinterpret_cast<const v4i_bq*>(in_scales + (ok ? k : 0) + 4);
                }
            }
            else
                areg[q] = *reinterpret_cast<const v4i_bq*>(a + (size_t)rr * a_stride + (ok ? k : 0));
        }
    }
    // (2) descales of the wavefront's blocks: float4 number j of them is (block j / 4, row group j % 4); with blocks of 32,
    // (step j / 8, half (j / 4) % 2, row group j % 4)
    const int dper = HALVES ? 4 << split : 4; // float4 per step
    const float4* dt = dpk + ((size_t)tile * kblocks + kb_base) * dper;
    __builtin_amdgcn_sched_barrier(0);
    const float4 dreg = dt[lane < nkb * dper ? lane : 0];
    float4 dreg2 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (HALVES) dreg2 = dt[lane + 64 < nkb * dper ? lane + 64 : 0];
    __builtin_amdgcn_sched_barrier(0);
    // (3) the weights, all of them; !ACT_LDS: each block's activations right behind its weights.  Lane l fetches 16 bytes of
    // rows l/8 and l/8 + 8, piece l%8 of the block's 128 bytes per row; a chunk beyond K is read from the start of the row
    // (it meets packed weights that are zero there), rows from M up repeat row 0 (their results are never stored).
    const unsigned char* wt = wpk + ((size_t)tile * kblocks + kb_base) * STEP_BYTES;
    v4i_bq w[BITS == 8 ? NB : 1]; // 8-bit: 16 bytes per lane and step
    v2i_bq w2[BITS != 8 ? NB : 1]; // 4-bit: all 8 bytes; 6-bit: the first two of three dwords
    int w1[BITS == 6 ? NB : 1];    // 6-bit: the third dword (the step's 64 x 8 bytes first, then its 64 x 4 bytes)
    v4i_bq a0[ACT_LDS ? 1 : NB], a1[ACT_LDS ? 1 : NB];
    const int tr_row = lane >> 3, tr_piece = lane & 7;
    const __half* arow0 = a + (size_t)(tr_row < M ? tr_row : 0) * a_stride;
    const __half* arow1 = a + (size_t)(tr_row + 8 < M ? tr_row + 8 : 0) * a_stride;
#pragma unroll
    for (int i = 0; i < NB; i++)
    {
        const unsigned char* ws = wt + (size_t)(i < nkb ? i : 0) * STEP_BYTES;
        if (BITS == 8)
            w[BITS == 8 ? i : 0] = __builtin_nontemporal_load(reinterpret_cast<const v4i_bq*>(ws) + lane);
        else
            w2[BITS != 8 ? i : 0] = __builtin_nontemporal_load(reinterpret_cast<const v2i_bq*>(ws) + lane);
        if (BITS == 6) w1[BITS == 6 ? i : 0] = __builtin_nontemporal_load(reinterpret_cast<const int*>(ws + 512) + lane);
        __builtin_amdgcn_sched_barrier(0);
        if (!ACT_LDS)
        {
            const int k = (kb_base + (i < nkb ? i : 0)) * 64 + tr_piece * 8;
            const int kk = k < K ? k : 0;
            a0[ACT_LDS ? 0 : i] = *reinterpret_cast<const v4i_bq*>(arow0 + kk);
            a1[ACT_LDS ? 0 : i] = *reinterpret_cast<const v4i_bq*>(arow1 + kk);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // (4) park activations and descales in the wavefront's own LDS (same wavefront writes and reads: program order holds)
    if (ACT_LDS)
    {
#pragma unroll
        for (int q = 0; q < AV; q++)
        {
            const int idx = q * 64 + lane;
            const int r = idx / (NB * 8), v = idx - r * (NB * 8);
            const int k = kb_base * 64 + v * 8;
            const bool ok = v < nkb * 8 && k < K;
            if (F32)
            {
                // 8 floats -> 8 bf16 in each of the three planes; lanes beyond the rows' vectors store into the padding behind row 0
                const bool spare = idx >= MT * NB * 8;
                unsigned char* dst = my_a + (spare ? NB * 128 : r * ACT_PITCH + v * 16);
                v4i_bq pl[3];
#pragma unroll
                for (int e = 0; e < 4; e++)
                {
                    unsigned h[2][3];
#pragma unroll
                    for (int o = 0; o < 2; o++)
                    {
                        const int j = 2 * e + o; // element of the vector
                        float x = __int_as_float(j < 4 ? areg[q][j & 3] : areg2[F32 ? q : 0][j & 3]);
                        if (INSC) x = mul_rn(x, __int_as_float(j < 4 ? sreg[INSC ? q : 0][j & 3] : sreg2[INSC ? q : 0][j & 3]));
                        x = ok ? x : 0.f;
                        split_bf16x3(x, h[o][0], h[o][1], h[o][2]);
                    }
#pragma unroll
                    for (int pnum = 0; pnum < 3; pnum++) pl[pnum][e] = (int)((h[0][pnum] >> 16) | h[1][pnum]);
                }
#pragma unroll
                for (int pnum = 0; pnum < 3; pnum++) *reinterpret_cast<v4i_bq*>(dst + pnum * PLANE_BYTES) = pl[pnum];
                continue;
            }
            v4i_bq t = areg[q];
#pragma unroll
            for (int e = 0; e < 4; e++) t[e] = ok ? t[e] : 0;
            *reinterpret_cast<v4i_bq*>(my_a + r * ACT_PITCH + v * 16) = t; // unconditional: a guarded store would pull its load into the branch
        }
    }
    my_d[lane] = lane < nkb * dper ? dreg : make_float4(0.f, 0.f, 0.f, 0.f);
    if (HALVES && split) my_d[lane + 64] = lane + 64 < nkb * dper ? dreg2 : make_float4(0.f, 0.f, 0.f, 0.f);

    // (5) block after block, as the weights arrive
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int A_LANE = HALVES ? 16 : 32; // bytes from one K group's operand to the next inside a staged row
    constexpr int A_SECOND = HALVES ? 64 : 16; // and from the first instruction's operand to the second's
    const unsigned char* act_rd = ACT_LDS ? my_a + (m < M && m < MT ? m : 0) * ACT_PITCH + kg * A_LANE : my_a + m * TR_PITCH + kg * A_LANE;
    if (F32)
    {
        static_assert(!F32 || MT <= 5, "three columns per row, 16 columns");
        const int prow = m / 3, ppl = m - prow * 3;
        const bool used = prow < M && prow < MT;
        act_rd = my_a + (used ? ppl * PLANE_BYTES + prow * ACT_PITCH : 0) + kg * A_LANE;
    }
    unsigned char* tr_wr = my_a + tr_row * TR_PITCH + tr_piece * 16;
#pragma unroll
    for (int i = 0; i < NB; i++)
    {
        if (F32)
        {
            v8bf fa, fb;
            if (BITS == 8)
            {
                fa = bytes_to_bf16((unsigned)w[BITS == 8 ? i : 0][0], (unsigned)w[BITS == 8 ? i : 0][1]);
                fb = bytes_to_bf16((unsigned)w[BITS == 8 ? i : 0][2], (unsigned)w[BITS == 8 ? i : 0][3]);
            }
            else if (BITS == 4)
            {
                fa = nibbles_to_bf16((unsigned)w2[BITS != 8 ? i : 0][0]);
                fb = nibbles_to_bf16((unsigned)w2[BITS != 8 ? i : 0][1]);
            }
            else
                sixbit_to_bf16((unsigned)w2[BITS != 8 ? i : 0][0], (unsigned)w2[BITS != 8 ? i : 0][1], (unsigned)w1[BITS == 6 ? i : 0], fa, fb);
            // column l%16 of the matrix-core product is (row, plane) = ((l%16) / 3, (l%16) % 3): the three partial products of a row
            // come out of the same two instructions, side by side, and are added at the very end
            const v4f zero = {0.f, 0.f, 0.f, 0.f};
            union
            {
                v4i_bq i4;
                v8bf h;
            } ya, yb;
            ya.i4 = *reinterpret_cast<const v4i_bq*>(act_rd + i * 128);
            yb.i4 = *reinterpret_cast<const v4i_bq*>(act_rd + i * 128 + A_SECOND);
            v4f t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, ya.h, zero, 0, 0, 0), t1 = zero;
            if (HALVES)
                t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb, yb.h, zero, 0, 0, 0);
            else
                t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb, yb.h, t0, 0, 0, 0);
            if (HALVES)
            {
                const float4 da = my_d[i * dper + kg];
                const float4 db = my_d[i * dper + (split << 2) + kg];
                acc[0] = fmaf(t1[0], db.x, fmaf(t0[0], da.x, acc[0]));
                acc[1] = fmaf(t1[1], db.y, fmaf(t0[1], da.y, acc[1]));
                acc[2] = fmaf(t1[2], db.z, fmaf(t0[2], da.z, acc[2]));
                acc[3] = fmaf(t1[3], db.w, fmaf(t0[3], da.w, acc[3]));
            }
            else
            {
                const float4 d = my_d[i * 4 + kg];
                acc[0] = fmaf(t0[0], d.x, acc[0]);
                acc[1] = fmaf(t0[1], d.y, acc[1]);
                acc[2] = fmaf(t0[2], d.z, acc[2]);
                acc[3] = fmaf(t0[3], d.w, acc[3]);
            }
            continue;
        }
        v8h wa, wb;
        if (BITS == 8)
        {
            wa = bytes_to_halves(w[BITS == 8 ? i : 0][0], w[BITS == 8 ? i : 0][1]);
            wb = bytes_to_halves(w[BITS == 8 ? i : 0][2], w[BITS == 8 ? i : 0][3]);
        }
        else if (BITS == 4)
        {
            wa = nibbles_to_halves((unsigned)w2[BITS != 8 ? i : 0][0]);
            wb = nibbles_to_halves((unsigned)w2[BITS != 8 ? i : 0][1]);
        }
        else
            sixbit_to_halves((unsigned)w2[BITS != 8 ? i : 0][0], (unsigned)w2[BITS != 8 ? i : 0][1], (unsigned)w1[BITS == 6 ? i : 0], wa, wb);
        union
        {
            v4i_bq i4;
            v8h h;
        } xa, xb;
        if (ACT_LDS)
        {
            xa.i4 = *reinterpret_cast<const v4i_bq*>(act_rd + i * 128);
            xb.i4 = *reinterpret_cast<const v4i_bq*>(act_rd + i * 128 + A_SECOND);
        }
        else
        {
            // the block's 16 rows x 128 bytes from the fetch mapping into the operand mapping (the wavefront's LDS operations
            // execute in order, so the next block's stores cannot overtake these reads)
            *reinterpret_cast<v4i_bq*>(tr_wr) = a0[ACT_LDS ? 0 : i];
            *reinterpret_cast<v4i_bq*>(tr_wr + 8 * TR_PITCH) = a1[ACT_LDS ? 0 : i];
            xa.i4 = *reinterpret_cast<const v4i_bq*>(act_rd);
            xb.i4 = *reinterpret_cast<const v4i_bq*>(act_rd + A_SECOND);
        }
        const v4f zero = {0.f, 0.f, 0.f, 0.f};
        if (HALVES)
        {
            // the two halves of the step apart: a block of 32 ends between them
            const v4f t0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, xa.h, zero, 0, 0, 0);
            const v4f t1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(wb, xb.h, zero, 0, 0, 0);
            const float4 da = my_d[i * dper + kg]; // zero for a step beyond the wavefront's range
            const float4 db = my_d[i * dper + (split << 2) + kg];
            acc[0] = fmaf(t1[0], db.x, fmaf(t0[0], da.x, acc[0]));
            acc[1] = fmaf(t1[1], db.y, fmaf(t0[1], da.y, acc[1]));
            acc[2] = fmaf(t1[2], db.z, fmaf(t0[2], da.z, acc[2]));
            acc[3] = fmaf(t1[3], db.w, fmaf(t0[3], da.w, acc[3]));
        }
        else
        {
            v4f t = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, xa.h, zero, 0, 0, 0);
            t = __builtin_amdgcn_mfma_f32_16x16x32_f16(wb, xb.h, t, 0, 0, 0);
            const float4 d = my_d[i * 4 + kg]; // zero for a block beyond the wavefront's range
            acc[0] = fmaf(t[0], d.x, acc[0]);
            acc[1] = fmaf(t[1], d.y, acc[1]);
            acc[2] = fmaf(t[2], d.z, acc[2]);
            acc[3] = fmaf(t[3], d.w, acc[3]);
        }
    }

    // (6) combine the wavefronts' K ranges in wavefront order; accumulator r of lane l is (weight row (l/16)*4 + r, activation row l%16)
    // (the exchange buffer lies over the wavefronts' own pieces, which everybody has finished with after the first barrier)
    float4* red = reinterpret_cast<float4*>(lds_up);
    __syncthreads();
    red[wave * 64 + lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    if (wave == 0 && m < M)
    {
        // fp32 activations: lane (l/16, row) adds the row's three columns, each summed over the wavefronts first
        const int src = F32 ? (lane & 48) + m * 3 : lane;
        float4 f = red[src];
        for (int w2 = 1; w2 < nwaves; w2++)
        {
            const float4 o = red[w2 * 64 + src];
            f.x = add_rn(f.x, o.x);
            f.y = add_rn(f.y, o.y);
            f.z = add_rn(f.z, o.z);
            f.w = add_rn(f.w, o.w);
        }
        if (F32)
        {
#pragma unroll
            for (int pnum = 1; pnum < 3; pnum++)
            {
                float4 g = red[src + pnum];
                for (int w2 = 1; w2 < nwaves; w2++)
                {
                    const float4 o = red[w2 * 64 + src + pnum];
                    g.x = add_rn(g.x, o.x);
                    g.y = add_rn(g.y, o.y);
                    g.z = add_rn(g.z, o.z);
                    g.w = add_rn(g.w, o.w);
                }
                f.x = add_rn(f.x, g.x);
                f.y = add_rn(f.y, g.y);
                f.z = add_rn(f.z, g.z);
                f.w = add_rn(f.w, g.w);
            }
        }
        const float fr[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int j = tile * 16 + kg * 4 + r;
            if (j < N)
            {
                float v = fr[r];
                if (bt >= 0) v = add_rn(mul_rn(load_c(c, bt, m, j, N), beta), v);
                out[(size_t)m * out_stride + j] = mul_rn(v, alpha); // (a non-temporal store measured 1-3 % slower)
            }
        }
    }
}

// The 5-to-16-row form for many weight rows: one workgroup takes TWO neighbouring tiles of 16 weight rows and multiplies both
// with the same activation registers.  A tile's 64 KB of weights at K = 4096 come with 128 KB of activations through the same
// L1; sharing them between two tiles takes that from 192 to 128 KB per tile (fp16 activations, K up to 4096).
template<int BITS, bool HALVES, int NB, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void blockquant8_rows16_pair_kernel(const __half* __restrict__ a, size_t a_stride, int M, int N, int K, int kblocks,
                                                                            int ntiles, const unsigned char* __restrict__ wpk, const float4* __restrict__ dpk,
                                                                            int split, const float* __restrict__ c, int bt, float alpha, float beta,
                                                                            float* __restrict__ out, size_t out_stride)
{
    static_assert(HALVES || BITS == 8, "4- and 6-bit fields come in the halves layout");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_up[];
    constexpr int TR_PITCH = 144; // one row of a step (128 bytes) + 16: 16 rows land on 16 different bank groups
    const int D_BYTES = HALVES ? 1024 << split : 1024;
    const int WAVE_BYTES = 2 * D_BYTES + 16 * TR_PITCH; // both tiles' descales, then the transpose buffer
    constexpr int STEP_BYTES = 128 * BITS;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int tile0 = blockIdx.x * 2;
    const int m = lane & 15;
    const int kg = lane >> 4;

    const int kb_begin = wave * NB;
    int nkb = kblocks - kb_begin;
    nkb = nkb > NB ? NB : nkb;
    nkb = nkb < 0 ? 0 : nkb;
    const int kb_base = nkb > 0 ? kb_begin : 0;

    unsigned char* mine = lds_up + wave * WAVE_BYTES;
    unsigned char* my_a = mine + 2 * D_BYTES;

    // an odd tile count: the last workgroup's second tile reads the first one's operands again and stores nothing
    const int dper = HALVES ? 4 << split : 4;
    float4 dreg[2], dreg2[2];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int tt = 0; tt < 2; tt++)
    {
        const int tl = tile0 + tt < ntiles ? tile0 + tt : tile0;
        const float4* dt = dpk + ((size_t)tl * kblocks + kb_base) * dper;
        dreg[tt] = dt[lane < nkb * dper ? lane : 0];
        dreg2[tt] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (HALVES) dreg2[tt] = dt[lane + 64 < nkb * dper ? lane + 64 : 0];
    }
    __builtin_amdgcn_sched_barrier(0);
    v4i_bq w[BITS == 8 ? 2 * NB : 1];
    v2i_bq w2[BITS != 8 ? 2 * NB : 1];
    int w1[BITS == 6 ? 2 * NB : 1];
    v4i_bq a0[NB], a1[NB];
    const int tr_row = lane >> 3, tr_piece = lane & 7;
    const __half* arow0 = a + (size_t)(tr_row < M ? tr_row : 0) * a_stride;
    const __half* arow1 = a + (size_t)(tr_row + 8 < M ? tr_row + 8 : 0) * a_stride;
#pragma unroll
    for (int i = 0; i < NB; i++)
    {
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
        {
            const int tl = tile0 + tt < ntiles ? tile0 + tt : tile0;
            const unsigned char* ws = wpk + ((size_t)tl * kblocks + kb_base + (i < nkb ? i : 0)) * STEP_BYTES;
            if (BITS == 8)
                w[BITS == 8 ? 2 * i + tt : 0] = __builtin_nontemporal_load(reinterpret_cast<const v4i_bq*>(ws) + lane);
            else
                w2[BITS != 8 ? 2 * i + tt : 0] = __builtin_nontemporal_load(reinterpret_cast<const v2i_bq*>(ws) + lane);
            if (BITS == 6) w1[BITS == 6 ? 2 * i + tt : 0] = __builtin_nontemporal_load(reinterpret_cast<const int*>(ws + 512) + lane);
            __builtin_amdgcn_sched_barrier(0);
        }
        const int k = (kb_base + (i < nkb ? i : 0)) * 64 + tr_piece * 8;
        const int kk = k < K ? k : 0;
        a0[i] = *reinterpret_cast<const v4i_bq*>(arow0 + kk);
        a1[i] = *reinterpret_cast<const v4i_bq*>(arow1 + kk);
        __builtin_amdgcn_sched_barrier(0);
    }

#pragma unroll
    for (int tt = 0; tt < 2; tt++)
    {
        float4* my_d = reinterpret_cast<float4*>(mine + tt * D_BYTES);
        my_d[lane] = lane < nkb * dper ? dreg[tt] : make_float4(0.f, 0.f, 0.f, 0.f);
        if (HALVES && split) my_d[lane + 64] = lane + 64 < nkb * dper ? dreg2[tt] : make_float4(0.f, 0.f, 0.f, 0.f);
    }

    v4f acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    constexpr int A_LANE = HALVES ? 16 : 32;
    constexpr int A_SECOND = HALVES ? 64 : 16;
    const unsigned char* act_rd = my_a + m * TR_PITCH + kg * A_LANE;
    unsigned char* tr_wr = my_a + tr_row * TR_PITCH + tr_piece * 16;
#pragma unroll
    for (int i = 0; i < NB; i++)
    {
        union
        {
            v4i_bq i4;
            v8h h;
        } xa, xb;
        *reinterpret_cast<v4i_bq*>(tr_wr) = a0[i];
        *reinterpret_cast<v4i_bq*>(tr_wr + 8 * TR_PITCH) = a1[i];
        xa.i4 = *reinterpret_cast<const v4i_bq*>(act_rd);
        xb.i4 = *reinterpret_cast<const v4i_bq*>(act_rd + A_SECOND);
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
        {
            v8h wa, wb;
            if (BITS == 8)
            {
                wa = bytes_to_halves(w[BITS == 8 ? 2 * i + tt : 0][0], w[BITS == 8 ? 2 * i + tt : 0][1]);
                wb = bytes_to_halves(w[BITS == 8 ? 2 * i + tt : 0][2], w[BITS == 8 ? 2 * i + tt : 0][3]);
            }
            else if (BITS == 4)
            {
                wa = nibbles_to_halves((unsigned)w2[BITS != 8 ? 2 * i + tt : 0][0]);
                wb = nibbles_to_halves((unsigned)w2[BITS != 8 ? 2 * i + tt : 0][1]);
            }
            else
                sixbit_to_halves((unsigned)w2[BITS != 8 ? 2 * i + tt : 0][0], (unsigned)w2[BITS != 8 ? 2 * i + tt : 0][1], (unsigned)w1[BITS == 6 ? 2 * i + tt : 0], wa, wb);
            const float4* my_d = reinterpret_cast<const float4*>(mine + tt * D_BYTES);
            const v4f zero = {0.f, 0.f, 0.f, 0.f};
            if (HALVES)
            {
                const v4f t0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, xa.h, zero, 0, 0, 0);
                const v4f t1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(wb, xb.h, zero, 0, 0, 0);
                const float4 da = my_d[i * dper + kg];
                const float4 db = my_d[i * dper + (split << 2) + kg];
                acc[tt][0] = fmaf(t1[0], db.x, fmaf(t0[0], da.x, acc[tt][0]));
                acc[tt][1] = fmaf(t1[1], db.y, fmaf(t0[1], da.y, acc[tt][1]));
                acc[tt][2] = fmaf(t1[2], db.z, fmaf(t0[2], da.z, acc[tt][2]));
                acc[tt][3] = fmaf(t1[3], db.w, fmaf(t0[3], da.w, acc[tt][3]));
            }
            else
            {
                v4f t = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, xa.h, zero, 0, 0, 0);
                t = __builtin_amdgcn_mfma_f32_16x16x32_f16(wb, xb.h, t, 0, 0, 0);
                const float4 d = my_d[i * 4 + kg];
                acc[tt][0] = fmaf(t[0], d.x, acc[tt][0]);
                acc[tt][1] = fmaf(t[1], d.y, acc[tt][1]);
                acc[tt][2] = fmaf(t[2], d.z, acc[tt][2]);
                acc[tt][3] = fmaf(t[3], d.w, acc[tt][3]);
            }
        }
    }

    // combine the wavefronts' K ranges in wavefront order: wavefront 0 finishes the first tile, wavefront 1 the second
    float4* red = reinterpret_cast<float4*>(lds_up);
    __syncthreads();
    red[wave * 64 + lane] = make_float4(acc[0][0], acc[0][1], acc[0][2], acc[0][3]);
    red[(nwaves + wave) * 64 + lane] = make_float4(acc[1][0], acc[1][1], acc[1][2], acc[1][3]);
    __syncthreads();
    // (a single wavefront, K up to 512, finishes both)
    for (int tt = wave; tt < 2 && m < M; tt += nwaves)
    {
        const float4* mr = red + tt * nwaves * 64;
        float4 f = mr[lane];
        for (int w2i = 1; w2i < nwaves; w2i++)
        {
            const float4 o = mr[w2i * 64 + lane];
            f.x = add_rn(f.x, o.x);
            f.y = add_rn(f.y, o.y);
            f.z = add_rn(f.z, o.z);
            f.w = add_rn(f.w, o.w);
        }
        const float fr[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int j = (tile0 + tt) * 16 + kg * 4 + r;
            if (j < N)
            {
                float v = fr[r];
                if (bt >= 0) v = add_rn(mul_rn(load_c(c, bt, m, j, N), beta), v);
                out[(size_t)m * out_stride + j] = mul_rn(v, alpha);
            }
        }
    }
}

// ---- many activation rows (prefill, attention projections) on the packed weights, fp32 activations ------------------------
// The same exact three-way bf16 split, made ONCE by a pass of its own into a workspace (three planes [rows][K], rows and K
// padded with zeros to multiples of 64), then a tiled Gemm on v_mfma_f32_16x16x32_bf16: three bf16 instructions do the work
// of one fp32 product exactly, at 16 times the fp32 matrix-core rate per instruction.  A workgroup (4 wavefronts) owns 128
// weight rows x 64 activation rows; a wavefront 32 weight rows (two packed tiles, straight from HBM into the operand layout
// they were packed in, converted to bf16 in registers) x all 64 activation rows, whose planes the workgroup stages per
// 64-wide K step in LDS (two buffers, 144-byte row pitch: 16 rows fall on 16 different bank groups).  Per step and
// (tile, 16-row group) the six instructions (3 planes x 2 halves of the step) add into a fresh accumulator that is then
// scaled by the step's 1/scale, like the few-row kernels do.
// SPLIT_VECS vectors of 8 activations per thread, all of them requested before the first is split: with one vector per thread
// the pass ran at 2 TB/s (20 us for 1024 x 4096), short of bytes in flight; with four 11 us; eight measured slower again.
static constexpr int SPLIT_VECS = 4;
__global__ __launch_bounds__(256) void blockquant_split_activations_kernel(const float* __restrict__ a, size_t a_stride, int M, int K,
                                                                            const float* __restrict__ in_scales, unsigned short* __restrict__ planes, int Mp,
                                                                            int Kp)
{
    const int vec_per_row = Kp >> 3;
    const size_t total = (size_t)Mp * vec_per_row;
    const size_t first = (size_t)blockIdx.x * (256 * SPLIT_VECS) + threadIdx.x;
    float x[SPLIT_VECS][8];
    int row[SPLIT_VECS], k[SPLIT_VECS];
#pragma unroll
    for (int u = 0; u < SPLIT_VECS; u++)
    {
        const size_t idx = first + (size_t)u * 256;
        const size_t ii = idx < total ? idx : 0;
        row[u] = (int)(ii / vec_per_row);
        k[u] = (int)(ii - (size_t)row[u] * vec_per_row) << 3;
        const bool inside = idx < total && row[u] < M && k[u] < K; // K % 16 == 0: a vector of 8 is all in or all out
        const float* p = a + (inside ? (size_t)row[u] * a_stride + k[u] : (size_t)0);
#pragma unroll
        for (int j = 0; j < 8; j++) x[u][j] = p[j]; // a valid address either way (K >= 16)
        if (!inside)
        {
#pragma unroll
            for (int j = 0; j < 8; j++) x[u][j] = 0.f;
        }
        else if (in_scales)
        {
#pragma unroll
            for (int j = 0; j < 8; j++) x[u][j] = mul_rn(x[u][j], in_scales[k[u] + j]);
        }
    }
#pragma unroll
    for (int u = 0; u < SPLIT_VECS; u++)
    {
        if (first + (size_t)u * 256 >= total) break;
        unsigned pl[3][4];
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            unsigned h[2][3];
#pragma unroll
            for (int o = 0; o < 2; o++) split_bf16x3(x[u][2 * e + o], h[o][0], h[o][1], h[o][2]);
#pragma unroll
            for (int pn = 0; pn < 3; pn++) pl[pn][e] = (h[0][pn] >> 16) | h[1][pn];
        }
#pragma unroll
        for (int pn = 0; pn < 3; pn++)
            *reinterpret_cast<uint4*>(planes + ((size_t)pn * Mp + row[u]) * Kp + k[u]) = make_uint4(pl[pn][0], pl[pn][1], pl[pn][2], pl[pn][3]);
    }
}

#define BQ_AS1 __attribute__((address_space(1)))
#define BQ_AS3 __attribute__((address_space(3)))
// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding)
#define BQ_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | ((((n) >> 4) & 3) << 14))

// Everything a K step needs goes from global memory straight into LDS (no registers in between), into a ring of STAGES
// stages of which STAGES - 1 are in flight while one is multiplied: one wait + one barrier per step, and a step's memory
// latency is spread over the arithmetic of the steps before it.  A direct load writes the wavefront's 64 x 16 bytes in lane
// order, so the layout is made on the SOURCE side: the 16-byte chunk c of activation row r lands at chunk position
// c ^ ((r / 2) % 8) of its 128-byte row, which makes the operand reads (16 rows x one chunk) conflict-free without padding.
// A stage: 3 planes x 64 rows x 128 bytes, then the workgroup's 8 weight tiles (1 KB apiece reserved) and their descales
// (128 bytes apiece).  Every wavefront issues exactly ten loads per stage (6 of activations, its 2 tiles, their 2 descale
// rows; beyond the last step it loads the last step again into a stage nobody reads any more), which is what the wait counts.
template<int BITS, bool HALVES, int STAGES, int RW>
__global__ __launch_bounds__(256) void blockquant_rows_bf16x3_kernel(const unsigned short* __restrict__ planes, int Mp, int Kp, int M, int N, int kblocks,
                                                                      int ntiles, const unsigned char* __restrict__ wpk, const float4* __restrict__ dpk, int split,
                                                                      const float* __restrict__ c, int bt, float alpha, float beta, float* __restrict__ out,
                                                                      size_t out_stride)
{
    static_assert(HALVES || BITS == 8, "4- and 6-bit fields come in the halves layout");
    constexpr int LOADS = 6 + 2 * RW; // per wavefront and stage
    static_assert(STAGES >= 2 && (STAGES - 2) * LOADS < 64, "the vmcnt field counts to 63");
    static_assert(RW >= 1 && RW <= 4, "one to four tiles of 16 weight rows per wavefront");
    constexpr int PLANE = 64 * 128;
    constexpr int ACT_BYTES = 3 * PLANE;
    constexpr int W_OFF = ACT_BYTES, D_OFF = ACT_BYTES + 4 * RW * 1024;
    constexpr int STAGE_BYTES = D_OFF + 4 * RW * 128;
    constexpr int STEP_BYTES = 128 * BITS;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds_rows[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int m = lane & 15, kg = lane >> 4;
    const int row0 = blockIdx.y * 64;
    const int dper = HALVES ? 4 << split : 4;

    // the wavefront's RW tiles (a tile beyond the last reads the last one again and stores nothing)
    const unsigned char* wsrc[RW];
    const float4* dsrc[RW];
#pragma unroll
    for (int rw = 0; rw < RW; rw++)
    {
        const int t = (blockIdx.x * 4 + wave) * RW + rw;
        const int tl = t < ntiles ? t : ntiles - 1;
        wsrc[rw] = wpk + (size_t)tl * kblocks * STEP_BYTES + lane * 16;
        dsrc[rw] = dpk + (size_t)tl * kblocks * dper + lane;
    }
    // activation loads: load i of wavefront w fills rows (i % 2) * 32 + w * 8 .. +8 of plane i / 2; lane l brings row + l / 8,
    // the chunk that belongs at position l % 8
    const unsigned short* asrc[6];
#pragma unroll
    for (int i = 0; i < 6; i++)
    {
        const int r = (i & 1) * 32 + wave * 8 + (lane >> 3);
        const int ch = (lane & 7) ^ ((r >> 1) & 7);
        asrc[i] = planes + ((size_t)(i >> 1) * Mp + row0 + r) * Kp + ch * 8;
    }
    auto issue = [&](int step, int slot) {
        unsigned char* st = lds_rows + slot * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 6; i++)
            __builtin_amdgcn_global_load_lds((const BQ_AS1 void*)(asrc[i] + (size_t)step * 64),
                                             (BQ_AS3 void*)(st + (i >> 1) * PLANE + ((i & 1) * 32 + wave * 8) * 128), 16, 0, 0);
#pragma unroll
        for (int rw = 0; rw < RW; rw++)
        {
            if (lane < STEP_BYTES / 16)
                __builtin_amdgcn_global_load_lds((const BQ_AS1 void*)(wsrc[rw] + (size_t)step * STEP_BYTES), (BQ_AS3 void*)(st + W_OFF + (wave * RW + rw) * 1024), 16, 0,
                                                 0);
        }
#pragma unroll
        for (int rw = 0; rw < RW; rw++)
        {
            if (lane < dper)
                __builtin_amdgcn_global_load_lds((const BQ_AS1 void*)(dsrc[rw] + (size_t)step * dper), (BQ_AS3 void*)(st + D_OFF + (wave * RW + rw) * 128), 16, 0, 0);
        }
    };

    v4f acc[RW][4];
#pragma unroll
    for (int rw = 0; rw < RW; rw++)
#pragma unroll
        for (int cw = 0; cw < 4; cw++) acc[rw][cw] = v4f{0.f, 0.f, 0.f, 0.f};

    // operand reads: row cw * 16 + m, chunk positions of the lane's two K groups (the swizzle does not depend on cw)
    const int sw = (m >> 1) & 7;
    const int rd_a = m * 128 + (((HALVES ? kg : 2 * kg) ^ sw) << 4);
    const int rd_b = m * 128 + (((HALVES ? 4 + kg : 2 * kg + 1) ^ sw) << 4);
    const int last = kblocks - 1;
    const unsigned lds_base = (unsigned)(uintptr_t)(BQ_AS3 unsigned char*)lds_rows;

#pragma unroll
    for (int j = 0; j < STAGES - 1; j++) issue(j < last ? j : last, j);
    int slot = 0, fill = STAGES - 1; // the stage multiplied in this step, and the one its loads refill (the one step - 1 used)
    for (int step = 0; step < kblocks; step++)
    {
        BQ_WAIT_VMCNT((STAGES - 2) * LOADS); // this wavefront's loads of stage `step` have landed; STAGES - 2 newer stages may still be on their way
        __builtin_amdgcn_s_barrier();     // and everybody else's; everybody has also left stage step - 1, which the next loads overwrite
        asm volatile("" ::: "memory");
        {
            const int ahead = step + STAGES - 1;
            issue(ahead < last ? ahead : last, fill);
        }
        // LDS is read with hand-written instructions and waits: the compiler treats a direct-to-LDS load as a store to all of LDS
        // and would drain every load in flight (vmcnt(0)) in front of each read it emits itself.  A wait names the registers it
        // covers as in/out operands, so nothing can use them ahead of it.
        const unsigned st = lds_base + (unsigned)(slot * STAGE_BYTES);
        fill = slot;
        slot = slot + 1 == STAGES ? 0 : slot + 1;
        v4i_bq wq[RW], dq0[RW], dq1[RW];
        v2i_bq wlo[RW]; // 4- and 6-bit: the lane's first 8 bytes
        int whi[RW];    // 6-bit: its third dword
#pragma unroll
        for (int rw = 0; rw < RW; rw++)
        {
            wq[rw] = v4i_bq{0, 0, 0, 0};
            wlo[rw] = v2i_bq{0, 0};
            whi[rw] = 0;
        }
        {
            const unsigned wl = st + W_OFF + (unsigned)(wave * RW * 1024) + (unsigned)(lane * (BITS == 8 ? 16 : 8));
            const unsigned wl3 = st + W_OFF + (unsigned)(wave * RW * 1024) + 512u + (unsigned)(lane * 4);
            const unsigned dl = st + D_OFF + (unsigned)(wave * RW * 128) + (unsigned)(kg * 16);
            const unsigned dl2 = dl + (unsigned)(split << 6);
#pragma unroll
            for (int rw = 0; rw < RW; rw++)
            {
                // every result register is written by its read and first touched after the wait below
                if (BITS == 8)
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(wq[rw]) : "v"(wl), "n"(rw * 1024));
                else
                    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(wlo[rw]) : "v"(wl), "n"(rw * 1024));
                if (BITS == 6) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(whi[rw]) : "v"(wl3), "n"(rw * 1024));
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dq0[rw]) : "v"(dl), "n"(rw * 128));
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dq1[rw]) : "v"(dl2), "n"(rw * 128));
            }
#pragma unroll
            for (int rw = 0; rw < RW; rw++) // (the first wait already covers every read; the later ones only tie their registers to it)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wq[rw]), "+v"(wlo[rw]), "+v"(whi[rw]), "+v"(dq0[rw]), "+v"(dq1[rw]));
        }
        v8bf fa[RW], fb[RW];
#pragma unroll
        for (int rw = 0; rw < RW; rw++)
        {
            if (BITS == 8)
            {
                fa[rw] = bytes_to_bf16((unsigned)wq[rw][0], (unsigned)wq[rw][1]);
                fb[rw] = bytes_to_bf16((unsigned)wq[rw][2], (unsigned)wq[rw][3]);
            }
            else if (BITS == 4)
            {
                fa[rw] = nibbles_to_bf16((unsigned)wlo[rw][0]);
                fb[rw] = nibbles_to_bf16((unsigned)wlo[rw][1]);
            }
            else
                sixbit_to_bf16((unsigned)wlo[rw][0], (unsigned)wlo[rw][1], (unsigned)whi[rw], fa[rw], fb[rw]);
        }
        // the six operand fragments of a 16-row group (3 planes x 2 halves of the step); the next group's are requested before this one is multiplied
        union Act
        {
            v4i_bq i4;
            v8bf h;
        };
        Act ya[2][3], yb[2][3];
        const unsigned ra = st + (unsigned)rd_a, rb = st + (unsigned)rd_b;
        auto read_group = [&](int set, int cw) {
            const unsigned pa = ra + (unsigned)(cw * 2048), pb = rb + (unsigned)(cw * 2048);
            asm volatile("ds_read_b128 %0, %1" : "=v"(ya[set][0].i4) : "v"(pa));
            asm volatile("ds_read_b128 %0, %1" : "=v"(yb[set][0].i4) : "v"(pb));
            asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(ya[set][1].i4) : "v"(pa));
            asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(yb[set][1].i4) : "v"(pb));
            asm volatile("ds_read_b128 %0, %1 offset:16384" : "=v"(ya[set][2].i4) : "v"(pa));
            asm volatile("ds_read_b128 %0, %1 offset:16384" : "=v"(yb[set][2].i4) : "v"(pb));
        };
        read_group(0, 0);
#pragma unroll
        for (int cw = 0; cw < 4; cw++)
        {
            const int set = cw & 1;
            if (cw + 1 < 4)
            {
                read_group(set ^ 1, cw + 1);
                asm volatile("s_waitcnt lgkmcnt(6)"
                             : "+v"(ya[set][0].i4), "+v"(yb[set][0].i4), "+v"(ya[set][1].i4), "+v"(yb[set][1].i4), "+v"(ya[set][2].i4), "+v"(yb[set][2].i4));
            }
            else
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(ya[set][0].i4), "+v"(yb[set][0].i4), "+v"(ya[set][1].i4), "+v"(yb[set][1].i4), "+v"(ya[set][2].i4), "+v"(yb[set][2].i4));
            // the tiles' chains alternate, so that no instruction waits for the one right before it
            v4f t0[RW], t1[RW];
#pragma unroll
            for (int rw = 0; rw < RW; rw++) t0[rw] = t1[rw] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int pn = 0; pn < 3; pn++)
            {
#pragma unroll
                for (int rw = 0; rw < RW; rw++) t0[rw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[rw], ya[set][pn].h, t0[rw], 0, 0, 0);
#pragma unroll
                for (int rw = 0; rw < RW; rw++)
                {
                    if (HALVES)
                        t1[rw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[rw], yb[set][pn].h, t1[rw], 0, 0, 0);
                    else
                        t0[rw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[rw], yb[set][pn].h, t0[rw], 0, 0, 0);
                }
            }
#pragma unroll
            for (int rw = 0; rw < RW; rw++)
            {
                const float da[4] = {__int_as_float(dq0[rw][0]), __int_as_float(dq0[rw][1]), __int_as_float(dq0[rw][2]), __int_as_float(dq0[rw][3])};
                const float db[4] = {__int_as_float(dq1[rw][0]), __int_as_float(dq1[rw][1]), __int_as_float(dq1[rw][2]), __int_as_float(dq1[rw][3])};
#pragma unroll
                for (int r = 0; r < 4; r++)
                {
                    if (HALVES)
                        acc[rw][cw][r] = fmaf(t1[rw][r], db[r], fmaf(t0[rw][r], da[r], acc[rw][cw][r]));
                    else
                        acc[rw][cw][r] = fmaf(t0[rw][r], da[r], acc[rw][cw][r]);
                }
            }
        }
    }
    BQ_WAIT_VMCNT(0); // the surplus loads of the last steps must not outlive the workgroup's LDS

    // accumulator r of lane l: weight row (l/16)*4 + r of the tile, activation row l%16 of the 16-row group
#pragma unroll
    for (int rw = 0; rw < RW; rw++)
    {
        const int t = (blockIdx.x * 4 + wave) * RW + rw;
#pragma unroll
        for (int cw = 0; cw < 4; cw++)
        {
            const int i = row0 + cw * 16 + m;
            if (i >= M) continue;
#pragma unroll
            for (int r = 0; r < 4; r++)
            {
                const int j = t * 16 + kg * 4 + r;
                if (j < N)
                {
                    float v = acc[rw][cw][r];
                    if (bt >= 0) v = add_rn(mul_rn(load_c(c, bt, i, j, N), beta), v);
                    out[(size_t)i * out_stride + j] = mul_rn(v, alpha);
                }
            }
        }
    }
}

// ---- 5 to 16 activation rows in fp32, K up to 4096: weight-streaming shape, exact split made by a pass of its own ----
// Between the four rows per pass of the few-row kernel (LDS cannot hold more rows' planes) and the tiled kernel (too few
// workgroups to stream the weights at this row count): the few-row kernel's shape -- one workgroup per tile of 16 weight
// rows, 8 wavefronts of 8 K steps, every weight byte requested up front -- with the activations' three bf16 planes
// written beforehand, by blockquant_split_operands_kernel, in the very order the lanes load them: for K step s the six
// operand fragments (plane p, half h of the step) are 64 x 16 bytes each, lane l = activation row l % 16, K group l / 16.
// They come from L2 in a window of three steps kept three ahead of the arithmetic (24 VGPRs per step).
template<bool HALVES>
__global__ __launch_bounds__(256) void blockquant_split_operands_kernel(const float* __restrict__ a, size_t a_stride, int M_total, int K, int kblocks,
                                                                         const float* __restrict__ in_scales, uint4* __restrict__ frags)
{
    // blockIdx.y = pass: rows 16 * pass .. + 15, fragments of their own (kblocks * 384 vectors per pass)
    a += (size_t)blockIdx.y * 16 * a_stride;
    frags += (size_t)blockIdx.y * kblocks * 384;
    const int M = M_total - 16 * (int)blockIdx.y < 16 ? M_total - 16 * (int)blockIdx.y : 16;
    // one thread = one lane's 8 activations of one (step, half): fragments [step][plane * 2 + half][lane]
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= kblocks * 128) return;
    const int lane = idx & 63, h = (idx >> 6) & 1, step = idx >> 7;
    const int row = lane & 15, kg = lane >> 4;
    const int k = step * 64 + (HALVES ? h * 32 + kg * 8 : kg * 16 + h * 8);
    unsigned pl[3][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    if (row < M && k < K) // K % 16 == 0: the 8 values are all in or all out
    {
        const float* p = a + (size_t)row * a_stride + k;
#pragma unroll
        for (int e = 0; e < 4; e++)
        {
            unsigned hh[2][3];
#pragma unroll
            for (int o = 0; o < 2; o++)
            {
                float x = p[2 * e + o];
                if (in_scales) x = mul_rn(x, in_scales[k + 2 * e + o]);
                split_bf16x3(x, hh[o][0], hh[o][1], hh[o][2]);
            }
#pragma unroll
            for (int pn = 0; pn < 3; pn++) pl[pn][e] = (hh[0][pn] >> 16) | hh[1][pn];
        }
    }
#pragma unroll
    for (int pn = 0; pn < 3; pn++) frags[((size_t)step * 6 + pn * 2 + h) * 64 + lane] = make_uint4(pl[pn][0], pl[pn][1], pl[pn][2], pl[pn][3]);
}

template<int BITS, bool HALVES>
__global__ __launch_bounds__(512) void blockquant_rows16_bf16x3_kernel(const uint4* __restrict__ frags, int M_total, int N, int kblocks,
                                                                        const unsigned char* __restrict__ wpk, const float4* __restrict__ dpk, int split,
                                                                        const float* __restrict__ c, int bt, float alpha, float beta, float* __restrict__ out,
                                                                        size_t out_stride)
{
    static_assert(HALVES || BITS == 8, "4- and 6-bit fields come in the halves layout");
    // blockIdx.y = pass: activation rows 16 * pass .. + 15 (all passes in one launch: the weights of a tile are streamed once per
    // pass, from L2 after the first)
    const int M = M_total - 16 * (int)blockIdx.y < 16 ? M_total - 16 * (int)blockIdx.y : 16;
    frags += (size_t)blockIdx.y * kblocks * 384;
    if (c && (bt == 1 || bt == 2)) c += 16 * blockIdx.y;
    if (c && bt == 3) c += (size_t)16 * blockIdx.y * N;
    out += (size_t)16 * blockIdx.y * out_stride;
    constexpr int NB = 8, WIN = 3;
    constexpr int STEP_BYTES = 128 * BITS;
    __shared__ float4 red[8 * 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int tile = blockIdx.x;
    const int m = lane & 15, kg = lane >> 4;
    const int dper = HALVES ? 4 << split : 4;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    // K beyond 8 wavefronts x 8 steps (4096) goes round by round: round r of wavefront w is steps (r * wavefronts + w) * 8 .. + 8
    // (a round's requests go out when the round before it is done: its registers are the same)
    const int rounds = (kblocks + nwaves * NB - 1) / (nwaves * NB);
    for (int round = 0; round < rounds; round++)
    {
    const int kb_begin = (round * nwaves + wave) * NB;
    int nkb = kblocks - kb_begin;
    nkb = nkb > NB ? NB : nkb;
    nkb = nkb < 0 ? 0 : nkb;
    const int kb_base = nkb > 0 ? kb_begin : 0;

    const unsigned char* wt = wpk + ((size_t)tile * kblocks + kb_base) * STEP_BYTES;
    const float4* dt = dpk + ((size_t)tile * kblocks + kb_base) * dper;
    const uint4* ft = frags + (size_t)kb_base * 6 * 64 + lane;
    v4i_bq w[BITS == 8 ? NB : 1];
    v2i_bq w2[BITS != 8 ? NB : 1];
    int w1[BITS == 6 ? NB : 1];
    float4 d0[NB], d1[HALVES ? NB : 1];
    uint4 fr[WIN][6];
    auto load_w = [&](int i) {
        const unsigned char* ws = wt + (size_t)(i < nkb ? i : 0) * STEP_BYTES;
        if (BITS == 8)
            w[BITS == 8 ? i : 0] = __builtin_nontemporal_load(reinterpret_cast<const v4i_bq*>(ws) + lane);
        else
            w2[BITS != 8 ? i : 0] = __builtin_nontemporal_load(reinterpret_cast<const v2i_bq*>(ws) + lane);
        if (BITS == 6) w1[BITS == 6 ? i : 0] = __builtin_nontemporal_load(reinterpret_cast<const int*>(ws + 512) + lane);
    };
#define R16_LOAD_FRAGS(slot_, i_)                                                          \
    do                                                                                     \
    {                                                                                      \
        const uint4* f_ = ft + (size_t)((i_) < nkb ? (i_) : 0) * 6 * 64;                   \
        _Pragma("unroll") for (int q = 0; q < 6; q++) fr[slot_][q] = f_[q * 64];           \
    } while (0)
    // requests in the order their data is needed: the first steps' weights and operands interleaved, then the rest of the weights,
    // then the descales (a step beyond the wavefront's range reads step 0 again and meets a zero descale)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < WIN; i++)
    {
        load_w(i);
        __builtin_amdgcn_sched_barrier(0);
        R16_LOAD_FRAGS(i, i);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = WIN; i < NB; i++)
    {
        load_w(i);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < NB; i++)
    {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        const float4 a0 = dt[(size_t)(i < nkb ? i : 0) * dper + kg];
        d0[i] = i < nkb ? a0 : z;
        if (HALVES)
        {
            const float4 a1 = dt[(size_t)(i < nkb ? i : 0) * dper + (split << 2) + kg];
            d1[HALVES ? i : 0] = i < nkb ? a1 : z;
        }
    }
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int i = 0; i < NB; i++)
    {
        const int slot = i % WIN;
        v8bf fa, fb;
        if (BITS == 8)
        {
            fa = bytes_to_bf16((unsigned)w[BITS == 8 ? i : 0][0], (unsigned)w[BITS == 8 ? i : 0][1]);
            fb = bytes_to_bf16((unsigned)w[BITS == 8 ? i : 0][2], (unsigned)w[BITS == 8 ? i : 0][3]);
        }
        else if (BITS == 4)
        {
            fa = nibbles_to_bf16((unsigned)w2[BITS != 8 ? i : 0][0]);
            fb = nibbles_to_bf16((unsigned)w2[BITS != 8 ? i : 0][1]);
        }
        else
            sixbit_to_bf16((unsigned)w2[BITS != 8 ? i : 0][0], (unsigned)w2[BITS != 8 ? i : 0][1], (unsigned)w1[BITS == 6 ? i : 0], fa, fb);
        union
        {
            uint4 u;
            v8bf h;
        } y[6];
#pragma unroll
        for (int q = 0; q < 6; q++) y[q].u = fr[slot][q];
        v4f t0 = {0.f, 0.f, 0.f, 0.f}, t1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int pn = 0; pn < 3; pn++)
        {
            t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, y[pn * 2].h, t0, 0, 0, 0);
            if (HALVES)
                t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb, y[pn * 2 + 1].h, t1, 0, 0, 0);
            else
                t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb, y[pn * 2 + 1].h, t0, 0, 0, 0);
        }
        if (i + WIN < NB)
        {
            R16_LOAD_FRAGS(slot, i + WIN);
            __builtin_amdgcn_sched_barrier(0);
        }
        const float4 da = d0[i];
        if (HALVES)
        {
            const float4 db = d1[HALVES ? i : 0];
            acc[0] = fmaf(t1[0], db.x, fmaf(t0[0], da.x, acc[0]));
            acc[1] = fmaf(t1[1], db.y, fmaf(t0[1], da.y, acc[1]));
            acc[2] = fmaf(t1[2], db.z, fmaf(t0[2], da.z, acc[2]));
            acc[3] = fmaf(t1[3], db.w, fmaf(t0[3], da.w, acc[3]));
        }
        else
        {
            acc[0] = fmaf(t0[0], da.x, acc[0]);
            acc[1] = fmaf(t0[1], da.y, acc[1]);
            acc[2] = fmaf(t0[2], da.z, acc[2]);
            acc[3] = fmaf(t0[3], da.w, acc[3]);
        }
    }
#undef R16_LOAD_FRAGS
    } // rounds

    red[wave * 64 + lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    if (wave == 0 && m < M)
    {
        float4 f = red[lane];
        for (int w2i = 1; w2i < nwaves; w2i++)
        {
            const float4 o = red[w2i * 64 + lane];
            f.x = add_rn(f.x, o.x);
            f.y = add_rn(f.y, o.y);
            f.z = add_rn(f.z, o.z);
            f.w = add_rn(f.w, o.w);
        }
        const float frr[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int j = tile * 16 + kg * 4 + r;
            if (j < N)
            {
                float v = frr[r];
                if (bt >= 0) v = add_rn(mul_rn(load_c(c, bt, m, j, N), beta), v);
                out[(size_t)m * out_stride + j] = mul_rn(v, alpha);
            }
        }
    }
}

// One pass of up to 16 activation rows; nwaves = ceil(kblocks / NB) wavefronts per workgroup.
template<int BITS, bool HALVES, int NB, int MAXW, int MT, bool ACT_LDS, int AIN, bool INSC>
static int launch_upfront_one(const void* a, size_t a_stride, int M, int N, int K, int kblocks, const unsigned char* wpk, const float4* dpk, int split,
                              const float* in_scales, const float* c, int bt, float alpha, float beta, float* out, size_t out_stride, hipStream_t stream,
                              bool* handled, const BqMulti* multi)
{
    constexpr int AV = ACT_LDS ? (MT * NB * 8 + 63) / 64 : 1;
    constexpr int AROWS = ACT_LDS ? (AIN == 4 ? MT : (AV * 64 + NB * 8 - 1) / (NB * 8)) : 0;
    const int WAVE_BYTES = (HALVES ? 1024 << split : 1024) + (ACT_LDS ? (AIN == 4 ? 3 : 1) * AROWS * (NB * 128 + 128) : 16 * 144);
    const int nwaves = (kblocks + NB - 1) / NB;
    const size_t lds = (size_t)nwaves * WAVE_BYTES; // >= 1 KB per wavefront, which the final exchange reuses
    if (lds > 160 * 1024)
    {
        *handled = false;
        return NCNNHIP_OK;
    }
    auto kernel = blockquant8_upfront_kernel<BITS, HALVES, NB, MAXW, MT, ACT_LDS, AIN, INSC>;
    if (lds > 65536)
    {
        // more than the 64 KB a kernel gets by default: raise this kernel's limit once per device (the chip has 160 KB per compute
        // unit).  The flags only ever go from 0 to 1 and the call may be repeated, so a race between two first callers is harmless.
        static std::atomic<unsigned char> raised[64];
        int device = 0;
        NCNNHIP_CHECK(hipGetDevice(&device));
        if (device < 0 || device >= 64 || !raised[device].load(std::memory_order_acquire))
        {
            NCNNHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            if (device >= 0 && device < 64) raised[device].store(1, std::memory_order_release);
        }
    }
    BqMulti one;
    one.count = 0;
    const int grid = multi ? multi->tile_end[multi->count - 1] : (N + 15) / 16;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(nwaves * 64), lds, stream, a, a_stride, M, N, K, kblocks, wpk, dpk, split, in_scales, c, bt, alpha, beta,
                       out, out_stride, multi ? *multi : one);
    return launch_status("blockquant8_upfront_kernel");
}

// handled = false: the shape is left to the caller (K beyond 16384; fp16: more than 4 rows with K beyond 8192; fp32: more than 4 rows,
// or rows whose three planes do not fit in LDS together: the caller then passes fewer rows)
template<int BITS, bool HALVES, int AIN, bool INSC>
static int launch_blockquant8_upfront(const void* a, size_t a_stride, int M, int N, int K, const unsigned char* wpk, const float4* dpk, int split,
                                      const float* in_scales, const float* c, int bt, float alpha, float beta, float* out, size_t out_stride,
                                      hipStream_t stream, bool* handled, const BqMulti* multi = 0)
{
    const int kblocks = (K + 63) / 64;
    *handled = true;
#define UPFRONT(NB_, MAXW_, MT_, LDS_) \
    return launch_upfront_one<BITS, HALVES, NB_, MAXW_, MT_, LDS_, AIN, INSC>(a, a_stride, M, N, K, kblocks, wpk, dpk, split, in_scales, c, bt, alpha, beta, out, \
                                                                              out_stride, stream, handled, multi)
    if (M <= 4)
    {
        // decoding: 8 steps per wavefront while 8 or 16 wavefronts cover K (K up to 8192; measured against 16 steps on half
        // as many wavefronts: the same at 4096 x 4096, 3-6 % faster from 11008 rows up), then 12 and 16 steps on 16 wavefronts
        // (K = 11008: 15 wavefronts of 12).  Two rows run as four in the halves layout with fp16 activations (fewer kernels
        // to build; the staging reads row 0 again for the missing ones); with fp32 activations two rows have a kernel of their
        // own, because LDS holds three planes per row.
        constexpr bool TWO = !HALVES || AIN == 4;
        constexpr bool F32 = AIN == 4; // its three planes per row: four rows fit up to K = 4096, two up to 8192, one beyond (no kernels built for the rest)
        if (kblocks <= 64)
        {
            if (M == 1) UPFRONT(8, 8, 1, true);
            if constexpr (TWO) { if (M == 2) UPFRONT(8, 8, 2, true); }
            UPFRONT(8, 8, 4, true);
        }
        if (kblocks <= 128)
        {
            if (M == 1) UPFRONT(8, 16, 1, true);
            if constexpr (TWO) { if (M == 2) UPFRONT(8, 16, 2, true); }
            if constexpr (!F32) UPFRONT(8, 16, 4, true);
        }
        else if (kblocks <= 192)
        {
            if (M == 1) UPFRONT(12, 16, 1, true);
            if constexpr (!F32)
            {
                if constexpr (TWO) { if (M == 2) UPFRONT(12, 16, 2, true); }
                UPFRONT(12, 16, 4, true);
            }
        }
        else if (kblocks <= 256)
        {
            if (M == 1) UPFRONT(16, 16, 1, true);
            if constexpr (!F32)
            {
                if constexpr (TWO) { if (M == 2) UPFRONT(16, 16, 2, true); }
                UPFRONT(16, 16, 4, true);
            }
        }
    }
    else if constexpr (AIN == 2)
    {
        // up to 12 VGPRs per step (weights and the 16 rows' activations): 8 steps per wavefront, up to 16 wavefronts
        // (7.7 -> 6.7 us at 4096 x 4096 against 16 steps on 4 wavefronts)
        const int ntiles = (N + 15) / 16;
#ifndef BQ_PAIR_MIN_TILES
#define BQ_PAIR_MIN_TILES 1024
#endif
        if (kblocks <= 64 && ntiles >= BQ_PAIR_MIN_TILES && !multi)
        {
            // many weight rows: two tiles per workgroup share the activation registers
            const int nwaves = (kblocks + 7) / 8;
            const size_t lds = (size_t)nwaves * (2 * (HALVES ? 1024 << split : 1024) + 16 * 144);
            hipLaunchKernelGGL((blockquant8_rows16_pair_kernel<BITS, HALVES, 8, 8>), dim3((ntiles + 1) / 2), dim3(nwaves * 64), lds, stream,
                               static_cast<const __half*>(a), a_stride, M, N, K, kblocks, ntiles, wpk, dpk, split, c, bt, alpha, beta, out, out_stride);
            return launch_status("blockquant8_rows16_pair_kernel");
        }
        if (kblocks <= 64) UPFRONT(8, 8, 1, false);
        if (kblocks <= 128) UPFRONT(8, 16, 1, false);
    }
#undef UPFRONT
    *handled = false;
    return NCNNHIP_OK;
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
    if (M >= 32 && K % 32 == 0 && a_stride % 4 == 0 && al16(a_dev) && al16(b_dev) && (!in_scales_dev || al16(in_scales_dev)))
    {
        const int shift = block == 32 ? 5 : block == 64 ? 6 : 7;
        dim3 tiles(ceil_div(N, 64), ceil_div(M, 64));
        NCNNHIP_REQUIRE(tiles.y <= 65535, "ncnnhip_gemm_blockquant: more than 65535*64 activation rows");
#define LAUNCH_BQ_MFMA(BITS_) \
    hipLaunchKernelGGL(blockquant8_f32_mfma_kernel<BITS_>, tiles, dim3(256), 0, as_stream(stream), a_dev, a_stride, M, N, K, b_dev, shift, nblk, scales_dev, \
                       in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride)
        if (bits == 8)
            LAUNCH_BQ_MFMA(8);
        else if (bits == 6)
            LAUNCH_BQ_MFMA(6);
        else
            LAUNCH_BQ_MFMA(4);
#undef LAUNCH_BQ_MFMA
        return launch_status("blockquant8_f32_mfma_kernel");
    }
    if (K % 16 == 0 && al16(b_dev))
    {
        // streaming kernel: 16 weights (8 / 12 / 16 bytes) per lane and step
        if (bits == 8)
            return launch_blockquant8<float, 8>(a_dev, a_stride, M, N, K, b_dev, block, scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride,
                                                as_stream(stream));
        if (bits == 6)
            return launch_blockquant8<float, 6>(a_dev, a_stride, M, N, K, b_dev, block, scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride,
                                                as_stream(stream));
        return launch_blockquant8<float, 4>(a_dev, a_stride, M, N, K, b_dev, block, scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride,
                                            as_stream(stream));
    }
    const int packed = (int)(((size_t)K * bits + 7) / 8);
    hipLaunchKernelGGL(blockquant_generic_kernel, grid, dim3(256), 0, as_stream(stream), a_dev, a_stride, M, N, K, b_dev, bits, block, packed,
                       nblk, scales_dev, in_scales_dev, c_dev, bt, alpha, beta, out_dev, out_stride);
    return launch_status("blockquant_generic_kernel");
}

// the halves layout (see blockquant8_upfront_kernel): everything but 8-bit fields in blocks of 64 or 128
static inline bool halves_layout(int bits, int block)
{
    return bits != 8 || block == 32;
}

// field k of a row of the .bin's LSB-first stream (src/layer/gemm.cpp:318-336), sign-extended
static inline int host_field(const uint8_t* row, size_t row_bytes, int k, int bits)
{
    const size_t bit = (size_t)k * bits, byte = bit >> 3;
    unsigned v = row[byte];
    if (byte + 1 < row_bytes) v |= (unsigned)row[byte + 1] << 8;
    const int field = (int)((v >> (bit & 7)) & ((1u << bits) - 1u));
    const int sign = 1 << (bits - 1);
    return (field ^ sign) - sign;
}

int ncnnhip_blockquant_packed_size(int N, int K, int bits, int block, size_t* weight_bytes, size_t* descale_bytes)
{
    NCNNHIP_REQUIRE(N >= 1 && K >= 1, "ncnnhip_blockquant_packed_size: bad shape");
    NCNNHIP_REQUIRE(bits == 4 || bits == 6 || bits == 8, "ncnnhip_blockquant_packed_size: weight bits %d", bits);
    NCNNHIP_REQUIRE(block == 32 || block == 64 || block == 128, "ncnnhip_blockquant_packed_size: block size %d", block);
    NCNNHIP_REQUIRE(!halves_layout(bits, block) || K <= 16384, "ncnnhip_blockquant_packed_size: %d-bit fields in blocks of %d are packed for K up to 16384, got %d",
                    bits, block, K);
    const size_t tiles = (size_t)(N + 15) / 16, kblocks = (size_t)(K + 63) / 64;
    if (weight_bytes) *weight_bytes = tiles * kblocks * 128 * bits;
    if (descale_bytes) *descale_bytes = tiles * kblocks * 16 * sizeof(float) * (block == 32 ? 2 : 1);
    return NCNNHIP_OK;
}

int ncnnhip_blockquant_pack(const uint8_t* b_host, const float* scales_host, int N, int K, int bits, int block, uint8_t* packed_w_host,
                            float* packed_descale_host)
{
    NCNNHIP_REQUIRE(b_host && scales_host && packed_w_host && packed_descale_host, "ncnnhip_blockquant_pack: null pointer");
    int ret = ncnnhip_blockquant_packed_size(N, K, bits, block, 0, 0);
    if (ret) return ret;
    const int tiles = (N + 15) / 16, kblocks = (K + 63) / 64, nblk = (K + block - 1) / block;
    const size_t row_bytes = ((size_t)K * bits + 7) / 8;
    const bool halves = halves_layout(bits, block);
    const int bias = 1 << (bits - 1);
    const int dper = block == 32 ? 2 : 1; // descale groups per 64-wide step
    for (int t = 0; t < tiles; t++)
        for (int kb = 0; kb < kblocks; kb++)
        {
            uint8_t* wt = packed_w_host + ((size_t)t * kblocks + kb) * 128 * bits;
            float* dt = packed_descale_host + ((size_t)t * kblocks + kb) * 16 * dper;
            for (int l = 0; l < 64; l++)
            {
                unsigned u[16]; // the lane's 16 fields, offset to be non-negative
                for (int e = 0; e < 16; e++)
                {
                    const int j = t * 16 + (l & 15);
                    const int k = halves ? kb * 64 + (e >> 3) * 32 + (l >> 4) * 8 + (e & 7) : kb * 64 + (l >> 4) * 16 + e;
                    const int q = (j < N && k < K) ? host_field(b_host + (size_t)j * row_bytes, row_bytes, k, bits) : 0;
                    u[e] = (unsigned)(q + bias);
                }
                if (bits == 8)
                    for (int e = 0; e < 16; e++) wt[l * 16 + e] = (uint8_t)u[e];
                else if (bits == 4)
                {
                    unsigned d[2] = {0, 0};
                    for (int e = 0; e < 16; e++) d[e >> 3] |= u[e] << (4 * ((e & 7) >> 1) + 16 * (e & 1)); // pair p = fields 2p, 2p+1: nibbles p and p + 4
                    memcpy(wt + l * 8, d, 8);
                }
                else
                {
                    // pair P = fields 2P (low half) and 2P+1 (high half); dword P/2 holds pair P at bit 0 (P even) or 6 (P odd) for P < 6,
                    // pairs 6 and 7 lie in the dwords' top nibbles: low four bits in dword 0 / 1, high two bits in dword 2
                    unsigned d[3] = {0, 0, 0};
                    for (int P = 0; P < 6; P++) d[P >> 1] |= (u[2 * P] | (u[2 * P + 1] << 16)) << (6 * (P & 1));
                    for (int P = 6; P < 8; P++)
                    {
                        d[P - 6] |= ((u[2 * P] & 15u) | ((u[2 * P + 1] & 15u) << 16)) << 12;
                        d[2] |= ((u[2 * P] >> 4) | ((u[2 * P + 1] >> 4) << 16)) << (12 + 2 * (P - 6));
                    }
                    memcpy(wt + l * 8, d, 8);
                    memcpy(wt + 512 + l * 4, d + 2, 4);
                }
            }
            for (int h = 0; h < dper; h++)
                for (int r = 0; r < 16; r++)
                {
                    const int j = t * 16 + r;
                    const int blk = (kb * 64 + h * 32) / block;
                    const bool live = j < N && blk < nblk;
                    // same single rounded division the reference performs per block (gemm.cpp:465)
                    volatile float sc = live ? scales_host[(size_t)j * nblk + blk] : 1.f;
                    dt[h * 16 + r] = live ? 1.f / sc : 0.f;
                }
        }
    return NCNNHIP_OK;
}

// shared body of the two packed entry points; ain = 2 (fp16 activations) or 4 (fp32)
static int gemm_blockquant_packed(const char* who, const void* a_dev, int ain, size_t a_stride, int M, int N, int K, const uint8_t* packed_w_dev,
                                  const float* packed_descale_dev, int bits, int block, const float* in_scales_dev, const float* c_dev, int broadcast_type_c,
                                  float alpha, float beta, float* out_dev, size_t out_stride, void* stream)
{
    NCNNHIP_REQUIRE(a_dev && packed_w_dev && packed_descale_dev && out_dev, "%s: null pointer", who);
    NCNNHIP_REQUIRE(M >= 1 && N >= 1 && K >= 1 && K % 16 == 0, "%s: bad shape %d %d %d (K must be a multiple of 16)", who, M, N, K);
    NCNNHIP_REQUIRE(bits == 4 || bits == 6 || bits == 8, "%s: weight bits %d", who, bits);
    NCNNHIP_REQUIRE(block == 32 || block == 64 || block == 128, "%s: block size %d", who, block);
    NCNNHIP_REQUIRE(a_stride >= (size_t)K && a_stride % (16 / ain) == 0 && al16(a_dev), "%s: activation rows must be 16-byte aligned", who);
    NCNNHIP_REQUIRE(!in_scales_dev || al16(in_scales_dev), "%s: input scales must be 16-byte aligned", who);
    NCNNHIP_REQUIRE(out_stride >= (size_t)N, "%s: output stride too small", who);
    const int bt = c_dev ? broadcast_type_c : -1;
    NCNNHIP_REQUIRE(bt >= -1 && bt <= 4, "%s: C broadcast %d", who, bt);
    NCNNHIP_REQUIRE((size_t)(K + 63) / 64 * 64 <= 60 * 1024, "%s: K %d too large for the descale stage", who, K);
    const bool halves = halves_layout(bits, block);
    NCNNHIP_REQUIRE(!(halves || ain == 4) || K <= 16384, "%s: K %d beyond 16384 has a kernel only for 8-bit fields in blocks of 64 or 128 with fp16 activations", who, K);
    const int tiles = (N + 15) / 16, kblocks = (K + 63) / 64;
    const float4* dpk = reinterpret_cast<const float4*>(packed_descale_dev);
    const int split = block == 32 ? 1 : 0;
    hipStream_t st = as_stream(stream);
    // one pass over the weights for rows m0 .. m0 + mc - 1
    auto upfront = [&](int m0, int mc, bool* handled) -> int {
        const float* cc = c_dev;
        if (cc && (bt == 1 || bt == 2)) cc += m0;
        if (cc && bt == 3) cc += (size_t)m0 * N;
        const void* ap = static_cast<const char*>(a_dev) + (size_t)m0 * a_stride * ain;
        float* op = out_dev + (size_t)m0 * out_stride;
#define UP(BITS_, HALVES_, AIN_, INSC_) \
    return launch_blockquant8_upfront<BITS_, HALVES_, AIN_, INSC_>(ap, a_stride, mc, N, K, packed_w_dev, dpk, split, in_scales_dev, cc, bt, alpha, beta, op, out_stride, \
                                                                   st, handled)
#define UP_BITS(AIN_, INSC_)                 \
    if (!halves) UP(8, false, AIN_, INSC_);  \
    if (bits == 8) UP(8, true, AIN_, INSC_); \
    if (bits == 6) UP(6, true, AIN_, INSC_); \
    UP(4, true, AIN_, INSC_)
        if (ain == 2)
        {
            UP_BITS(2, false);
        }
        if (in_scales_dev)
        {
            UP_BITS(4, true);
        }
        UP_BITS(4, false);
#undef UP_BITS
#undef UP
    };
    const int pass = ain == 4 ? 4 : 16; // rows per pass at most
    for (int m0 = 0; m0 < M; m0 += pass)
    {
        const int mc = M - m0 < pass ? M - m0 : pass;
        bool handled = false;
        int ret = upfront(m0, mc, &handled);
        if (ret != NCNNHIP_OK) return ret;
        if (handled) continue;
        if (halves || ain == 4)
        {
            // rows that do not fit in LDS together (long K; fp32: three planes per row): four, two, one at a time
            for (int m1 = m0; m1 < m0 + mc;)
            {
                int rows = m0 + mc - m1 < 4 ? m0 + mc - m1 : 4;
                for (;;)
                {
                    ret = upfront(m1, rows, &handled);
                    if (ret != NCNNHIP_OK) return ret;
                    if (handled || rows == 1) break;
                    rows = rows > 2 ? 2 : 1;
                }
                NCNNHIP_REQUIRE(handled, "%s: no kernel for M %d K %d", who, M, K);
                m1 += rows;
            }
            continue;
        }
        const __half* ah = static_cast<const __half*>(a_dev);
        const float* cc = c_dev;
        if (cc && (bt == 1 || bt == 2)) cc += m0;
        if (cc && bt == 3) cc += (size_t)m0 * N;
        const size_t act_bytes = (size_t)mc * kblocks * 64 * sizeof(__half);
        if (act_bytes <= 32768 && tiles >= 512) // measured: pays from about 8192 weight rows (up to four rows of 4096), not for long rows (K = 11008) or few tiles
            hipLaunchKernelGGL((blockquant8_mfma_kernel<BQ_MFMA_NS_LDS, 1, true>), dim3(tiles), dim3(256), (size_t)kblocks * 64 + act_bytes, st,
                               ah + (size_t)m0 * a_stride, a_stride, mc, N, K, kblocks, reinterpret_cast<const v4i_bq*>(packed_w_dev), dpk, cc, bt, alpha, beta,
                               out_dev + (size_t)m0 * out_stride, out_stride);
        else
            hipLaunchKernelGGL((blockquant8_mfma_kernel<BQ_MFMA_NS, BQ_MFMA_U, false>), dim3(tiles), dim3(256), (size_t)kblocks * 64, st,
                               ah + (size_t)m0 * a_stride, a_stride, mc, N, K, kblocks, reinterpret_cast<const v4i_bq*>(packed_w_dev), dpk, cc, bt, alpha, beta,
                               out_dev + (size_t)m0 * out_stride, out_stride);
    }
    return launch_status("blockquant8_mfma_kernel");
}

int ncnnhip_gemm_blockquant_packed_f16a(const uint16_t* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* packed_w_dev,
                                        const float* packed_descale_dev, int bits, int block, const float* c_dev, int broadcast_type_c, float alpha,
                                        float beta, float* out_dev, size_t out_stride, void* stream)
{
    return gemm_blockquant_packed("ncnnhip_gemm_blockquant_packed_f16a", a_dev, 2, a_stride, M, N, K, packed_w_dev, packed_descale_dev, bits, block, 0, c_dev,
                                  broadcast_type_c, alpha, beta, out_dev, out_stride, stream);
}

int ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(int M, int K, size_t* bytes)
{
    NCNNHIP_REQUIRE(bytes && M >= 1 && K >= 1, "ncnnhip_gemm_blockquant_packed_rows_workspace_bytes: bad arguments");
    const size_t Mp = ((size_t)M + 63) / 64 * 64, Kp = ((size_t)K + 63) / 64 * 64;
    *bytes = 3 * Mp * Kp * sizeof(unsigned short);
    return NCNNHIP_OK;
}

int ncnnhip_gemm_blockquant_packed_rows(const float* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* packed_w_dev, const float* packed_descale_dev,
                                        int bits, int block, const float* in_scales_dev, const float* c_dev, int broadcast_type_c, float alpha, float beta,
                                        float* out_dev, size_t out_stride, void* workspace_dev, size_t workspace_bytes, void* stream)
{
    const char* who = "ncnnhip_gemm_blockquant_packed_rows";
    NCNNHIP_REQUIRE(a_dev && packed_w_dev && packed_descale_dev && out_dev && workspace_dev, "%s: null pointer", who);
    NCNNHIP_REQUIRE(M >= 1 && N >= 1 && K >= 1 && K % 16 == 0, "%s: bad shape %d %d %d (K must be a multiple of 16)", who, M, N, K);
    NCNNHIP_REQUIRE(bits == 4 || bits == 6 || bits == 8, "%s: weight bits %d", who, bits);
    NCNNHIP_REQUIRE(block == 32 || block == 64 || block == 128, "%s: block size %d", who, block);
    NCNNHIP_REQUIRE(a_stride >= (size_t)K && out_stride >= (size_t)N, "%s: stride too small", who);
    const int bt = c_dev ? broadcast_type_c : -1;
    NCNNHIP_REQUIRE(bt >= -1 && bt <= 4, "%s: C broadcast %d", who, bt);
    const bool halves = halves_layout(bits, block);
    NCNNHIP_REQUIRE(!halves || K <= 16384, "%s: %d-bit fields in blocks of %d are packed for K up to 16384, got %d", who, bits, block, K);
    size_t need = 0;
    ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(M, K, &need);
    NCNNHIP_REQUIRE(workspace_bytes >= need && al16(workspace_dev), "%s: the workspace must hold %zu bytes, 16-byte aligned (got %zu)", who, need, workspace_bytes);
    const int Mp = (M + 63) / 64 * 64, Kp = (K + 63) / 64 * 64, kblocks = Kp / 64, ntiles = (N + 15) / 16;
    NCNNHIP_REQUIRE(Mp / 64 <= 65535, "%s: more than 65535*64 activation rows", who);
    hipStream_t st = as_stream(stream);
    const float4* dpk = reinterpret_cast<const float4*>(packed_descale_dev);
    const int split = block == 32 ? 1 : 0;
    // Which form: the 16-row passes (all in one launch, spread over the chip; every pass streams the weights again, from L2
    // after the first) cost about 5 us + passes x weight bytes at 2 TB/s; the tiled kernel's 64-row tiles about 6 us + K / 85
    // whatever the row count up to 64 (18-20 us at K = 1024, 54-58 at K = 4096).  Measured on 16..96 rows: 3072 x 1024
    // 6.9..12.5 us against 18..20 tiled, 4096 x 4096 11.7..52.7 against 55..58, 11008 x 4096 26.8 / 49 / 72 / 90 at
    // 16 / 32 / 48 / 64 rows against 57..59.
    const double weight_mb = (double)N * (double)K * bits / 8.0 / 1.0e6;
    const int passes16 = (M + 15) / 16;
    if (M <= 128 && 5.0 + passes16 * weight_mb / 2.0 <= 6.0 + K / 85.0)
    {
        // fewer rows than the tiled kernel can spread over the chip: 16 rows per pass in the weight-streaming shape
        // (the fragments of a pass take kblocks * 6 KB of the workspace: all passes together no more than the planes it was sized for)
        uint4* frags = static_cast<uint4*>(workspace_dev);
        const int nwaves = kblocks >= 64 ? 8 : (kblocks + 7) / 8; // K beyond 4096: rounds of 8 x 8 steps
        const unsigned passes = (unsigned)((M + 15) / 16);
        const dim3 sgrid((kblocks * 128 + 255) / 256, passes);
        if (halves)
            hipLaunchKernelGGL(blockquant_split_operands_kernel<true>, sgrid, dim3(256), 0, st, a_dev, a_stride, M, K, kblocks, in_scales_dev, frags);
        else
            hipLaunchKernelGGL(blockquant_split_operands_kernel<false>, sgrid, dim3(256), 0, st, a_dev, a_stride, M, K, kblocks, in_scales_dev, frags);
#define ROWS16(BITS_, HALVES_)                                                                                                                                 \
    hipLaunchKernelGGL((blockquant_rows16_bf16x3_kernel<BITS_, HALVES_>), dim3(ntiles, passes), dim3(nwaves * 64), 0, st, frags, M, N, kblocks, packed_w_dev, dpk, split, \
                       c_dev, bt, alpha, beta, out_dev, out_stride)
        if (!halves)
            ROWS16(8, false);
        else if (bits == 8)
            ROWS16(8, true);
        else if (bits == 6)
            ROWS16(6, true);
        else
            ROWS16(4, true);
#undef ROWS16
        return launch_status("blockquant_rows16_bf16x3_kernel");
    }
    unsigned short* planes = static_cast<unsigned short*>(workspace_dev);
    const size_t vectors = (size_t)Mp * (Kp / 8);
    hipLaunchKernelGGL(blockquant_split_activations_kernel, dim3((unsigned)((vectors + 256 * SPLIT_VECS - 1) / (256 * SPLIT_VECS))), dim3(256), 0, st, a_dev, a_stride, M, K, in_scales_dev, planes, Mp,
                       Kp);
    // Two tiles per wavefront and two stages: 66 KB of LDS, so two workgroups share a compute unit and one's loads, waits and
    // vector work overlap the other's matrix-core instructions.  Measured at 1024 x 4096 x 4096 / 2048 x 11008 x 4096: 135 / 616 us;
    // four tiles per wavefront with three stages (one workgroup per unit, half the LDS reads per instruction) 145 / 714 us; two
    // tiles with four stages (one workgroup per unit) 172 / 795 us.  While that leaves fewer workgroups than the chip has compute
    // units, one tile per wavefront (64 weight rows per workgroup) doubles them: 128 x 4096 x 4096 77 -> 58 us, 256 rows 82 -> 63,
    // 512 x 1024 x 1024 28.6 -> 22.3.
    // One, two or three tiles per wavefront (64, 128 or 192 weight rows per workgroup).  The chip holds 512 workgroups at once:
    // where some choice fits in one round, the one with the most workgroups; else the fewest rounds weighted by a
    // workgroup's cost (0.68 : 1 : 1.4, measured).  1500 x 3072 x 1024 is 576 workgroups with two tiles - a second round
    // for 64 of them - and 384 with three: 63.6 -> 55.9 us; 1100 x 4096 x 4096 189 -> 173; 2048 x 11008 x 4096 672 -> 650.
    int rw_tiles = 2;
    {
        const long long row_tiles = Mp / 64;
        const double cost[4] = {0.0, 0.68, 1.0, 1.4};
        int fits = 0;
        double best = 0.0;
        for (int rw = 1; rw <= 3; rw++)
        {
            const long long groups = (long long)((ntiles + 4 * rw - 1) / (4 * rw)) * row_tiles;
            if (groups <= 512)
            {
                if (!fits) rw_tiles = rw; // the smallest such rw has the most workgroups
                fits = 1;
            }
            else if (!fits)
            {
                const double t = (double)((groups + 511) / 512) * cost[rw];
                if (best == 0.0 || t < best)
                {
                    best = t;
                    rw_tiles = rw;
                }
            }
        }
    }
    // (a ring of four stages where a workgroup has its compute unit to itself measured the same as two: 57.6 against 57.8 us at 128 x 4096 x 4096)
    const dim3 grid((ntiles + 4 * rw_tiles - 1) / (4 * rw_tiles), Mp / 64);
#define ROWS_RW(BITS_, HALVES_, RW_, STAGES_)                                                                                                                      \
    do                                                                                                                                                             \
    {                                                                                                                                                              \
        auto kernel = blockquant_rows_bf16x3_kernel<BITS_, HALVES_, STAGES_, RW_>;                                                                                 \
        const size_t lds = (size_t)(STAGES_) * (3 * 64 * 128 + 4 * (RW_) * 1024 + 4 * (RW_) * 128);                                                                  \
        static std::atomic<unsigned char> raised[64];                                                                                                              \
        int device = 0;                                                                                                                                            \
        NCNNHIP_CHECK(hipGetDevice(&device));                                                                                                                      \
        if (device < 0 || device >= 64 || !raised[device].load(std::memory_order_acquire))                                                                         \
        {                                                                                                                                                          \
            NCNNHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                     \
            if (device >= 0 && device < 64) raised[device].store(1, std::memory_order_release);                                                                    \
        }                                                                                                                                                          \
        hipLaunchKernelGGL(kernel, grid, dim3(256), lds, st, planes, Mp, Kp, M, N, kblocks, ntiles, packed_w_dev, dpk, split, c_dev, bt, alpha, beta, out_dev, out_stride); \
    } while (0)
#define ROWS(BITS_, HALVES_)            \
    do                                  \
    {                                   \
        if (rw_tiles == 1)                 \
            ROWS_RW(BITS_, HALVES_, 1, 2); \
        else if (rw_tiles == 3)            \
            ROWS_RW(BITS_, HALVES_, 3, 2); \
        else                               \
            ROWS_RW(BITS_, HALVES_, 2, 2); \
    } while (0)
    if (!halves)
        ROWS(8, false);
    else if (bits == 8)
        ROWS(8, true);
    else if (bits == 6)
        ROWS(6, true);
    else
        ROWS(4, true);
#undef ROWS
#undef ROWS_RW
    return launch_status("blockquant_rows_bf16x3_kernel");
}

int ncnnhip_gemm_blockquant_packed_supported(int K)
{
    return K >= 1 && K % 16 == 0 && K <= 16384;
}

int ncnnhip_gemm_blockquant_packed(const float* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* packed_w_dev, const float* packed_descale_dev,
                                   int bits, int block, const float* in_scales_dev, const float* c_dev, int broadcast_type_c, float alpha, float beta,
                                   float* out_dev, size_t out_stride, void* stream)
{
    return gemm_blockquant_packed("ncnnhip_gemm_blockquant_packed", a_dev, 4, a_stride, M, N, K, packed_w_dev, packed_descale_dev, bits, block, in_scales_dev,
                                  c_dev, broadcast_type_c, alpha, beta, out_dev, out_stride, stream);
}

// Several matrices on the same activation rows in one launch (see BqMulti).  Shapes the one-pass kernel does not take (more
// than 16 rows of fp16 or 4 of fp32 activations, long K) run matrix by matrix through the single-matrix entries.
int ncnnhip_gemm_blockquant_packed_multi(const void* a_dev, int a_elemsize, size_t a_stride, int M, int K, int count, const int* N,
                                         const uint8_t* const* packed_w_dev, const float* const* packed_descale_dev, int bits, int block,
                                         const float* in_scales_dev, const float* const* c_dev, const int* broadcast_type_c, const float* alpha,
                                         const float* beta, float* const* out_dev, const size_t* out_stride, void* stream)
{
    const char* who = "ncnnhip_gemm_blockquant_packed_multi";
    NCNNHIP_REQUIRE(a_dev && N && packed_w_dev && packed_descale_dev && out_dev && out_stride, "%s: null pointer", who);
    NCNNHIP_REQUIRE(count >= 1 && count <= BQ_MULTI_MAX, "%s: %d matrices (1 to %d)", who, count, BQ_MULTI_MAX);
    NCNNHIP_REQUIRE(a_elemsize == 2 || a_elemsize == 4, "%s: activations of %d bytes", who, a_elemsize);
    NCNNHIP_REQUIRE(a_elemsize == 4 || !in_scales_dev, "%s: input scales come with fp32 activations", who);
    auto single = [&](int i) -> int {
        const float* ci = c_dev ? c_dev[i] : 0;
        return gemm_blockquant_packed(who, a_dev, a_elemsize, a_stride, M, N[i], K, packed_w_dev[i], packed_descale_dev[i], bits, block, in_scales_dev, ci,
                                      broadcast_type_c ? broadcast_type_c[i] : -1, alpha ? alpha[i] : 1.f, beta ? beta[i] : 1.f, out_dev[i], out_stride[i], stream);
    };
    const bool halves = halves_layout(bits, block);
    bool one_pass = count > 1 && M >= 1 && K >= 1 && K % 16 == 0 && K <= 16384 && M <= (a_elemsize == 2 ? 16 : 4) && (bits == 4 || bits == 6 || bits == 8) &&
                    (block == 32 || block == 64 || block == 128) && a_stride >= (size_t)K && a_stride % (16 / a_elemsize) == 0 && al16(a_dev) &&
                    (!in_scales_dev || al16(in_scales_dev));
    BqMulti mm;
    mm.count = count;
    long long tiles = 0;
    for (int i = 0; i < count && one_pass; i++)
    {
        const int bt = (c_dev && c_dev[i]) ? (broadcast_type_c ? broadcast_type_c[i] : -1) : -1;
        one_pass = packed_w_dev[i] && packed_descale_dev[i] && out_dev[i] && N[i] >= 1 && out_stride[i] >= (size_t)N[i] && bt >= -1 && bt <= 4;
        tiles += (N[i] + 15) / 16;
        one_pass = one_pass && tiles < (1ll << 31);
        mm.tile_end[i] = (int)tiles;
        mm.N[i] = N[i];
        mm.bt[i] = bt;
        mm.alpha[i] = alpha ? alpha[i] : 1.f;
        mm.beta[i] = beta ? beta[i] : 1.f;
        mm.wpk[i] = packed_w_dev[i];
        mm.dpk[i] = reinterpret_cast<const float4*>(packed_descale_dev[i]);
        mm.c[i] = bt >= 0 ? c_dev[i] : 0;
        mm.out[i] = out_dev[i];
        mm.out_stride[i] = out_stride[i];
    }
    for (int i = count; i < BQ_MULTI_MAX; i++)
    {
        mm.tile_end[i] = (int)tiles, mm.N[i] = 0, mm.bt[i] = -1, mm.alpha[i] = mm.beta[i] = 1.f;
        mm.wpk[i] = 0, mm.dpk[i] = 0, mm.c[i] = 0, mm.out[i] = 0, mm.out_stride[i] = 0;
    }
    if (one_pass)
    {
        const int split = block == 32 ? 1 : 0;
        hipStream_t st = as_stream(stream);
        bool handled = false;
        int ret = NCNNHIP_OK;
        auto up = [&]() -> int {
#define UPM(BITS_, HALVES_, AIN_, INSC_)                                                                                                                        \
    return launch_blockquant8_upfront<BITS_, HALVES_, AIN_, INSC_>(a_dev, a_stride, M, N[0], K, mm.wpk[0], mm.dpk[0], split, in_scales_dev, mm.c[0], mm.bt[0], \
                                                                   mm.alpha[0], mm.beta[0], mm.out[0], mm.out_stride[0], st, &handled, &mm)
#define UPM_BITS(AIN_, INSC_)                 \
    if (!halves) UPM(8, false, AIN_, INSC_);  \
    if (bits == 8) UPM(8, true, AIN_, INSC_); \
    if (bits == 6) UPM(6, true, AIN_, INSC_); \
    UPM(4, true, AIN_, INSC_)
            if (a_elemsize == 2)
            {
                UPM_BITS(2, false);
            }
            if (in_scales_dev)
            {
                UPM_BITS(4, true);
            }
            UPM_BITS(4, false);
#undef UPM_BITS
#undef UPM
        };
        ret = up();
        if (ret != NCNNHIP_OK) return ret;
        if (handled) return NCNNHIP_OK;
    }
    for (int i = 0; i < count; i++)
    {
        const int ret = single(i);
        if (ret != NCNNHIP_OK) return ret;
    }
    return NCNNHIP_OK;
}

int ncnnhip_gemm_blockquant_f16a(const uint16_t* a_dev, size_t a_stride, int M, int N, int K, const uint8_t* b_dev, int bits,
                                 int block, const float* scales_dev, float* out_dev, size_t out_stride, void* stream)
{
    int ret = check_blockquant(a_dev, b_dev, scales_dev, out_dev, M, N, K, bits, block, 0, -1);
    if (ret) return ret;
    NCNNHIP_REQUIRE(K % 16 == 0 && al16(b_dev), "ncnnhip_gemm_blockquant_f16a: needs K %% 16 == 0 and 16-byte aligned weights");
    NCNNHIP_REQUIRE(a_stride >= (size_t)K && out_stride >= (size_t)N, "ncnnhip_gemm_blockquant_f16a: stride too small");
    const __half* ah = reinterpret_cast<const __half*>(a_dev);
    if (bits == 8)
        return launch_blockquant8<__half, 8>(ah, a_stride, M, N, K, b_dev, block, scales_dev, (const float*)0, (const float*)0, -1, 1.f, 1.f, out_dev, out_stride,
                                             as_stream(stream));
    if (bits == 6)
        return launch_blockquant8<__half, 6>(ah, a_stride, M, N, K, b_dev, block, scales_dev, (const float*)0, (const float*)0, -1, 1.f, 1.f, out_dev, out_stride,
                                             as_stream(stream));
    return launch_blockquant8<__half, 4>(ah, a_stride, M, N, K, b_dev, block, scales_dev, (const float*)0, (const float*)0, -1, 1.f, 1.f, out_dev, out_stride,
                                         as_stream(stream));
}

} // extern "C"
