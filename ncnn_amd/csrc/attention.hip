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
#include <limits.h>

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
                                                            size_t kv_stride, float* __restrict__ out, size_t q_stride, float q_scale)
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
        qs[e] = t < rows ? mul_rn(q[(size_t)(i0 + t) * q_stride + h * head_dim + l], q_scale) : 0.f;
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

// ---- the same on the fp32 matrix cores, for head dimensions 32 / 64 / 96 / 128 ------------------------------------
// One workgroup = 32 query rows of one head; its 4 wavefronts take key tiles (32 keys) in turn and each keeps a
// running softmax (maximum m, sum l, unnormalised output) for its share; the shares are merged at the end.
// Everything is computed transposed, so that both MFMA operands come straight from where they lie:
//   S^T = K Q^T : A = k[channel][key] read coalesced along the keys, B = q values held in registers.  The result has
//                 keys down the registers and the 32 queries across the lanes: a query's softmax is per-lane arithmetic
//                 plus one exchange with lane^32.
//   O^T = V P^T : B = exp(S^T - m) is used from the accumulator registers as they are: MFMA step kk of half hh is given
//                 key 8*(kk/4) + 4*hh + kk%4, the key that register kk of that lane holds; A = v[channel][key] with the
//                 same key order, four 16-byte loads per lane and 32 channels.
// Scores and products are fp32 throughout; the order of the additions (and the running rescale by exp(m_old - m_new))
// differs from the reference's two-pass softmax: compared with an fp32 tolerance.
// e^x for x <= 0 in three instructions: the hardware's 2^y (1 ulp) on y = x * log2(e).  Rounding y moves the result by at most
// |y| * 2^-24 of itself, so a term of relative size e^x carries an error below 2^-24 * |x| e^x <= 2.2e-8 of the row's largest
// term; -inf and differences beyond the exponent range give 0.  (The library's expf spends 14 instructions on range
// reduction and range checks; with 16 probabilities per lane and tile that was the largest part of the vector work.)
__device__ __forceinline__ float exp_of_nonpositive(float x)
{
    return __builtin_amdgcn_exp2f(mul_rn(x, 1.44269504088896341f));
}

typedef float v16f_at __attribute__((ext_vector_type(16)));
typedef float v4f_at __attribute__((ext_vector_type(4)));

// Nothing moves across it: the empty asm holds memory accesses in place for the passes that work on the IR, the scheduling
// barrier holds every instruction in place for the machine scheduler.
#define ATT_PHASE_BOUNDARY()                \
    do                                      \
    {                                       \
        asm volatile("" ::: "memory");      \
        __builtin_amdgcn_sched_barrier(0);  \
    } while (0)

// the 16 values of one channel that a lane feeds to the products of O^T: keys j0 + 8*(kk/4) + 4*hh + kk%4
__device__ __forceinline__ void load_value_block(float (&vv)[16], const float* __restrict__ vr, int j0, int hh, int dst, bool vec)
{
    if (vec)
    {
#pragma unroll
        for (int a = 0; a < 4; a++)
        {
            const v4f_at t4 = *reinterpret_cast<const v4f_at*>(vr + j0 + 8 * a + 4 * hh);
#pragma unroll
            for (int e = 0; e < 4; e++) vv[4 * a + e] = t4[e];
        }
    }
    else
    {
#pragma unroll
        for (int kk = 0; kk < 16; kk++)
        {
            const int key = j0 + 8 * (kk >> 2) + 4 * hh + (kk & 3);
            vv[kk] = vr[key < dst ? key : dst - 1]; // past the end: its probability is 0
        }
    }
}

// One tile's step of the running softmax of a query (lanes l and l^32 hold the two halves of its 32 scores): scores
// become exp(score - new maximum), the running sum and maximum are brought up to date, and the factor that rescales what
// was accumulated under the old maximum is returned.
__device__ __forceinline__ float running_softmax_step(v16f_at& s, float& m, float& l)
{
    float mx = -FLT_MAX;
#pragma unroll
    for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m, mx);
    const float corr = exp_of_nonpositive(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++)
    {
        s[r] = exp_of_nonpositive(s[r] - m_new);
        psum += s[r];
    }
    psum += __shfl_xor(psum, 32);
    l = l * corr + psum;
    m = m_new;
    return corr;
}

template<int HD>
__global__ __launch_bounds__(256) void attention_f32_mfma_kernel(const float* __restrict__ q, const float* __restrict__ kt, const float* __restrict__ vt,
                                                                 const float* __restrict__ mask, int mask_heads, int embed_dim, int src, int dst,
                                                                 size_t kv_stride, float* __restrict__ out, int v_vec_ok, int keys_per_split,
                                                                 float* __restrict__ partial, size_t q_stride, float q_scale)
{
    // keys_per_split > 0: blockIdx.z takes keys [z*keys_per_split, ...) and leaves (m, l, unnormalised o) in `partial`
    // for attention_merge_kernel; 0: the workgroup sees every key and writes the result
    constexpr int CB = HD / 32;
    constexpr int LD = 33;
    __shared__ float o_s[HD * LD];
    __shared__ float m_s[4][32], l_s[4][32];
    const int h = blockIdx.y, i0 = blockIdx.x * 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hh = lane >> 5;
    const int qi = i0 + l32 < src ? i0 + l32 : src - 1; // lanes past the last query repeat it; nothing of theirs is stored

    float qreg[HD / 2];
#pragma unroll
    for (int kk = 0; kk < HD / 2; kk++) qreg[kk] = mul_rn(q[(size_t)qi * q_stride + h * HD + 2 * kk + hh], q_scale);

    v16f_at o[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[cb][r] = 0.f;
    float m = -FLT_MAX, l = 0.f;

    const float* kh = kt + (size_t)h * HD * kv_stride;
    const float* vh = vt + (size_t)h * HD * kv_stride;
    const float* mrow = mask ? mask + ((size_t)(mask_heads > 1 ? h : 0) * src + qi) * dst : nullptr;

    const int key_begin = keys_per_split > 0 ? (int)blockIdx.z * keys_per_split : 0;
    const int key_end = keys_per_split > 0 && key_begin + keys_per_split < dst ? key_begin + keys_per_split : dst; // a multiple of 32, or dst
    // Key loads: channel pair kk starts at a wave-uniform address (scalar registers), the lane adds one 32-bit offset that
    // is the same for every kk (the host checks that kv_stride + dst fits) - 64-bit per-lane addresses for 32 rows would
    // cost 64 registers and with them the second wavefront per SIMD.
    //
    // The loop is pipelined by hand over the wavefront's tiles of 32 keys.  Iteration t:
    //   (1) request the values of tile t (and its mask values), (2) add the mask / drop keys past the end in the scores of
    //   tile t, which the previous iteration left in s_cur, (3) the products of S^T for tile t+1 (its keys were requested
    //   one iteration ago) together with the softmax arithmetic of tile t: one block of code, the vector instructions
    //   issue while the matrix pipe works on the chain of products, (4) request the keys of tile t+2, (5) the products
    //   of O^T for tile t.
    // The phase boundaries keep the compiler from sinking loads back to their first use (left to itself it keeps one to
    // eight loads in flight and a wavefront stands on each latency in turn).
    constexpr int VB = CB <= 2 ? CB : 1; // value blocks requested ahead: all of them while the registers last, else one at a time
    const int j_first = key_begin + wave * 32;
    float kreg[HD / 2];
    v16f_at s_cur;
#pragma unroll
    for (int r = 0; r < 16; r++) s_cur[r] = 0.f;
    if (j_first < key_end)
    {
        {
            const unsigned koff = (unsigned)hh * (unsigned)kv_stride + (unsigned)(j_first + l32 < dst ? j_first + l32 : dst - 1);
#pragma unroll
            for (int kk = 0; kk < HD / 2; kk++) kreg[kk] = (kh + (size_t)(2 * kk) * kv_stride)[koff];
        }
        ATT_PHASE_BOUNDARY();
#pragma unroll
        for (int kk = 0; kk < HD / 2; kk++) s_cur = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[kk], qreg[kk], s_cur, 0, 0, 0);
        asm volatile("" : "+v"(s_cur)); // the products are pure arithmetic and would be sunk past the boundary to their first use: this pins them before it
        ATT_PHASE_BOUNDARY();
        {
            // past the last tile of this wavefront the loads repeat a key and are never used
            const int jn = j_first + 128 < key_end ? j_first + 128 : j_first;
            const unsigned koff = (unsigned)hh * (unsigned)kv_stride + (unsigned)(jn + l32 < dst ? jn + l32 : dst - 1);
#pragma unroll
            for (int kk = 0; kk < HD / 2; kk++) kreg[kk] = (kh + (size_t)(2 * kk) * kv_stride)[koff];
        }
    }
    for (int j0 = j_first; j0 < key_end; j0 += 128)
    {
        const bool full = j0 + 32 <= dst;
        float vv[VB][16];
        if constexpr (CB <= 2)
        {
#pragma unroll
            for (int cb = 0; cb < CB; cb++) load_value_block(vv[cb], vh + (size_t)(cb * 32 + l32) * kv_stride, j0, hh, dst, full && v_vec_ok);
        }
        // register r of this lane: key j0 + 8*(r/4) + 4*hh + r%4 for query l32
        if (mrow)
        {
            // all 16 mask values requested before the first is used; a key past the end repeats the last one and is dropped below
            float mv[16];
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int key = j0 + 8 * (r >> 2) + 4 * hh + (r & 3);
                mv[r] = mrow[key < dst ? key : dst - 1];
            }
#pragma unroll
            for (int r = 0; r < 16; r++) s_cur[r] = add_rn(s_cur[r], mv[r]);
        }
        if (!full)
        {
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (j0 + 8 * (r >> 2) + 4 * hh + (r & 3) >= dst) s_cur[r] = -INFINITY;
        }
        ATT_PHASE_BOUNDARY();
        v16f_at s_next;
#pragma unroll
        for (int r = 0; r < 16; r++) s_next[r] = 0.f;
        float corr;
        if (j0 + 128 < key_end)
        {
#pragma unroll
            for (int kk = 0; kk < HD / 2; kk++) s_next = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[kk], qreg[kk], s_next, 0, 0, 0);
            corr = running_softmax_step(s_cur, m, l);
            // issue order within the block: one product, then three of the vector instructions, while these last
#pragma unroll
            for (int kk = 0; kk < HD / 2; kk++)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
            }
        }
        else
            corr = running_softmax_step(s_cur, m, l);
        asm volatile("" : "+v"(s_next), "+v"(s_cur));
        ATT_PHASE_BOUNDARY();
        {
            const int jn = j0 + 256 < key_end ? j0 + 256 : j0;
            const unsigned koff = (unsigned)hh * (unsigned)kv_stride + (unsigned)(jn + l32 < dst ? jn + l32 : dst - 1);
#pragma unroll
            for (int kk = 0; kk < HD / 2; kk++) kreg[kk] = (kh + (size_t)(2 * kk) * kv_stride)[koff];
        }
        ATT_PHASE_BOUNDARY();
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
        {
#pragma unroll
            for (int r = 0; r < 16; r++) o[cb][r] *= corr;
            if constexpr (CB > 2) load_value_block(vv[0], vh + (size_t)(cb * 32 + l32) * kv_stride, j0, hh, dst, full && v_vec_ok);
#pragma unroll
            for (int kk = 0; kk < 16; kk++) o[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[CB <= 2 ? cb : 0][kk], s_cur[kk], o[cb], 0, 0, 0);
        }
        s_cur = s_next;
    }

    // ---- merge the four shares: common maximum, then each wavefront adds its rescaled part in turn
    if (hh == 0)
    {
        m_s[wave][l32] = m;
        l_s[wave][l32] = l;
    }
    __syncthreads();
    const float mall = fmaxf(fmaxf(m_s[0][l32], m_s[1][l32]), fmaxf(m_s[2][l32], m_s[3][l32]));
    const float f = expf(m - mall); // a wavefront that saw no key has m = -FLT_MAX, l = 0, o = 0
    for (int w = 0; w < 4; w++)
    {
        if (wave == w)
        {
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                {
                    const int ch = cb * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
                    const float v = o[cb][r] * f;
                    o_s[ch * LD + l32] = w == 0 ? v : o_s[ch * LD + l32] + v;
                }
        }
        __syncthreads();
    }
    if (keys_per_split > 0)
    {
        // [query block][head][split] records of 32 maxima, 32 sums, 32 x HD outputs (query-major; only real queries are written)
        float* rec = partial + (((size_t)blockIdx.x * gridDim.y + h) * gridDim.z + blockIdx.z) * (size_t)(64 + HD * 32);
        const int nq = src - i0 < 32 ? src - i0 : 32;
        if (tid < 32)
        {
            const float ma = fmaxf(fmaxf(m_s[0][tid], m_s[1][tid]), fmaxf(m_s[2][tid], m_s[3][tid]));
            float lt = 0.f;
#pragma unroll
            for (int w = 0; w < 4; w++) lt += l_s[w][tid] * expf(m_s[w][tid] - ma);
            rec[tid] = ma;
            rec[32 + tid] = lt;
        }
        for (int idx = tid; idx < nq * HD; idx += 256) rec[64 + idx] = o_s[(idx % HD) * LD + idx / HD];
        return;
    }
    for (int idx = tid; idx < 32 * HD; idx += 256)
    {
        const int qq = idx / HD, ch = idx - qq * HD;
        if (i0 + qq < src)
        {
            float lt = 0.f;
#pragma unroll
            for (int w = 0; w < 4; w++) lt += l_s[w][qq] * expf(m_s[w][qq] - fmaxf(fmaxf(m_s[0][qq], m_s[1][qq]), fmaxf(m_s[2][qq], m_s[3][qq])));
            out[(size_t)(i0 + qq) * embed_dim + h * HD + ch] = div_rn(o_s[ch * LD + qq], lt);
        }
    }
}

// merges the records of the key splits: one workgroup per (query block, head).  First every (split, query) pair gets its factor
// exp(m_split - m) and the queries their sums, through LDS; then the outputs are added with eight independent loads in
// flight per thread (a thread that walks the splits for each of its outputs, one dependent load after the other, took 35 us
// for 64 queries x 16 heads x 11 splits).
__global__ __launch_bounds__(256) void attention_merge_kernel(const float* __restrict__ partial, int splits, int head_dim, int embed_dim, int src,
                                                              float* __restrict__ out)
{
    __shared__ float fac[64][32]; // splits <= 64 (attention_key_splits)
    __shared__ float l_all[32];
    const int h = blockIdx.y, i0 = blockIdx.x * 32;
    const size_t rec_size = (size_t)(64 + head_dim * 32);
    const float* rec0 = partial + ((size_t)blockIdx.x * gridDim.y + h) * splits * rec_size;
    const int nq = src - i0 < 32 ? src - i0 : 32;
    const int tid = threadIdx.x;
    for (int e = tid; e < splits * 32; e += 256) fac[e >> 5][e & 31] = rec0[(size_t)(e >> 5) * rec_size + (e & 31)];
    __syncthreads();
    if (tid < 32)
    {
        float ma = -FLT_MAX;
        for (int z = 0; z < splits; z++) ma = fmaxf(ma, fac[z][tid]);
        float lt = 0.f;
        for (int z = 0; z < splits; z++)
        {
            const float f = exp_of_nonpositive(fac[z][tid] - ma);
            fac[z][tid] = f;
            lt += rec0[(size_t)z * rec_size + 32 + tid] * f; // independent loads: the compiler keeps several in flight
        }
        l_all[tid] = lt;
    }
    __syncthreads();
    // the outputs of the block are shared out over gridDim.z workgroups (each makes the factors for itself: they are cheap)
    const int total = nq * head_dim, share = (total + (int)gridDim.z - 1) / (int)gridDim.z;
    const int begin = (int)blockIdx.z * share, end = begin + share < total ? begin + share : total;
    for (int idx = begin + tid; idx < end; idx += 256)
    {
        const int qq = idx / head_dim, ch = idx - qq * head_dim;
        const float* op = rec0 + 64 + idx;
        float ot = 0.f;
#pragma unroll 8
        for (int z = 0; z < splits; z++) ot += op[(size_t)z * rec_size] * fac[z][qq];
        out[(size_t)(i0 + qq) * embed_dim + h * head_dim + ch] = div_rn(ot, l_all[qq]);
    }
}

// ---- one to four queries on a long key sequence (a decoding step against a cache) ------------------------------------
// With so few queries the work is reading the keys and values once, and the matrix-core kernel above, built around 32
// queries per workgroup, spends its time in a chain of latencies.  Here one workgroup streams 64 keys of one head:
//   scores : thread = (key, quarter of the channels); k[channel][key] is read coalesced along the keys, the four partial
//            dot products of a key are added through LDS;
//   softmax: wavefront t takes query t (maximum, exp, sum over the 64 keys by shuffles);
//   p v    : thread = (channel, quarter of the keys); v[channel][key] is read as 16-byte pieces along the keys, four lanes
//            add their parts by shuffles.
// It leaves (maximum, sum, unnormalised output) per query for attention_fewq_merge_kernel.  fp32 throughout; the order of
// the additions differs from the reference's: fp32 tolerance.
static constexpr int FEWQ_KEYS = 64;
static constexpr int FEWQ_MAX_HEAD_DIM = 256;

// 16 consecutive values of one channel from key j on: 16-byte pieces where the rows allow, else one by one (a key past the
// end repeats the last one; its probability is 0)
__device__ __forceinline__ void load_fewq_values(float (&vv)[16], const float* __restrict__ vr, int j, int dst, bool vec)
{
    if (vec)
    {
#pragma unroll
        for (int a = 0; a < 4; a++)
        {
            const v4f_at t4 = *reinterpret_cast<const v4f_at*>(vr + j + 4 * a);
#pragma unroll
            for (int e = 0; e < 4; e++) vv[4 * a + e] = t4[e];
        }
    }
    else
    {
#pragma unroll
        for (int e = 0; e < 16; e++) vv[e] = vr[j + e < dst ? j + e : dst - 1];
    }
}

// new_k / new_v (or null): the keys and values of the last dst - past positions, rows of new_stride floats ([position][embed]).
// The workgroup whose 64 keys reach past `past` first copies its share of them into kt / vt (appending to the cache is then
// no launch of its own) and reads them back like the rest after a barrier; nobody else reads those columns.
__global__ __launch_bounds__(256) void attention_fewq_split_kernel(const float* __restrict__ q, size_t q_stride, float q_scale, float* kt, float* vt, size_t kv_stride,
                                                                   const float* __restrict__ mask, int mask_heads, int head_dim, int src, int dst, int v_vec_ok,
                                                                   float* __restrict__ partial, const float* __restrict__ new_k, const float* __restrict__ new_v,
                                                                   size_t new_stride, int past)
{
    __shared__ float qs[ATT_TQ * FEWQ_MAX_HEAD_DIM];
    __shared__ float red[4][ATT_TQ][FEWQ_KEYS];
    __shared__ float sc[ATT_TQ][FEWQ_KEYS];
    const int split = blockIdx.x, h = blockIdx.y, i0 = blockIdx.z * ATT_TQ;
    const int rows = src - i0 < ATT_TQ ? src - i0 : ATT_TQ;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j0 = split * FEWQ_KEYS;

    if (new_k && j0 + FEWQ_KEYS > past) // uniform
    {
        const int kb = j0 > past ? j0 : past, ke = j0 + FEWQ_KEYS < dst ? j0 + FEWQ_KEYS : dst;
        for (int e = tid; e < (ke - kb) * head_dim; e += 256)
        {
            const int pos = e / head_dim, c = e - pos * head_dim;
            const size_t from = (size_t)(kb + pos - past) * new_stride + (size_t)h * head_dim + c;
            const size_t to = ((size_t)h * head_dim + c) * kv_stride + kb + pos;
            kt[to] = new_k[from];
            vt[to] = new_v[from];
        }
        __threadfence_block();
        __syncthreads();
    }
    // every load that does not depend on the scores is requested before the first wait: the first 16 channels of this
    // wavefront's keys, this thread's values of the first 64 channels, the queries
    const int per = (head_dim + 3) >> 2, c0 = wave * per, c1 = c0 + per < head_dim ? c0 + per : head_dim;
    const int key = j0 + lane < dst ? j0 + lane : dst - 1; // past the end: repeated, dropped below
    const float* kp = kt + ((size_t)h * head_dim + c0) * kv_stride + key;
    float kfirst[16];
#pragma unroll
    for (int i = 0; i < 16; i++) kfirst[i] = c0 + i < c1 ? kp[(size_t)i * kv_stride] : 0.f;
    const int kq = tid & 3;
    const bool vec = v_vec_ok && j0 + FEWQ_KEYS <= dst;
    float vfirst[16];
    load_fewq_values(vfirst, vt + ((size_t)h * head_dim + ((tid >> 2) < head_dim ? (tid >> 2) : 0)) * kv_stride, j0 + 16 * kq, dst, vec);
    for (int e = tid; e < ATT_TQ * head_dim; e += 256)
    {
        const int t = e / head_dim, l = e - t * head_dim;
        qs[e] = t < rows ? mul_rn(q[(size_t)(i0 + t) * q_stride + h * head_dim + l], q_scale) : 0.f;
    }
    __syncthreads();

    // ---- scores: wavefront g takes the g-th quarter of the channels, lane = key
    {
        float acc[ATT_TQ];
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++) acc[t] = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++)
            if (c0 + i < c1)
            {
#pragma unroll
                for (int t = 0; t < ATT_TQ; t++) acc[t] = add_rn(acc[t], mul_rn(qs[t * head_dim + c0 + i], kfirst[i]));
            }
        kp += (size_t)16 * kv_stride;
#pragma unroll 8
        for (int c = c0 + 16; c < c1; c++)
        {
            const float kv = *kp;
            kp += kv_stride;
#pragma unroll
            for (int t = 0; t < ATT_TQ; t++) acc[t] = add_rn(acc[t], mul_rn(qs[t * head_dim + c], kv));
        }
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++) red[wave][t][lane] = acc[t];
    }
    __syncthreads();

    // ---- softmax over this workgroup's keys: wavefront t = query t
    float m_t = -FLT_MAX, l_t = 0.f;
    {
        const int t = wave;
        float s = add_rn(add_rn(red[0][t][lane], red[1][t][lane]), add_rn(red[2][t][lane], red[3][t][lane]));
        const bool live = j0 + lane < dst && t < rows;
        if (live && mask) s = add_rn(s, mask[((size_t)(mask_heads > 1 ? h : 0) * src + i0 + t) * dst + j0 + lane]);
        if (!live) s = -INFINITY;
        m_t = fmaxf(wave_max(s), -FLT_MAX); // a query that is not there (or all keys at -inf): every probability 0
        const float pr = exp_of_nonpositive(s - m_t);
        l_t = wave_sum(pr);
        sc[t][lane] = pr;
    }
    __syncthreads();

    // ---- p v: thread = (channel tid/4, keys 16*(tid%4)..+15), four lanes share a channel
    float* rec = partial + (((size_t)blockIdx.z * gridDim.y + h) * gridDim.x + split) * (size_t)(2 * ATT_TQ + ATT_TQ * head_dim);
    for (int ch = tid >> 2; ch < ((head_dim + 63) & ~63); ch += 64)
    {
        float acc[ATT_TQ];
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++) acc[t] = 0.f;
        if (ch < head_dim)
        {
            float vv[16];
            if (ch < 64)
            {
#pragma unroll
                for (int e = 0; e < 16; e++) vv[e] = vfirst[e];
            }
            else
                load_fewq_values(vv, vt + ((size_t)h * head_dim + ch) * kv_stride, j0 + 16 * kq, dst, vec);
#pragma unroll
            for (int e = 0; e < 16; e++)
#pragma unroll
                for (int t = 0; t < ATT_TQ; t++) acc[t] = add_rn(acc[t], mul_rn(sc[t][16 * kq + e], vv[e]));
        }
#pragma unroll
        for (int t = 0; t < ATT_TQ; t++)
        {
            acc[t] = add_rn(acc[t], __shfl_xor(acc[t], 1));
            acc[t] = add_rn(acc[t], __shfl_xor(acc[t], 2));
        }
        if (kq == 0 && ch < head_dim)
#pragma unroll
            for (int t = 0; t < ATT_TQ; t++) rec[2 * ATT_TQ + t * head_dim + ch] = acc[t];
    }
    if (lane == 0)
    {
        rec[wave] = m_t;
        rec[ATT_TQ + wave] = l_t;
    }
}

// merges the records of attention_fewq_split_kernel: one workgroup per (head, group of four queries).  The maxima and
// sums of all splits are fetched side by side into LDS (wavefront t = query t) and turned into one factor per split;
// then four groups of 64 threads each add every fourth split's outputs, eight loads in flight, and the groups' parts
// are added through LDS - a thread that walks the splits one load after the other takes 14 us for 24 of them.
static constexpr int FEWQ_MAX_SPLITS = 512; // 8 per lane of a wavefront in the merge

__global__ __launch_bounds__(256) void attention_fewq_merge_kernel(const float* __restrict__ partial, int splits, int head_dim, int embed_dim, int src,
                                                                   float* __restrict__ out)
{
    __shared__ float fac[ATT_TQ][FEWQ_MAX_SPLITS];
    __shared__ float l_all[ATT_TQ];
    __shared__ float part[4][64];
    const int h = blockIdx.x, i0 = blockIdx.y * ATT_TQ;
    const int rows = src - i0 < ATT_TQ ? src - i0 : ATT_TQ;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t rec_size = (size_t)(2 * ATT_TQ + ATT_TQ * head_dim);
    const float* rec0 = partial + ((size_t)blockIdx.y * gridDim.x + h) * splits * rec_size;
    // Everything the first 64 outputs need is requested before the first wait (one trip to memory instead of three): this
    // lane's maxima and sums of chunks lane, lane + 64, ... and, for output `lane`, the parts of this group's first 8 chunks.
    float ofirst[8], mz[8], lz[8];
    {
        const float* op = rec0 + 2 * ATT_TQ + lane;
#pragma unroll
        for (int k = 0; k < 8; k++) ofirst[k] = lane < rows * head_dim && wave + 4 * k < splits ? op[(size_t)(wave + 4 * k) * rec_size] : 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++)
        {
            const int z = lane + 64 * k; // FEWQ_MAX_SPLITS = 8 * 64
            mz[k] = z < splits ? rec0[z * rec_size + wave] : -FLT_MAX;
            lz[k] = z < splits ? rec0[z * rec_size + ATT_TQ + wave] : 0.f;
        }
    }
    {
        const int t = wave;
        float ma = -FLT_MAX;
#pragma unroll
        for (int k = 0; k < 8; k++) ma = fmaxf(ma, mz[k]);
        ma = wave_max(ma);
        float lt = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++)
        {
            const int z = lane + 64 * k;
            const float f = exp_of_nonpositive(mz[k] - ma);
            if (z < splits) fac[t][z] = f;
            lt += lz[k] * f;
        }
        lt = wave_sum(lt);
        if (lane == 0) l_all[t] = lt;
    }
    __syncthreads();
    for (int base = 0; base < rows * head_dim; base += 64)
    {
        const int idx = base + lane;
        float ot = 0.f;
        if (idx < rows * head_dim)
        {
            const int t = idx / head_dim;
            const float* op = rec0 + 2 * ATT_TQ + idx;
            int z = wave;
            if (base == 0)
            {
#pragma unroll
                for (int k = 0; k < 8; k++)
                    if (wave + 4 * k < splits) ot += ofirst[k] * fac[t][wave + 4 * k];
                z = wave + 32;
            }
#pragma unroll 8
            for (; z < splits; z += 4) ot += op[z * rec_size] * fac[t][z];
        }
        part[wave][lane] = ot;
        __syncthreads();
        if (wave == 0 && idx < rows * head_dim)
        {
            const int t = idx / head_dim;
            const float sum = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
            out[(size_t)(i0 + t) * embed_dim + h * head_dim + (idx - t * head_dim)] = div_rn(sum, l_all[t]);
        }
        __syncthreads();
    }
}

// the few-query kernels take over where they apply: up to four queries, a key sequence long enough to be worth splitting
static bool attention_fewq_applies(int head_dim, int src, int dst)
{
    return src <= ATT_TQ && dst >= 256 && dst <= FEWQ_KEYS * FEWQ_MAX_SPLITS && head_dim <= FEWQ_MAX_HEAD_DIM;
}
static size_t attention_fewq_workspace_bytes(int num_heads, int head_dim, int src, int dst)
{
    return (size_t)((src + ATT_TQ - 1) / ATT_TQ) * num_heads * ((dst + FEWQ_KEYS - 1) / FEWQ_KEYS) * (size_t)(2 * ATT_TQ + ATT_TQ * head_dim) * sizeof(float);
}

// how many ways to split the keys: enough workgroups for the chip, at least 128 keys (one tile per wavefront) each.
// (With 256 workgroups or more a split does not pay even where the last round over the chip is mostly empty - 47 query
// blocks x 16 heads at head dimension 64 run in 1.47 rounds of 512: split in two, the kernel took 145 us against 136 and
// the merge another 13.)
static int attention_key_splits(int num_heads, int src, int dst)
{
    const long long groups = (long long)((src + 31) / 32) * num_heads;
    if (groups >= 256 || dst < 256) return 1;
    long long want = (512 + groups - 1) / groups;
    const long long most = dst / 128;
    if (want > most) want = most;
    if (want > 64) want = 64;
    return want < 2 ? 1 : (int)want;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_attention_workspace_bytes(int num_heads, int head_dim, int src_seqlen, int dst_seqlen, size_t* workspace_bytes)
{
    NCNNHIP_REQUIRE(num_heads >= 1 && head_dim >= 1 && src_seqlen >= 1 && dst_seqlen >= 1 && workspace_bytes, "ncnnhip_attention_workspace_bytes: bad argument");
    *workspace_bytes = 0;
    if (head_dim % 32 == 0 && head_dim <= 128)
    {
        const int splits = attention_key_splits(num_heads, src_seqlen, dst_seqlen);
        if (splits > 1) *workspace_bytes = (size_t)((src_seqlen + 31) / 32) * num_heads * splits * (size_t)(64 + head_dim * 32) * sizeof(float);
    }
    if (attention_fewq_applies(head_dim, src_seqlen, dst_seqlen))
    {
        const size_t need = attention_fewq_workspace_bytes(num_heads, head_dim, src_seqlen, dst_seqlen);
        if (need > *workspace_bytes) *workspace_bytes = need;
    }
    return NCNNHIP_OK;
}

// append_k / append_v (or null): new rows to be written into columns past.. of kt / vt before they are read
static int attention_dispatch(const float* q_dev, size_t q_stride, float q_scale, float* kt_dev, float* vt_dev, size_t kv_stride, const float* mask_dev, int mask_heads,
                              int num_heads, int head_dim, int src_seqlen, int dst_seqlen, float* out_dev, void* workspace_dev, size_t workspace_bytes, void* stream,
                              const float* append_k, const float* append_v, size_t append_stride, int past);

int ncnnhip_attention_f32(const float* q_dev, const float* kt_dev, const float* vt_dev, size_t kv_stride, const float* mask_dev, int mask_heads,
                          int num_heads, int head_dim, int src_seqlen, int dst_seqlen, float* out_dev, void* workspace_dev, size_t workspace_bytes,
                          void* stream)
{
    return ncnnhip_attention_f32_strided(q_dev, (size_t)num_heads * (size_t)(head_dim > 0 ? head_dim : 0), 1.f, kt_dev, vt_dev, kv_stride, mask_dev, mask_heads, num_heads,
                                         head_dim, src_seqlen, dst_seqlen, out_dev, workspace_dev, workspace_bytes, stream);
}

int ncnnhip_attention_f32_strided(const float* q_dev, size_t q_stride, float q_scale, const float* kt_dev, const float* vt_dev, size_t kv_stride, const float* mask_dev,
                                  int mask_heads, int num_heads, int head_dim, int src_seqlen, int dst_seqlen, float* out_dev, void* workspace_dev,
                                  size_t workspace_bytes, void* stream)
{
    return attention_dispatch(q_dev, q_stride, q_scale, const_cast<float*>(kt_dev), const_cast<float*>(vt_dev), kv_stride, mask_dev, mask_heads, num_heads, head_dim,
                              src_seqlen, dst_seqlen, out_dev, workspace_dev, workspace_bytes, stream, nullptr, nullptr, 0, 0);
}

int ncnnhip_attention_f32_append(const float* qkv_dev, size_t qkv_stride, float q_scale, float* kt_dev, float* vt_dev, size_t kv_stride, int past_seqlen,
                                 const float* mask_dev, int mask_heads, int num_heads, int head_dim, int src_seqlen, float* out_dev, void* workspace_dev,
                                 size_t workspace_bytes, void* stream)
{
    NCNNHIP_REQUIRE(qkv_dev && num_heads >= 1 && head_dim >= 1 && src_seqlen >= 1 && past_seqlen >= 0, "ncnnhip_attention_f32_append: bad argument");
    const size_t e = (size_t)num_heads * (size_t)head_dim;
    NCNNHIP_REQUIRE(qkv_stride >= 3 * e, "ncnnhip_attention_f32_append: rows of q, k and v need a stride of at least 3 * embed_dim");
    NCNNHIP_REQUIRE(past_seqlen <= INT_MAX - src_seqlen, "ncnnhip_attention_f32_append: sequence too long");
    return attention_dispatch(qkv_dev, qkv_stride, q_scale, kt_dev, vt_dev, kv_stride, mask_dev, mask_heads, num_heads, head_dim, src_seqlen, past_seqlen + src_seqlen,
                              out_dev, workspace_dev, workspace_bytes, stream, qkv_dev + e, qkv_dev + 2 * e, qkv_stride, past_seqlen);
}

} // extern "C"

static int attention_dispatch(const float* q_dev, size_t q_stride, float q_scale, float* kt_dev, float* vt_dev, size_t kv_stride, const float* mask_dev, int mask_heads,
                              int num_heads, int head_dim, int src_seqlen, int dst_seqlen, float* out_dev, void* workspace_dev, size_t workspace_bytes, void* stream,
                              const float* append_k, const float* append_v, size_t append_stride, int past)
{
    NCNNHIP_REQUIRE(q_dev && kt_dev && vt_dev && out_dev, "ncnnhip_attention_f32: null pointer");
    NCNNHIP_REQUIRE(num_heads >= 1 && head_dim >= 1 && src_seqlen >= 1 && dst_seqlen >= 1, "ncnnhip_attention_f32: bad shape");
    NCNNHIP_REQUIRE(num_heads <= 65535, "ncnnhip_attention_f32: more than 65535 heads");
    NCNNHIP_REQUIRE(q_stride >= (size_t)num_heads * (size_t)head_dim, "ncnnhip_attention_f32: query row stride below embed_dim");
    NCNNHIP_REQUIRE(kv_stride >= (size_t)dst_seqlen, "ncnnhip_attention_f32: key/value row stride below dst_seqlen");
    NCNNHIP_REQUIRE(kv_stride + (size_t)dst_seqlen < ((size_t)1 << 30), "ncnnhip_attention_f32: key/value row stride beyond the 32-bit byte offsets of the kernel");
    NCNNHIP_REQUIRE(!mask_dev || mask_heads == 1 || mask_heads == num_heads, "ncnnhip_attention_f32: the mask is shared (1) or one per head");
    if (attention_fewq_applies(head_dim, src_seqlen, dst_seqlen) && workspace_dev
        && workspace_bytes >= attention_fewq_workspace_bytes(num_heads, head_dim, src_seqlen, dst_seqlen))
    {
        const int v_vec_ok = (kv_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(vt_dev) & 15) == 0) ? 1 : 0;
        const int splits = (dst_seqlen + FEWQ_KEYS - 1) / FEWQ_KEYS, qgroups = (src_seqlen + ATT_TQ - 1) / ATT_TQ;
        hipStream_t st = as_stream(stream);
        hipLaunchKernelGGL(attention_fewq_split_kernel, dim3((unsigned)splits, (unsigned)num_heads, (unsigned)qgroups), dim3(256), 0, st, q_dev, q_stride, q_scale, kt_dev,
                           vt_dev, kv_stride, mask_dev, mask_dev ? mask_heads : 0, head_dim, src_seqlen, dst_seqlen, v_vec_ok, (float*)workspace_dev, append_k, append_v,
                           append_stride, past);
        hipLaunchKernelGGL(attention_fewq_merge_kernel, dim3((unsigned)num_heads, (unsigned)qgroups), dim3(256), 0, st, (const float*)workspace_dev, splits, head_dim,
                           num_heads * head_dim, src_seqlen, out_dev);
        return launch_status("attention_fewq_split_kernel");
    }
    if (append_k)
    {
        // the other kernels read a finished cache: the new columns are written by a launch of their own
        const int rc = ncnnhip_transpose_pair_f32(append_k, append_v, append_stride, dst_seqlen - past, num_heads * head_dim, kt_dev + past, vt_dev + past, kv_stride, stream);
        if (rc != NCNNHIP_OK) return rc;
    }
    if (head_dim % 32 == 0 && head_dim <= 128)
    {
        // 16-byte loads of the values need the rows and the start aligned
        const int v_vec_ok = (kv_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(vt_dev) & 15) == 0) ? 1 : 0;
        // few queries (decoding): split the keys over workgroups when the caller brought the scratch for it
        int splits = attention_key_splits(num_heads, src_seqlen, dst_seqlen);
        size_t need = 0;
        if (splits > 1) need = (size_t)((src_seqlen + 31) / 32) * num_heads * splits * (size_t)(64 + head_dim * 32) * sizeof(float);
        if (splits > 1 && (!workspace_dev || workspace_bytes < need)) splits = 1;
        int keys_per_split = 0;
        if (splits > 1)
        {
            keys_per_split = ((dst_seqlen + splits - 1) / splits + 31) / 32 * 32;
            splits = (dst_seqlen + keys_per_split - 1) / keys_per_split;
        }
        dim3 grid((unsigned)((src_seqlen + 31) / 32), (unsigned)num_heads, (unsigned)(splits > 1 ? splits : 1));
        if (splits <= 1) keys_per_split = 0;
        float* partial = (float*)workspace_dev;
        const int e = num_heads * head_dim, mh = mask_dev ? mask_heads : 0;
        hipStream_t st = as_stream(stream);
#define LAUNCH_ATT(HD_) \
    hipLaunchKernelGGL(attention_f32_mfma_kernel<HD_>, grid, dim3(256), 0, st, q_dev, kt_dev, vt_dev, mask_dev, mh, e, src_seqlen, dst_seqlen, kv_stride, out_dev, \
                       v_vec_ok, keys_per_split, partial, q_stride, q_scale)
        if (head_dim == 32)
            LAUNCH_ATT(32);
        else if (head_dim == 64)
            LAUNCH_ATT(64);
        else if (head_dim == 96)
            LAUNCH_ATT(96);
        else
            LAUNCH_ATT(128);
#undef LAUNCH_ATT
        if (keys_per_split > 0)
        {
            // enough workgroups for the chip: the outputs of a (query block, head) shared out over up to 8 of them
            unsigned shares = 1;
            while (shares < 8 && grid.x * grid.y * shares < 256 && (unsigned)(32 * head_dim) / (shares * 2) >= 256) shares *= 2;
            hipLaunchKernelGGL(attention_merge_kernel, dim3(grid.x, grid.y, shares), dim3(256), 0, st, partial, splits, head_dim, e, src_seqlen, out_dev);
        }
        return launch_status("attention_f32_mfma_kernel");
    }
    const size_t lds = (size_t)ATT_TQ * ((size_t)head_dim + (size_t)dst_seqlen) * sizeof(float);
    NCNNHIP_REQUIRE(lds <= 65536, "ncnnhip_attention_f32: head_dim %d is not 32/64/96/128 and head_dim + dst_seqlen = %d exceeds the 4096 the general kernel keeps in LDS",
                    head_dim, head_dim + dst_seqlen);
    dim3 grid((unsigned)((src_seqlen + ATT_TQ - 1) / ATT_TQ), (unsigned)num_heads);
    hipLaunchKernelGGL(attention_f32_kernel, grid, dim3(256), lds, as_stream(stream), q_dev, kt_dev, vt_dev, mask_dev, mask_dev ? mask_heads : 0, head_dim,
                       num_heads * head_dim, src_seqlen, dst_seqlen, kv_stride, out_dev, q_stride, q_scale);
    return launch_status("attention_f32_kernel");
}
