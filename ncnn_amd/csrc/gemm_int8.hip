// int8 Gemm and InnerProduct launchers on top of the MFMA tile contraction.
#include "conv_nhwc.h"
#include "epilogues.h"
#include "mfma_tile.h"

namespace ncnnhip {

template<int BM, int BN, typename Epilogue>
__global__ __launch_bounds__(256) void gemm_tile_kernel(DenseOperand a, DenseOperand b, Epilogue epi, int M, int N, int K)
{
    mfma_tile_body<BM, BN, DenseOperand, Epilogue>(a, b, epi, M, N, K, blockIdx.y * BM, blockIdx.x * BN);
}

// skinny case (up to a few dozen activation rows): one wavefront per output channel streams the weight row with
// 16-byte loads, multiplies it against up to 8 activation rows at a time held in registers (v_dot4_i32_i8) and
// reduces with cross-lane adds; no matrix cores involved.  The layer is bound by reading the weights once.
// ROW_FIRST: the epilogue takes (activation row, output column, acc), as Gemm's does; else (output channel, row, acc)
template<typename Epilogue, bool ROW_FIRST>
__global__ __launch_bounds__(256) void fc_gemv_kernel(const int8_t* __restrict__ x, size_t xs, int rows, int K,
                                                       const int8_t* __restrict__ wgt, size_t ws, int num_output, Epilogue epi, int vec)
{
    const int lane = threadIdx.x & 63;
    const int p = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= num_output) return;
    const int8_t* wr = wgt + (size_t)p * ws;
    for (int r0 = 0; r0 < rows; r0 += 8)
    {
        const int nr = rows - r0 < 8 ? rows - r0 : 8;
        int acc[8];
#pragma unroll
        for (int r = 0; r < 8; r++) acc[r] = 0;
        if (vec)
        {
            for (int k = lane * 16; k + 16 <= K; k += 64 * 16)
            {
                const v4i wv = *reinterpret_cast<const v4i*>(wr + k);
#pragma unroll
                for (int r = 0; r < 8; r++)
                    if (r < nr)
                    {
                        const v4i xv = *reinterpret_cast<const v4i*>(x + (size_t)(r0 + r) * xs + k);
#pragma unroll
                        for (int d = 0; d < 4; d++) acc[r] = __builtin_amdgcn_sdot4(wv[d], xv[d], acc[r], false);
                    }
            }
            for (int k = (K & ~15) + lane; k < K; k += 64)
#pragma unroll
                for (int r = 0; r < 8; r++)
                    if (r < nr) acc[r] += (int)wr[k] * (int)x[(size_t)(r0 + r) * xs + k];
        }
        else
        {
            for (int k = lane; k < K; k += 64)
#pragma unroll
                for (int r = 0; r < 8; r++)
                    if (r < nr) acc[r] += (int)wr[k] * (int)x[(size_t)(r0 + r) * xs + k];
        }
#pragma unroll
        for (int r = 0; r < 8; r++)
        {
            int v = acc[r];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0 && r < nr)
            {
                if (ROW_FIRST)
                    epi(r0 + r, p, v);
                else
                    epi(p, r0 + r, v);
            }
        }
    }
}

// Up to 16 rows of A on the matrix cores: a workgroup owns 16 rows of B, its four wavefronts every fourth 64-wide K step each
// (v_mfma_i32_16x16x64_i8: the rows of B as one operand, the rows of A as the other, so a lane ends up with four consecutive
// columns of one output row); eight steps of B and A are requested before the first product; the four partial tiles are
// added through LDS.  B is read once; A (at most 16 x K bytes) comes from the cache.
typedef int v4i_sk __attribute__((ext_vector_type(4)));
template<typename Epilogue, bool ROW_FIRST>
__global__ __launch_bounds__(256) void gemm_skinny_int8_kernel(const int8_t* __restrict__ a, size_t as, int M_total, const int8_t* __restrict__ b, size_t bs, int N, int K,
                                                                Epilogue epi)
{
    __shared__ int red[4][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c16 = lane & 15, q = lane >> 4;
    const int tile = blockIdx.x;
    const int row0 = blockIdx.y * 16; // blockIdx.y: which 16 rows of A (every group of 16 reads B again, from the cache after the first)
    const int M = M_total - row0 < 16 ? M_total - row0 : 16;
    a += (size_t)row0 * as;
    const int brow = tile * 16 + c16 < N ? tile * 16 + c16 : N - 1; // rows past the end repeat the last one; nothing of theirs is stored
    const int arow = c16 < M ? c16 : M - 1;
    const int8_t* bp = b + (size_t)brow * bs + q * 16;
    const int8_t* ap = a + (size_t)arow * as + q * 16;
    const int ksteps = K >> 6;
    v4i_sk acc = {0, 0, 0, 0};
    for (int k0 = wave; k0 < ksteps; k0 += 32) // this wavefront's steps k0, k0 + 4, ..., eight at a time
    {
        v4i_sk wv[8], xv[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
        {
            const int ks = k0 + 4 * u;
            const int kk = ks < ksteps ? ks : k0; // past the end: a step that is there, its product dropped below
            wv[u] = *reinterpret_cast<const v4i_sk*>(bp + (size_t)kk * 64);
            xv[u] = *reinterpret_cast<const v4i_sk*>(ap + (size_t)kk * 64);
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (k0 + 4 * u < ksteps) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[u], xv[u], acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) red[wave][lane][r] = acc[r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int r = 0; r < 4; r++)
    {
        const int v = (red[0][lane][r] + red[1][lane][r]) + (red[2][lane][r] + red[3][lane][r]);
        const int j = tile * 16 + 4 * q + r;
        if (c16 < M && j < N)
        {
            if (ROW_FIRST)
                epi(row0 + c16, j, v); // Gemm's epilogue: (row of A, column)
            else
                epi(j, row0 + c16, v); // InnerProduct's: (output channel, row)
        }
    }
}

// InnerProduct on 2 to 48 rows (a batch through the classifier of a net): the same kernel with InnerProduct's epilogue, under the
// same estimate as Gemm's.  false: the shape is not one it takes.
static bool launch_fc_skinny(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output, const int8_t* weight_dev, const FcEpilogue& epi,
                             hipStream_t stream);

#ifndef GEMM_GEMV_MAX_ROWS
#define GEMM_GEMV_MAX_ROWS 4
#endif
#ifndef GEMM_SKINNY_MIN_ROWS
#define GEMM_SKINNY_MIN_ROWS 0
#endif
#ifndef GEMM_SKINNY_MAX_ROWS
#define GEMM_SKINNY_MAX_ROWS 48
#endif
static inline bool aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

static DenseOperand make_dense(const int8_t* base, size_t stride, int rows, int K)
{
    DenseOperand d;
    d.base = base;
    d.stride = stride;
    d.rows = rows;
    d.K = K;
    d.vec = aligned16(base) && stride % 16 == 0;
    return d;
}

int launch_gemm_int8_pipelined(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K,
                               const GemmEpilogue& epi, hipStream_t stream, bool* handled);

int launch_gemm_int8_tiled(const int8_t* aq_tiled, const int8_t* bq_tiled, int M, int N, int K, const GemmEpilogue& epi, hipStream_t stream);
int launch_gemm_int8_ring128(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K, const GemmEpilogue& epi,
                             hipStream_t stream, bool* handled);
int launch_gemm_tile_operand(const int8_t* src, size_t stride, int rows, int K, int operand_b, int8_t* dst, hipStream_t stream);

// the shapes the few-row kernel takes for InnerProduct (operands aligned): no workspace, no hand-off between workgroups
bool fc_skinny_takes(int rows, int num_input, int num_output)
{
    if (rows < 2 || rows > GEMM_SKINNY_MAX_ROWS || num_output < 64 || num_input % 64 != 0) return false;
    const int groups16 = (rows + 15) / 16;
    return !(rows > 16 && 3.0 + groups16 * ((double)num_output * (double)num_input / 4.0e6) > 4.0 + num_input / 300.0);
}

static bool launch_fc_skinny(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output, const int8_t* weight_dev, const FcEpilogue& epi,
                             hipStream_t stream)
{
    if (!fc_skinny_takes(rows, num_input, num_output)) return false;
    if (!aligned16(x_dev) || !aligned16(weight_dev) || x_stride % 16 != 0) return false;
    const int groups16 = (rows + 15) / 16;
    hipLaunchKernelGGL((gemm_skinny_int8_kernel<FcEpilogue, false>), dim3(ceil_div(num_output, 16), groups16), dim3(256), 0, stream, x_dev, x_stride, rows, weight_dev,
                       (size_t)num_input, num_output, num_input, epi);
    return true;
}

} // namespace ncnnhip

using namespace ncnnhip;

extern "C" {

int ncnnhip_gemm_int8(const int8_t* aq_dev, size_t aq_stride, const int8_t* bq_dev, size_t bq_stride, int M, int N, int K,
                      const float* a_scales_dev, const float* b_scales_dev, int n_b_scales, const float* c_dev,
                      int broadcast_type_c, float alpha, float beta, int output_transpose, float* out_dev,
                      size_t out_stride, int32_t* acc_out_dev, void* stream)
{
    NCNNHIP_REQUIRE(aq_dev && bq_dev && a_scales_dev && b_scales_dev && out_dev, "ncnnhip_gemm_int8: null pointer");
    NCNNHIP_REQUIRE(M >= 1 && N >= 1 && K >= 1, "ncnnhip_gemm_int8: bad shape %d %d %d", M, N, K);
    NCNNHIP_REQUIRE(aq_stride >= (size_t)K && bq_stride >= (size_t)K, "ncnnhip_gemm_int8: operand stride below K");
    NCNNHIP_REQUIRE(n_b_scales == 1 || n_b_scales == N, "ncnnhip_gemm_int8: %d B scales for N=%d", n_b_scales, N);
    NCNNHIP_REQUIRE(broadcast_type_c >= -1 && broadcast_type_c <= 4, "ncnnhip_gemm_int8: broadcast_type_c %d", broadcast_type_c);
    NCNNHIP_REQUIRE(broadcast_type_c < 0 || c_dev, "ncnnhip_gemm_int8: C pointer missing");
    NCNNHIP_REQUIRE(out_stride >= (size_t)(output_transpose ? M : N), "ncnnhip_gemm_int8: output stride too small");

    GemmEpilogue epi;
    epi.a_scales = a_scales_dev;
    epi.b_scales = b_scales_dev;
    epi.per_col = n_b_scales != 1;
    epi.c = c_dev;
    epi.bt = c_dev ? broadcast_type_c : -1;
    epi.alpha = alpha;
    epi.beta = beta;
    epi.transpose = output_transpose;
    epi.out = out_dev;
    epi.out_stride = out_stride;
    epi.N = N;
    epi.acc_out = acc_out_dev;

    // up to four rows of A whose shape the matrix-core form above does not take (K % 64, unaligned rows): one wavefront per row
    // of B with v_dot4.  Quantise + Gemm, one / four rows: 4096 x 4096 19.6 / 20.3 -> 9.2 / 12.3 us, 11008 x 4096
    // 21.9 / 22.0 -> 16.9 / 23.3, 1024 x 1024 9.5 / 9.5 -> 7.0 / 8.1.  (Eight pieces of the weight row requested at once per
    // lane instead of one were measured: no better at 4096 x 4096, worse on the other two.)
    // up to 16 rows of A, or up to 48 while reading B once per 16 rows (about 3 us + groups x bytes of B at 4 TB/s, from the cache
    // after the first) stays below what the tiled kernels take for so few rows (about 4 us + K / 300): quantise + Gemm for
    // 16 / 32 / 48 rows 4096 x 4096 20.6 / 21.2 / 21.4 -> 10.1 / 13.6 / 17.3 us, 11008 x 4096 22.1 -> 17.6 at 16 rows (beyond:
    // tiled), 1024 x 1024 9.9 / 10.2 / 10.3 -> 7.2 / 7.5 / 7.3; one row 19.6 -> 8.7 / 21.9 -> 13.7 / 9.5 -> 7.5
    const int groups16 = (M + 15) / 16;
    const bool skinny_pays = M <= 16 || 3.0 + groups16 * ((double)N * (double)K / 4.0e6) <= 4.0 + K / 300.0;
    if (skinny_pays && M > GEMM_SKINNY_MIN_ROWS && M <= GEMM_SKINNY_MAX_ROWS && N >= 64 && K % 64 == 0 && aligned16(aq_dev) && aligned16(bq_dev) && aq_stride % 16 == 0 && bq_stride % 16 == 0)
    {
        hipLaunchKernelGGL((gemm_skinny_int8_kernel<GemmEpilogue, true>), dim3(ceil_div(N, 16), ceil_div(M, 16)), dim3(256), 0, as_stream(stream), aq_dev, aq_stride, M, bq_dev, bq_stride, N, K,
                           epi);
        return launch_status("gemm_skinny_int8_kernel");
    }
    if (M <= GEMM_GEMV_MAX_ROWS && N >= 64)
    {
        const int vec = (aligned16(aq_dev) && aligned16(bq_dev) && aq_stride % 16 == 0 && bq_stride % 16 == 0) ? 1 : 0;
        hipLaunchKernelGGL((fc_gemv_kernel<GemmEpilogue, true>), dim3(ceil_div(N, 4)), dim3(256), 0, as_stream(stream), aq_dev, aq_stride, M, K, bq_dev, bq_stride, N, epi,
                           vec);
        return launch_status("fc_gemv_kernel");
    }
    // big aligned problems: the 256x256 kernel (it needs a few hundred tiles to fill the chip)
    bool handled = false;
    int ret = NCNNHIP_OK;
    if ((long long)M * N >= 256ll * 256 * 128)
    {
        ret = launch_gemm_int8_pipelined(aq_dev, aq_stride, bq_dev, bq_stride, M, N, K, epi, as_stream(stream), &handled);
        if (handled) return ret;
    }
    // too few 256x256 tiles for that: the same ring on 128x128 tiles, from 48 of them up (below, the 64-row tiles of the convolution
    // kernel spread the work over more CUs)
    if ((long long)(M / 128) * (N / 128) >= 48)
    {
        ret = launch_gemm_int8_ring128(aq_dev, aq_stride, bq_dev, bq_stride, M, N, K, epi, as_stream(stream), &handled);
        if (handled) return ret;
    }
    // anything else with K % 64 == 0: the convolution's pipelined kernel run as a 1x1 convolution over the rows of A
    if (!output_transpose && !acc_out_dev)
    {
        GemmTail tail;
        tail.a_scales = a_scales_dev;
        tail.b_scales = b_scales_dev;
        tail.per_col = epi.per_col;
        tail.c = c_dev;
        tail.bt = epi.bt;
        tail.alpha = alpha;
        tail.beta = beta;
        ret = launch_gemm_via_conv_pipelined(aq_dev, aq_stride, bq_dev, bq_stride, M, N, K, tail, out_dev, out_stride, as_stream(stream), &handled);
        if (handled) return ret;
    }

    DenseOperand a = make_dense(aq_dev, aq_stride, M, K);
    DenseOperand b = make_dense(bq_dev, bq_stride, N, K);
    dim3 grid(ceil_div(N, 128), ceil_div(M, 128));
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_gemm_int8: M too large");
    hipLaunchKernelGGL((gemm_tile_kernel<128, 128, GemmEpilogue>), grid, dim3(256), 0, as_stream(stream), a, b, epi, M, N, K);
    return launch_status("gemm_tile_kernel");
}

int ncnnhip_innerproduct_int8(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output,
                              const int8_t* weight_dev, const float* scale_in_dev, const float* bias_dev,
                              ncnnhip_activation act, float* out_dev, size_t out_stride, int32_t* acc_out_dev, void* stream)
{
    NCNNHIP_REQUIRE(x_dev && weight_dev && scale_in_dev && out_dev, "ncnnhip_innerproduct_int8: null pointer");
    NCNNHIP_REQUIRE(rows >= 1 && num_input >= 1 && num_output >= 1, "ncnnhip_innerproduct_int8: bad shape");
    NCNNHIP_REQUIRE(x_stride >= (size_t)num_input && out_stride >= (size_t)num_output, "ncnnhip_innerproduct_int8: stride too small");

    FcEpilogue epi;
    epi.scale_in = scale_in_dev;
    epi.bias = bias_dev;
    epi.act = act;
    epi.out = out_dev;
    epi.out_stride = out_stride;
    epi.num_output = num_output;
    epi.acc_out = acc_out_dev;

    if (launch_fc_skinny(x_dev, x_stride, rows, num_input, num_output, weight_dev, epi, as_stream(stream))) return launch_status("gemm_skinny_int8_kernel<fc>");
    if (rows <= 64)
    {
        const int vec = aligned16(x_dev) && aligned16(weight_dev) && x_stride % 16 == 0 && num_input % 16 == 0;
        hipLaunchKernelGGL((fc_gemv_kernel<FcEpilogue, false>), dim3(ceil_div(num_output, 4)), dim3(256), 0, as_stream(stream), x_dev, x_stride, rows,
                           num_input, weight_dev, (size_t)num_input, num_output, epi, vec);
        return launch_status("fc_gemv_kernel");
    }

    DenseOperand a = make_dense(weight_dev, (size_t)num_input, num_output, num_input);
    DenseOperand b = make_dense(x_dev, x_stride, rows, num_input);
    dim3 grid(ceil_div(rows, 64), ceil_div(num_output, 128));
    NCNNHIP_REQUIRE(grid.y <= 65535, "ncnnhip_innerproduct_int8: num_output too large");
    hipLaunchKernelGGL((gemm_tile_kernel<128, 64, FcEpilogue>), grid, dim3(256), 0, as_stream(stream), a, b, epi, num_output, rows, num_input);
    return launch_status("gemm_tile_kernel<fc>");
}

int ncnnhip_innerproduct_workspace_bytes(int rows, int num_input, int num_output, size_t* workspace_bytes)
{
    NCNNHIP_REQUIRE(rows >= 1 && num_input >= 1 && num_output >= 1 && workspace_bytes, "ncnnhip_innerproduct_workspace_bytes: bad argument");
    // (the few-row kernel needs none; the tiled kernel splits K over workgroups when its tiles are few)
    *workspace_bytes = (rows >= 8 && num_input % 64 == 0 && !fc_skinny_takes(rows, num_input, num_output))
                           ? conv_nhwc_pipelined_workspace_words(num_output, rows, num_input / 64) * sizeof(int32_t)
                           : 0;
    return NCNNHIP_OK;
}

int ncnnhip_innerproduct_int8_ws(const int8_t* x_dev, size_t x_stride, int rows, int num_input, int num_output, const int8_t* weight_dev,
                                 const float* scale_in_dev, const float* bias_dev, ncnnhip_activation act, float* out_dev, size_t out_stride,
                                 void* workspace_dev, size_t workspace_bytes, void* stream)
{
    NCNNHIP_REQUIRE(x_dev && weight_dev && scale_in_dev && out_dev, "ncnnhip_innerproduct_int8_ws: null pointer");
    NCNNHIP_REQUIRE(rows >= 1 && num_input >= 1 && num_output >= 1, "ncnnhip_innerproduct_int8_ws: bad shape");
    NCNNHIP_REQUIRE(x_stride >= (size_t)num_input && out_stride >= (size_t)num_output, "ncnnhip_innerproduct_int8_ws: stride too small");
    {
        FcEpilogue fe;
        fe.scale_in = scale_in_dev;
        fe.bias = bias_dev;
        fe.act = act;
        fe.out = out_dev;
        fe.out_stride = out_stride;
        fe.num_output = num_output;
        fe.acc_out = 0;
        if (launch_fc_skinny(x_dev, x_stride, rows, num_input, num_output, weight_dev, fe, as_stream(stream))) return launch_status("gemm_skinny_int8_kernel<fc>");
    }
    if (rows >= 8)
    {
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
        bool handled = false;
        int ret = launch_fc_via_conv_pipelined(x_dev, x_stride, rows, num_input, num_output, weight_dev, epi, out_stride, workspace_dev, workspace_bytes,
                                               as_stream(stream), &handled);
        if (handled) return ret;
    }
    return ncnnhip_innerproduct_int8(x_dev, x_stride, rows, num_input, num_output, weight_dev, scale_in_dev, bias_dev, act, out_dev, out_stride, 0, stream);
}

int ncnnhip_gemm_int8_tile_operand(const int8_t* src_dev, size_t src_stride, int rows, int K, int operand, int8_t* dst_dev, void* stream)
{
    NCNNHIP_REQUIRE(src_dev && dst_dev, "ncnnhip_gemm_int8_tile_operand: null pointer");
    NCNNHIP_REQUIRE(rows >= 256 && rows % 256 == 0 && K >= 64 && K % 64 == 0, "ncnnhip_gemm_int8_tile_operand: %d rows of %d (multiples of 256 and 64 only)", rows, K);
    NCNNHIP_REQUIRE(operand == 0 || operand == 1, "ncnnhip_gemm_int8_tile_operand: operand %d (0 = A, 1 = B)", operand);
    NCNNHIP_REQUIRE(src_stride >= (size_t)K && src_stride % 16 == 0 && aligned16(src_dev) && aligned16(dst_dev),
                    "ncnnhip_gemm_int8_tile_operand: rows must be 16-byte aligned");
    return launch_gemm_tile_operand(src_dev, src_stride, rows, K, operand, dst_dev, as_stream(stream));
}

int ncnnhip_gemm_int8_tiled(const int8_t* aq_tiled_dev, const int8_t* bq_tiled_dev, int M, int N, int K, const float* a_scales_dev,
                            const float* b_scales_dev, int n_b_scales, const float* c_dev, int broadcast_type_c, float alpha, float beta,
                            float* out_dev, size_t out_stride, void* stream)
{
    NCNNHIP_REQUIRE(aq_tiled_dev && bq_tiled_dev && a_scales_dev && b_scales_dev && out_dev, "ncnnhip_gemm_int8_tiled: null pointer");
    NCNNHIP_REQUIRE(M >= 256 && N >= 256 && K >= 64 && M % 256 == 0 && N % 256 == 0 && K % 64 == 0,
                    "ncnnhip_gemm_int8_tiled: shape %d %d %d (M, N multiples of 256, K of 64)", M, N, K);
    NCNNHIP_REQUIRE(n_b_scales == 1 || n_b_scales == N, "ncnnhip_gemm_int8_tiled: %d B scales for N=%d", n_b_scales, N);
    const int bt = c_dev ? broadcast_type_c : -1;
    NCNNHIP_REQUIRE(bt == -1 || bt == 4, "ncnnhip_gemm_int8_tiled: C broadcast %d (none or per column only)", bt);
    NCNNHIP_REQUIRE(out_stride >= (size_t)N && out_stride % 4 == 0 && aligned16(out_dev), "ncnnhip_gemm_int8_tiled: output rows must be 16-byte aligned");
    NCNNHIP_REQUIRE(aligned16(aq_tiled_dev) && aligned16(bq_tiled_dev), "ncnnhip_gemm_int8_tiled: operands must be 16-byte aligned");
    GemmEpilogue epi;
    epi.a_scales = a_scales_dev;
    epi.b_scales = b_scales_dev;
    epi.per_col = n_b_scales != 1;
    epi.c = c_dev;
    epi.bt = bt;
    epi.alpha = alpha;
    epi.beta = beta;
    epi.transpose = 0;
    epi.out = out_dev;
    epi.out_stride = out_stride;
    epi.N = N;
    epi.acc_out = 0;
    return launch_gemm_int8_tiled(aq_tiled_dev, bq_tiled_dev, M, N, K, epi, as_stream(stream));
}

} // extern "C"
