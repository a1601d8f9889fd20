// Large aligned int8 Gemm on the gfx950 matrix cores.
//
// One workgroup (4 wavefronts, one per SIMD) owns a 256x256 output tile; each wavefront owns a
// 128x128 quadrant = 4x4 v_mfma_i32_32x32x32_i8 blocks = 256 int32 accumulators per lane.
// K is walked in 64-byte steps through a 4-deep ring of LDS stages (32 KB each: 256 A rows and
// 256 B rows of 64 bytes).  Stages are filled with direct global->LDS 128-bit loads (no register
// staging), three steps ahead of the step being multiplied, so HBM/L2 latency is covered by
// about three steps of matrix work.
//
// LDS layout of one operand stage: row r occupies bytes [64 r, 64 r + 64); its four 16-byte
// chunks are stored at chunk position c ^ ((r >> 2) & 3).  A direct-to-LDS load writes the 64
// lanes' 16-byte items back to back, so the swizzle is applied by choosing which global chunk
// each lane fetches.  With it, any 16 consecutive rows read at one K offset hit 16 different
// 16-byte bank groups.
//
// TILED operands: element (r, k) of an operand lies at ((r / 256 * (K / 64) + k / 64) * 256 + r % 256) * 64 + k % 64, i.e.
// the 256 x 64-byte panel of one tile and one K step is 16 KB of consecutive memory, and every direct-to-LDS load of a
// wavefront fetches one whole KB (eight full 128-byte lines).  From row-major operands the same load touches 16 half
// lines, each line being fetched again one K step later: twice the L2-to-L1 traffic and twice the tag look-ups, which is
// what bounds the row-major kernel (without any fills its K loop runs 25 % faster).  The B operand is tiled with its rows
// already in the column-interleaved order described at the loads below.
//
// Workgroup ids are remapped so that each of the 8 XCDs (ids are dealt round-robin to XCDs)
// works on a compact block of output tiles and re-uses its A/B panels out of its own L2.
#include <type_traits>

#include "epilogues.h"
#include "mfma_tile.h"

#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))

namespace ncnnhip {

constexpr int PT = 256;            // tile edge
constexpr int PK = 64;             // K bytes per stage
constexpr int STAGES = 4;
constexpr int OPERAND_BYTES = PT * PK;        // 16 KB
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES; // 32 KB

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding)
#define WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | ((((n) >> 4) & 3) << 14))


template<bool PER_COL, int BT, bool TILED>
__global__ __launch_bounds__(256) void gemm_int8_256x256_kernel(const int8_t* __restrict__ A, size_t lda, const int8_t* __restrict__ B,
                                                                 size_t ldb, int nk, int tiles_m, int tiles_n,
                                                                 const float* __restrict__ a_scales, const float* __restrict__ b_scales,
                                                                 const float* __restrict__ cvec, float alpha, float beta,
                                                                 float* __restrict__ out, size_t ldo)
{
    __shared__ __attribute__((aligned(1024))) int8_t smem[STAGES * STAGE_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // wave-uniform, lives in an SGPR
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    // ---- XCD-aware tile choice: 8 XCDs take contiguous ranges of a 4-row-grouped tile order
    int b = blockIdx.x;
    const int T = tiles_m * tiles_n;
    if ((T & 7) == 0) b = (b & 7) * (T >> 3) + (b >> 3);
    constexpr int GM = 4;
    const int per_group = GM * tiles_n;
    const int group = b / per_group;
    const int first_m = group * GM;
    const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int in_group = b - group * per_group;
    const int tile_m = first_m + in_group % gsz;
    const int tile_n = in_group / gsz;

    // ---- per-lane global sources of the direct-to-LDS loads
    // load i of wave w fills LDS rows (i*4 + w)*16 .. +16 of the operand stage
    const int ld_row = wave * 16 + (lane >> 2);                 // + i*64
    const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);        // swizzled source chunk
    const int8_t* ga = TILED ? A + ((size_t)tile_m * nk * PT + ld_row) * PK + ld_chunk * 16 : A + ((size_t)tile_m * PT + ld_row) * lda + ld_chunk * 16;
    // B rows are permuted on their way into LDS: LDS row wn*128 + j*32 + l holds B row wn*128 + 4*l + j, so that the four
    // accumulator blocks j of a lane are four consecutive output columns and the epilogue stores 16 bytes per lane.
    // LDS row of this lane in quarter i = i*64 + wave*16 + (lane >> 2): wn = i >> 1, j = (i & 1)*2 + (wave >> 1),
    // l = (wave & 1)*16 + (lane >> 2).
    const int ld_row_b = 4 * ((wave & 1) * 16 + (lane >> 2)) + (wave >> 1); // + (i >> 1)*128 + (i & 1)*2
    const int8_t* gb = TILED ? B + ((size_t)tile_n * nk * PT + ld_row) * PK + ld_chunk * 16 : B + ((size_t)tile_n * PT + ld_row_b) * ldb + ld_chunk * 16;
    const size_t a_step = 64 * lda;

    // quarter i of the loads of step t: 16 A rows and 16 B rows per wave
    auto issue_quarter = [&](int t, int i) {
        int8_t* sa = smem + (t & (STAGES - 1)) * STAGE_BYTES + wave * 1024 + i * 4096;
        const int8_t* pa = TILED ? ga + (size_t)t * OPERAND_BYTES + i * 4096 : ga + (size_t)t * PK + i * a_step;
        const int8_t* pb = TILED ? gb + (size_t)t * OPERAND_BYTES + i * 4096 : gb + (size_t)t * PK + (size_t)((i >> 1) * 128 + (i & 1) * 2) * ldb;
        __builtin_amdgcn_global_load_lds((const AS1 void*)pa, (AS3 void*)sa, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const AS1 void*)pb, (AS3 void*)(sa + OPERAND_BYTES), 16, 0, 0);
    };
    auto issue_one = [&](int t, int i, int which) {
        int8_t* sa = smem + (t & (STAGES - 1)) * STAGE_BYTES + wave * 1024 + i * 4096;
        if (which == 0)
        {
            const int8_t* pa = TILED ? ga + (size_t)t * OPERAND_BYTES + i * 4096 : ga + (size_t)t * PK + i * a_step;
            __builtin_amdgcn_global_load_lds((const AS1 void*)pa, (AS3 void*)sa, 16, 0, 0);
        }
        else
        {
            const int8_t* pb = TILED ? gb + (size_t)t * OPERAND_BYTES + i * 4096 : gb + (size_t)t * PK + (size_t)((i >> 1) * 128 + (i & 1) * 2) * ldb;
            __builtin_amdgcn_global_load_lds((const AS1 void*)pb, (AS3 void*)(sa + OPERAND_BYTES), 16, 0, 0);
        }
    };
    auto issue_stage = [&](int t) {
#pragma unroll
        for (int i = 0; i < 4; i++) issue_quarter(t, i);
    };

    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // ---- per-lane LDS read offsets: fragment row l32 (+32 per block), K chunk ks*2 + lhi, swizzled
    const int sw = (l32 >> 2) & 3;
    const int rd_a0 = (wm * 128 + l32) * PK + ((0 + lhi) ^ sw) * 16;
    const int rd_a1 = (wm * 128 + l32) * PK + ((2 + lhi) ^ sw) * 16;
    const int rd_b0 = OPERAND_BYTES + (wn * 128 + l32) * PK + ((0 + lhi) ^ sw) * 16;
    const int rd_b1 = OPERAND_BYTES + (wn * 128 + l32) * PK + ((2 + lhi) ^ sw) * 16;

    // ---- prologue: three steps in flight
    if (0 < nk) issue_stage(0);
    if (1 < nk) issue_stage(1);
    if (2 < nk) issue_stage(2);

    // Fragment registers are double-buffered (F0 = first 32 bytes of a K step, F1 = second).  The LDS reads and their
    // waits are written as asm so that a wait only covers the reads the next MFMAs need and leaves the others in flight.
    v4i fa0[4], fb0[4], fa1[4], fb1[4];
    const unsigned lds_base = (unsigned)(uintptr_t)(AS3 int8_t*)smem;
    auto frag_addr_a = [&](int t, int ks) { return lds_base + (unsigned)((t & (STAGES - 1)) * STAGE_BYTES) + (ks ? rd_a1 : rd_a0); };
    auto frag_addr_b = [&](int t, int ks) { return lds_base + (unsigned)((t & (STAGES - 1)) * STAGE_BYTES) + (ks ? rd_b1 : rd_b0); };
#define LDS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))
    auto read_frags = [&](int t, int ks, v4i (&fa)[4], v4i (&fb)[4]) {
        const unsigned pa = frag_addr_a(t, ks), pb = frag_addr_b(t, ks);
        LDS_READ(fa[0], pa, 0);
        LDS_READ(fb[0], pb, 0);
        LDS_READ(fb[1], pb, 2048);
        LDS_READ(fb[2], pb, 4096);
        LDS_READ(fb[3], pb, 6144);
        LDS_READ(fa[1], pa, 2048);
        LDS_READ(fa[2], pa, 4096);
        LDS_READ(fa[3], pa, 6144);
    };
    // waits until at most `pending` LDS reads are outstanding and ties the fragment registers to
    // the wait so the MFMAs that use them cannot be moved above it
#define WAIT_FRAGS(pending, fa, fb)                                                                                   \
    asm volatile("s_waitcnt lgkmcnt(" #pending ")"                                                                    \
                 : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]))
#define PIN __builtin_amdgcn_sched_barrier(0)
    auto mma_row = [&](int i, const v4i (&fa)[4], const v4i (&fb)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    auto wait_step = [&](int t) {
        // wait for the loads of step t (8 per step; newer steps may stay in flight)
        if (t + 2 < nk)
            WAIT_VMCNT(16);
        else if (t + 1 < nk)
            WAIT_VMCNT(8);
        else
            WAIT_VMCNT(0);
    };

    wait_step(0);
    __builtin_amdgcn_s_barrier();
    if (3 < nk) issue_stage(3);
    read_frags(0, 0, fa0, fb0);

    // One K step, one memory instruction after each MFMA.  A wavefront issues in order and an MFMA occupies the matrix pipe
    // for 32 cycles, so whatever stands between two MFMAs must issue within those 32 cycles or the pipe idles: the 8 reads of
    // the second fragment set follow the first 8 MFMAs of the step one by one, and after the barrier the 8 reads of the next
    // step's first set alternate with the 8 global->LDS loads of step t+4.  LDS reads return in order, so the wait before a row
    // of MFMAs only covers the reads that row needs (counted in reads still allowed in flight).
#define WAIT_LGKM(n, ...) asm volatile("s_waitcnt lgkmcnt(" #n ")" : __VA_ARGS__)
    auto mma1 = [&](int i, int j, const v4i (&fa)[4], const v4i (&fb)[4]) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    auto k_step_fine = [&](int t, auto steady) {
        constexpr bool STEADY = decltype(steady)::value;
        const bool more = STEADY || t + 1 < nk;
        const bool refill = STEADY || t + 4 < nk;
        const unsigned qa = frag_addr_a(t, 1), qb = frag_addr_b(t, 1);
        // first set: issued in the order fa0[0], fb0[0..3], fa0[1..3]
        WAIT_LGKM(3, "+v"(fa0[0]), "+v"(fb0[0]), "+v"(fb0[1]), "+v"(fb0[2]), "+v"(fb0[3]));
        PIN;
        mma1(0, 0, fa0, fb0); PIN; LDS_READ(fa1[0], qa, 0); PIN;
        mma1(0, 1, fa0, fb0); PIN; LDS_READ(fb1[0], qb, 0); PIN;
        mma1(0, 2, fa0, fb0); PIN; LDS_READ(fb1[1], qb, 2048); PIN;
        mma1(0, 3, fa0, fb0); PIN; LDS_READ(fb1[2], qb, 4096); PIN;
        WAIT_LGKM(6, "+v"(fa0[1]));
        PIN;
        mma1(1, 0, fa0, fb0); PIN; LDS_READ(fb1[3], qb, 6144); PIN;
        mma1(1, 1, fa0, fb0); PIN; LDS_READ(fa1[1], qa, 2048); PIN;
        mma1(1, 2, fa0, fb0); PIN; LDS_READ(fa1[2], qa, 4096); PIN;
        mma1(1, 3, fa0, fb0); PIN; LDS_READ(fa1[3], qa, 6144); PIN;
        WAIT_LGKM(9, "+v"(fa0[2]));
        PIN;
        mma_row(2, fa0, fb0);
        PIN;
        WAIT_LGKM(8, "+v"(fa0[3]));
        PIN;
        mma_row(3, fa0, fb0);
        PIN;
        if (more)
        {
            if (STEADY)
                WAIT_VMCNT(16);
            else
                wait_step(t + 1);
        }
        WAIT_FRAGS(0, fa1, fb1);
        if (more) __builtin_amdgcn_s_barrier();
        PIN;
        const unsigned pa = frag_addr_a(t + 1, 0), pb = frag_addr_b(t + 1, 0);
        mma1(0, 0, fa1, fb1); PIN; if (more) LDS_READ(fa0[0], pa, 0); PIN;
        mma1(0, 1, fa1, fb1); PIN; if (refill) issue_one(t + 4, 0, 0); PIN;
        mma1(0, 2, fa1, fb1); PIN; if (more) LDS_READ(fb0[0], pb, 0); PIN;
        mma1(0, 3, fa1, fb1); PIN; if (refill) issue_one(t + 4, 0, 1); PIN;
        mma1(1, 0, fa1, fb1); PIN; if (more) LDS_READ(fb0[1], pb, 2048); PIN;
        mma1(1, 1, fa1, fb1); PIN; if (refill) issue_one(t + 4, 1, 0); PIN;
        mma1(1, 2, fa1, fb1); PIN; if (more) LDS_READ(fb0[2], pb, 4096); PIN;
        mma1(1, 3, fa1, fb1); PIN; if (refill) issue_one(t + 4, 1, 1); PIN;
        mma1(2, 0, fa1, fb1); PIN; if (more) LDS_READ(fb0[3], pb, 6144); PIN;
        mma1(2, 1, fa1, fb1); PIN; if (refill) issue_one(t + 4, 2, 0); PIN;
        mma1(2, 2, fa1, fb1); PIN; if (more) LDS_READ(fa0[1], pa, 2048); PIN;
        mma1(2, 3, fa1, fb1); PIN; if (refill) issue_one(t + 4, 2, 1); PIN;
        mma1(3, 0, fa1, fb1); PIN; if (more) LDS_READ(fa0[2], pa, 4096); PIN;
        mma1(3, 1, fa1, fb1); PIN; if (refill) issue_one(t + 4, 3, 0); PIN;
        mma1(3, 2, fa1, fb1); PIN; if (more) LDS_READ(fa0[3], pa, 6144); PIN;
        mma1(3, 3, fa1, fb1); PIN; if (refill) issue_one(t + 4, 3, 1); PIN;
    };
    int t = 0;
    for (; t + 4 < nk; t++) k_step_fine(t, std::true_type{});
    for (; t < nk; t++) k_step_fine(t, std::false_type{});

    // ---- fused epilogue: dequantise, bias, scale, store fp32
    const int col_base = tile_n * PT + wn * 128 + 4 * l32; // accumulator block j of this lane is column col_base + j
    float colscale[4], colc[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
    {
        const int col = col_base + j;
        colscale[j] = PER_COL ? div_rn(1.f, b_scales[col]) : 0.f;
        colc[j] = BT == 4 ? mul_rn(cvec[col], beta) : 0.f;
    }
    // one descale per row of the tile, computed once by thread `row` and handed round through LDS (the stages are free
    // once every wavefront has left the K loop)
    float* rowscale_lds = reinterpret_cast<float*>(smem);
    {
        const float sa = a_scales[tile_m * PT + threadIdx.x];
        const float rs = PER_COL ? div_rn(1.f, sa) : div_rn(1.f, mul_rn(sa, b_scales[0]));
        __builtin_amdgcn_s_barrier();
        rowscale_lds[threadIdx.x] = rs;
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
    {
#pragma unroll
        for (int r = 0; r < 16; r++)
        {
            const int row_in_tile = wm * 128 + 4 * lhi + i * 32 + 8 * (r >> 2) + (r & 3);
            const float rowscale = rowscale_lds[row_in_tile];
            float* orow = out + (size_t)(tile_m * PT + row_in_tile) * ldo + col_base;
            float f4[4];
#pragma unroll
            for (int j = 0; j < 4; j++)
            {
                float f = mul_rn((float)acc[i][j][r], rowscale);
                if (PER_COL) f = mul_rn(f, colscale[j]);
                if (BT == 4) f = add_rn(f, colc[j]);
                f4[j] = mul_rn(f, alpha);
            }
            *reinterpret_cast<float4*>(orow) = make_float4(f4[0], f4[1], f4[2], f4[3]); // (non-temporal stores: neutral at 4096 cubed, 3 % slower at 8192 cubed)
        }
    }
}

static inline bool al16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

template<bool TILED>
static int launch_256x256(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K, const GemmEpilogue& epi,
                          hipStream_t stream)
{
    const int tm = M / PT, tn = N / PT, nk = K / PK;
    dim3 grid(tm * tn), block(256);
#define LAUNCH(PC, BTV)                                                                                                                    \
    hipLaunchKernelGGL((gemm_int8_256x256_kernel<PC, BTV, TILED>), grid, block, 0, stream, aq, aq_stride, bq, bq_stride, nk, tm, tn,        \
                       epi.a_scales, epi.b_scales, epi.c, epi.alpha, epi.beta, epi.out, epi.out_stride)
    if (epi.per_col)
    {
        if (epi.bt == 4)
            LAUNCH(true, 4);
        else
            LAUNCH(true, -1);
    }
    else
    {
        if (epi.bt == 4)
            LAUNCH(false, 4);
        else
            LAUNCH(false, -1);
    }
#undef LAUNCH
    return launch_status("gemm_int8_256x256_kernel");
}

int launch_gemm_int8_pipelined(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K,
                               const GemmEpilogue& epi, hipStream_t stream, bool* handled)
{
    *handled = false;
    if (M % PT || N % PT || K % PK || aq_stride % 16 || bq_stride % 16 || !al16(aq) || !al16(bq)) return NCNNHIP_OK;
    if (epi.transpose || epi.acc_out || !(epi.bt == -1 || epi.bt == 4)) return NCNNHIP_OK;
    if (epi.out_stride % 4 || !al16(epi.out)) return NCNNHIP_OK; // the epilogue stores 16 bytes per lane
    if ((long long)(M / PT) * (N / PT) > 0x7fffffff) return NCNNHIP_OK;
    *handled = true;
    return launch_256x256<false>(aq, aq_stride, bq, bq_stride, M, N, K, epi, stream);
}

// operands in the tiled layout; the caller has checked shapes and alignment
int launch_gemm_int8_tiled(const int8_t* aq_tiled, const int8_t* bq_tiled, int M, int N, int K, const GemmEpilogue& epi, hipStream_t stream)
{
    return launch_256x256<true>(aq_tiled, 0, bq_tiled, 0, M, N, K, epi, stream);
}

// row-major [rows][K] -> tiled; operand_b: position p of a 256-row tile holds row (p >> 7)*128 + 4*(p & 31) + ((p >> 5) & 3),
// the order in which the kernel wants the rows of B in LDS.  One 16-byte chunk per thread.
__global__ __launch_bounds__(256) void gemm_tile_operand_kernel(const int8_t* __restrict__ src, size_t stride, int nk, size_t chunks, int operand_b,
                                                                 int8_t* __restrict__ dst)
{
    const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= chunks) return;
    const int c = (int)(g & 3);
    const int p = (int)((g >> 2) & 255);
    const size_t panel = g >> 10; // tile * nk + t
    const size_t tile = panel / nk;
    const int t = (int)(panel - tile * nk);
    const int r = operand_b ? (p >> 7) * 128 + 4 * (p & 31) + ((p >> 5) & 3) : p;
    const v4i v = *reinterpret_cast<const v4i*>(src + (tile * PT + r) * stride + (size_t)t * PK + c * 16);
    *reinterpret_cast<v4i*>(dst + g * 16) = v;
}

int launch_gemm_tile_operand(const int8_t* src, size_t stride, int rows, int K, int operand_b, int8_t* dst, hipStream_t stream)
{
    const size_t chunks = (size_t)rows * K / 16;
    const size_t blocks = (chunks + 255) / 256;
    if (blocks > 0x7fffffffull) return NCNNHIP_ERROR;
    hipLaunchKernelGGL(gemm_tile_operand_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, stride, K / PK, chunks, operand_b, dst);
    return launch_status("gemm_tile_operand_kernel");
}

} // namespace ncnnhip
