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
#include <cstdlib>
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

// ---------------------------------------------------------------------------------------------------------------------------
// The same ring with a 128x128 output tile, for problems that have too few 256x256 tiles to fill 256 CUs (1024 cubed is
// 16 of them, 2048 cubed 64).  Four wavefronts own 64x64 quadrants (2x2 blocks, 64 accumulators per lane); a stage is 128 A
// rows and 128 B rows of 64 bytes (16 KB), S stages deep.  A wavefront issues 4 direct-to-LDS loads, 8 LDS reads and 8 MFMA
// per K step; the loads of step t + S and the reads of step t + 1 are dealt out between the MFMAs of step t as above.  Per
// output the tile reads twice the operand bytes of the 256x256 tile, which is what it costs to have four times the tiles.
constexpr int QT = 128;
constexpr int Q_OPERAND = QT * PK;     // 8 KB
constexpr int Q_STAGE = 2 * Q_OPERAND; // 16 KB

template<bool PER_COL, int BT, int S>
__global__ __launch_bounds__(256) void gemm_int8_128x128_kernel(const int8_t* __restrict__ A, size_t lda, const int8_t* __restrict__ B, size_t ldb, int nk,
                                                                 int tiles_m, int tiles_n, const float* __restrict__ a_scales,
                                                                 const float* __restrict__ b_scales, const float* __restrict__ cvec, float alpha, float beta,
                                                                 float* __restrict__ out, size_t ldo)
{
    static_assert(S == 4 || S == 8, "the ring is indexed with a mask");
    __shared__ __attribute__((aligned(1024))) int8_t smem[S * Q_STAGE];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    // XCD-aware tile choice, as in the 256x256 kernel
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

    // load i (0, 1) of wave w fills LDS rows i*64 + w*16 .. +16 of an operand stage; chunks swizzled as in the 256x256 kernel
    const int ld_row = wave * 16 + (lane >> 2);
    const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);
    const int8_t* ga = A + ((size_t)tile_m * QT + ld_row) * lda + ld_chunk * 16;
    // LDS row wn*64 + j*32 + l holds B row wn*64 + 2*l + j: the two accumulator blocks j of a lane are two consecutive output
    // columns (8-byte stores).  LDS row of this lane in half i = i*64 + wave*16 + (lane >> 2): wn = i, j = wave >> 1,
    // l = (wave & 1)*16 + (lane >> 2).
    const int ld_row_b = 2 * ((wave & 1) * 16 + (lane >> 2)) + (wave >> 1);
    const int8_t* gb = B + ((size_t)tile_n * QT + ld_row_b) * ldb + ld_chunk * 16;
    const size_t a_half = 64 * lda, b_half = 64 * ldb;

    auto issue_one = [&](int t, int i, int which) {
        int8_t* sa = smem + (t & (S - 1)) * Q_STAGE + wave * 1024 + i * 4096;
        if (which == 0)
            __builtin_amdgcn_global_load_lds((const AS1 void*)(ga + (size_t)t * PK + i * a_half), (AS3 void*)sa, 16, 0, 0);
        else
            __builtin_amdgcn_global_load_lds((const AS1 void*)(gb + (size_t)t * PK + i * b_half), (AS3 void*)(sa + Q_OPERAND), 16, 0, 0);
    };
    auto issue_stage = [&](int t) {
        issue_one(t, 0, 0);
        issue_one(t, 0, 1);
        issue_one(t, 1, 0);
        issue_one(t, 1, 1);
    };

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // what the epilogue needs from memory is requested now, so that it has arrived long before the K loop ends
    const int col_base = tile_n * QT + wn * 64 + 2 * l32; // accumulator block j of this lane is column col_base + j
    // (as asm: these loads must stand before the direct-to-LDS loads, whose waits count instructions; EARLY_ARRIVED below ties
    // the values to a point behind the K loop, where every load of the wavefront has returned)
    float early_sa, early_sb[2] = {0.f, 0.f}, early_c[2] = {0.f, 0.f};
#define EARLY_LOAD(dst, ptr) asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory")
    EARLY_LOAD(early_sa, a_scales + tile_m * QT + (threadIdx.x & (QT - 1)));
    EARLY_LOAD(early_sb[0], b_scales + (PER_COL ? col_base : 0));
    if (PER_COL) EARLY_LOAD(early_sb[1], b_scales + col_base + 1);
    if (BT == 4)
    {
        EARLY_LOAD(early_c[0], cvec + col_base);
        EARLY_LOAD(early_c[1], cvec + col_base + 1);
    }
#undef EARLY_LOAD
#define EARLY_ARRIVED asm volatile("s_waitcnt vmcnt(0)" : "+v"(early_sa), "+v"(early_sb[0]), "+v"(early_sb[1]), "+v"(early_c[0]), "+v"(early_c[1]))
    PIN;

    const int sw = (l32 >> 2) & 3;
    const int rd_a0 = (wm * 64 + l32) * PK + ((0 + lhi) ^ sw) * 16;
    const int rd_a1 = (wm * 64 + l32) * PK + ((2 + lhi) ^ sw) * 16;
    const int rd_b0 = Q_OPERAND + (wn * 64 + l32) * PK + ((0 + lhi) ^ sw) * 16;
    const int rd_b1 = Q_OPERAND + (wn * 64 + l32) * PK + ((2 + lhi) ^ sw) * 16;
    const unsigned lds_base = (unsigned)(uintptr_t)(AS3 int8_t*)smem;
    auto frag_addr_a = [&](int t, int ks) { return lds_base + (unsigned)((t & (S - 1)) * Q_STAGE) + (ks ? rd_a1 : rd_a0); };
    auto frag_addr_b = [&](int t, int ks) { return lds_base + (unsigned)((t & (S - 1)) * Q_STAGE) + (ks ? rd_b1 : rd_b0); };

    // at most `newer` stages (4 loads each) may stay in flight
    auto wait_stages = [&](int newer) {
        switch (newer)
        {
        case 0: WAIT_VMCNT(0); break;
        case 1: WAIT_VMCNT(4); break;
        case 2: WAIT_VMCNT(8); break;
        case 3: WAIT_VMCNT(12); break;
        case 4: WAIT_VMCNT(16); break;
        case 5: WAIT_VMCNT(20); break;
        default: WAIT_VMCNT(24); break;
        }
    };

    // ---- prologue: the whole ring in flight
#pragma unroll
    for (int t0 = 0; t0 < S; t0++)
        if (t0 < nk) issue_stage(t0);
    {
        const int newer = nk - 1 < S - 1 ? nk - 1 : S - 1;
        if (newer == S - 1)
            WAIT_VMCNT((S - 1) * 4);
        else
            wait_stages(newer);
    }
    __builtin_amdgcn_s_barrier();

    v4i fa0[2], fb0[2], fa1[2], fb1[2];
    {
        const unsigned pa = frag_addr_a(0, 0), pb = frag_addr_b(0, 0);
        LDS_READ(fa0[0], pa, 0);
        LDS_READ(fb0[0], pb, 0);
        LDS_READ(fb0[1], pb, 2048);
        LDS_READ(fa0[1], pa, 2048);
    }
    auto mma1 = [&](int i, int j, const v4i (&fa)[2], const v4i (&fb)[2]) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    auto k_step = [&](int t, auto steady) {
        constexpr bool STEADY = decltype(steady)::value;
        const bool more = STEADY || t + 1 < nk;
        const bool refill = STEADY || t + S < nk;
        const unsigned qa = frag_addr_a(t, 1), qb = frag_addr_b(t, 1);
        // first set: requested in the order fa0[0], fb0[0], fb0[1], fa0[1]
        WAIT_LGKM(1, "+v"(fa0[0]), "+v"(fb0[0]), "+v"(fb0[1]));
        PIN;
        mma1(0, 0, fa0, fb0); PIN; LDS_READ(fa1[0], qa, 0); PIN;
        mma1(0, 1, fa0, fb0); PIN; LDS_READ(fb1[0], qb, 0); PIN;
        WAIT_LGKM(2, "+v"(fa0[1]));
        PIN;
        mma1(1, 0, fa0, fb0); PIN; LDS_READ(fb1[1], qb, 2048); PIN;
        mma1(1, 1, fa0, fb0); PIN; LDS_READ(fa1[1], qa, 2048); PIN;
        if (more)
        {
            // the loads of step t + 1; stages t + 2 .. t + S - 1 may stay in flight
            if (STEADY)
                WAIT_VMCNT((S - 2) * 4);
            else
                wait_stages(nk - 2 - t < S - 2 ? nk - 2 - t : S - 2);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa1[0]), "+v"(fa1[1]), "+v"(fb1[0]), "+v"(fb1[1]));
        if (more) __builtin_amdgcn_s_barrier();
        PIN;
        const unsigned pa = frag_addr_a(t + 1, 0), pb = frag_addr_b(t + 1, 0);
        mma1(0, 0, fa1, fb1); PIN; if (more) LDS_READ(fa0[0], pa, 0); PIN; if (refill) issue_one(t + S, 0, 0); PIN;
        mma1(0, 1, fa1, fb1); PIN; if (more) LDS_READ(fb0[0], pb, 0); PIN; if (refill) issue_one(t + S, 0, 1); PIN;
        mma1(1, 0, fa1, fb1); PIN; if (more) LDS_READ(fb0[1], pb, 2048); PIN; if (refill) issue_one(t + S, 1, 0); PIN;
        mma1(1, 1, fa1, fb1); PIN; if (more) LDS_READ(fa0[1], pa, 2048); PIN; if (refill) issue_one(t + S, 1, 1); PIN;
    };
    int t = 0;
    for (; t + S < nk; t++) k_step(t, std::true_type{});
    for (; t < nk; t++) k_step(t, std::false_type{});

    // ---- fused epilogue: dequantise, bias, scale, store fp32
    EARLY_ARRIVED;
#undef EARLY_ARRIVED
    float colscale[2], colc[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
    {
        colscale[j] = PER_COL ? div_rn(1.f, early_sb[j]) : 0.f;
        colc[j] = BT == 4 ? mul_rn(early_c[j], beta) : 0.f;
    }
    float* rowscale_lds = reinterpret_cast<float*>(smem);
    {
        const float rs = PER_COL ? div_rn(1.f, early_sa) : div_rn(1.f, mul_rn(early_sa, early_sb[0]));
        __builtin_amdgcn_s_barrier(); // every wavefront has left the K loop: the stages are free
        if (threadIdx.x < QT) rowscale_lds[threadIdx.x] = rs;
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
    {
#pragma unroll
        for (int r = 0; r < 16; r++)
        {
            const int row_in_tile = wm * 64 + 4 * lhi + i * 32 + 8 * (r >> 2) + (r & 3);
            const float rowscale = rowscale_lds[row_in_tile];
            float* orow = out + (size_t)(tile_m * QT + row_in_tile) * ldo + col_base;
            float f2[2];
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                float f = mul_rn((float)acc[i][j][r], rowscale);
                if (PER_COL) f = mul_rn(f, colscale[j]);
                if (BT == 4) f = add_rn(f, colc[j]);
                f2[j] = mul_rn(f, alpha);
            }
            *reinterpret_cast<float2*>(orow) = make_float2(f2[0], f2[1]);
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

// The 128x128 tile with K steps of 128 bytes (K % 128 == 0).  A direct-to-LDS load of a wavefront then fetches 8 whole 128-byte
// lines instead of 16 half lines: the fills of this tile are bound by the lines a CU can have in flight (about 32 KB of 64-byte
// pieces), not by bytes, and whole lines double what that buys.  A stage is 128 A rows and 128 B rows of 128 bytes (32 KB), four
// stages; row r keeps its eight 16-byte chunks at positions c ^ ((r >> 1) & 7), which spreads any 16 consecutive rows read at one
// K offset over the 16 bank groups.  Per K step a wavefront issues 8 loads, 16 LDS reads and 16 MFMA; the step's four quarters
// alternate between two fragment sets, the barrier stands before the last quarter (all reads of the stage are done by then), and
// the loads of step t + 4 and the first reads of step t + 1 go between the last quarter's MFMAs.  Global addresses are a uniform
// base (SGPRs, advanced per step) plus a per-lane 32-bit offset, so the loop spends no vector instructions on them.
constexpr int RK = 128;
constexpr int R_OPERAND = QT * RK;     // 16 KB
constexpr int R_STAGE = 2 * R_OPERAND; // 32 KB
constexpr int R_STAGES = 4;

template<bool PER_COL, int BT>
__global__ __launch_bounds__(256) void gemm_int8_128x128_k128_kernel(const int8_t* __restrict__ A, size_t lda, const int8_t* __restrict__ B, size_t ldb,
                                                                      int nk, int tiles_m, int tiles_n, const float* __restrict__ a_scales,
                                                                      const float* __restrict__ b_scales, const float* __restrict__ cvec, float alpha,
                                                                      float beta, float* __restrict__ out, size_t ldo)
{
    constexpr int S = R_STAGES;
    __shared__ __attribute__((aligned(1024))) int8_t smem[S * R_STAGE];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

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

    // load i (0..3) of wave w fills LDS rows (i*4 + w)*8 .. +8 of an operand stage: lane l writes row + (l >> 3), chunk position l & 7,
    // and fetches the chunk that belongs there: (l & 7) ^ ((row >> 1) & 7) with row >> 1 = 4*(i*4 + w) + (l >> 4)
    const int ld_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    const int8_t* ua = A + (size_t)tile_m * QT * lda; // uniform
    const int8_t* ub = B + (size_t)tile_n * QT * ldb;
    unsigned off_a[4], off_b[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
    {
        const int row_a = (i * 4 + wave) * 8 + (lane >> 3);
        // LDS row wn*64 + j*32 + l holds B row wn*64 + 2*l + j (two consecutive output columns per lane): here wn = i >> 1, j = i & 1,
        // l = wave*8 + (lane >> 3)
        const int row_b = (i >> 1) * 64 + 2 * (wave * 8 + (lane >> 3)) + (i & 1);
        off_a[i] = (unsigned)(row_a * lda + ld_chunk * 16);
        off_b[i] = (unsigned)(row_b * ldb + ld_chunk * 16);
    }
    auto issue_one = [&](int t, int i, int which) {
        int8_t* sa = smem + (t & (S - 1)) * R_STAGE + (i * 4 + wave) * 1024;
        if (which == 0)
            __builtin_amdgcn_global_load_lds((const AS1 void*)(ua + (size_t)t * RK + off_a[i]), (AS3 void*)sa, 16, 0, 0);
        else
            __builtin_amdgcn_global_load_lds((const AS1 void*)(ub + (size_t)t * RK + off_b[i]), (AS3 void*)(sa + R_OPERAND), 16, 0, 0);
    };
    auto issue_stage = [&](int t) {
#pragma unroll
        for (int i = 0; i < 4; i++)
        {
            issue_one(t, i, 0);
            issue_one(t, i, 1);
        }
    };

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // what the epilogue needs from memory is requested now, so that it has arrived long before the K loop ends
    const int col_base = tile_n * QT + wn * 64 + 2 * l32; // accumulator block j of this lane is column col_base + j
    // (as asm: these loads must stand before the direct-to-LDS loads, whose waits count instructions; EARLY_ARRIVED below ties
    // the values to a point behind the K loop, where every load of the wavefront has returned)
    float early_sa, early_sb[2] = {0.f, 0.f}, early_c[2] = {0.f, 0.f};
#define EARLY_LOAD(dst, ptr) asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory")
    EARLY_LOAD(early_sa, a_scales + tile_m * QT + (threadIdx.x & (QT - 1)));
    EARLY_LOAD(early_sb[0], b_scales + (PER_COL ? col_base : 0));
    if (PER_COL) EARLY_LOAD(early_sb[1], b_scales + col_base + 1);
    if (BT == 4)
    {
        EARLY_LOAD(early_c[0], cvec + col_base);
        EARLY_LOAD(early_c[1], cvec + col_base + 1);
    }
#undef EARLY_LOAD
#define EARLY_ARRIVED asm volatile("s_waitcnt vmcnt(0)" : "+v"(early_sa), "+v"(early_sb[0]), "+v"(early_sb[1]), "+v"(early_c[0]), "+v"(early_c[1]))
    PIN;

    // fragment of quarter q (32 bytes of K): chunk 2q + lhi of row l32 (+32 for the second block), swizzled
    const int sw = (l32 >> 1) & 7;
    int rd_a[4], rd_b[4];
#pragma unroll
    for (int q = 0; q < 4; q++)
    {
        rd_a[q] = (wm * 64 + l32) * RK + ((2 * q + lhi) ^ sw) * 16;
        rd_b[q] = R_OPERAND + (wn * 64 + l32) * RK + ((2 * q + lhi) ^ sw) * 16;
    }
    const unsigned lds_base = (unsigned)(uintptr_t)(AS3 int8_t*)smem;

    auto wait_stages = [&](int newer) { // at most `newer` stages (8 loads each) may stay in flight
        switch (newer)
        {
        case 0: WAIT_VMCNT(0); break;
        case 1: WAIT_VMCNT(8); break;
        case 2: WAIT_VMCNT(16); break;
        default: WAIT_VMCNT(24); break;
        }
    };

    // ---- prologue: the whole ring in flight
#pragma unroll
    for (int t0 = 0; t0 < S; t0++)
        if (t0 < nk) issue_stage(t0);
    wait_stages(nk - 1 < S - 1 ? nk - 1 : S - 1);
    __builtin_amdgcn_s_barrier();

    v4i fa0[2], fb0[2], fa1[2], fb1[2];
    // requests one quarter's fragments in the order a[0], b[0], b[1], a[1]
#define REQUEST_QUARTER(fa, fb, stage_base, q)                  \
    do                                                          \
    {                                                           \
        const unsigned pa_ = (stage_base) + (unsigned)rd_a[q];  \
        const unsigned pb_ = (stage_base) + (unsigned)rd_b[q];  \
        LDS_READ(fa[0], pa_, 0);                                \
        LDS_READ(fb[0], pb_, 0);                                \
        LDS_READ(fb[1], pb_, 4096);                             \
        LDS_READ(fa[1], pa_, 4096);                             \
    } while (0)
    REQUEST_QUARTER(fa0, fb0, lds_base, 0);

    auto mma1 = [&](int i, int j, const v4i (&fa)[2], const v4i (&fb)[2]) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    // one quarter's four MFMAs with the next quarter's four reads between them (LDS answers in order: the wait before a product
    // counts the reads that may still be out)
#define QUARTER(fa, fb, na, nb, stage_base, nq)                                          \
    do                                                                                   \
    {                                                                                    \
        const unsigned pa_ = (stage_base) + (unsigned)rd_a[nq];                          \
        const unsigned pb_ = (stage_base) + (unsigned)rd_b[nq];                          \
        WAIT_LGKM(1, "+v"(fa[0]), "+v"(fb[0]), "+v"(fb[1]));                             \
        PIN;                                                                             \
        mma1(0, 0, fa, fb); PIN; LDS_READ(na[0], pa_, 0); PIN;                           \
        mma1(0, 1, fa, fb); PIN; LDS_READ(nb[0], pb_, 0); PIN;                           \
        WAIT_LGKM(2, "+v"(fa[1]));                                                       \
        PIN;                                                                             \
        mma1(1, 0, fa, fb); PIN; LDS_READ(nb[1], pb_, 4096); PIN;                        \
        mma1(1, 1, fa, fb); PIN; LDS_READ(na[1], pa_, 4096); PIN;                        \
    } while (0)
    auto k_step = [&](int t, auto steady) {
        constexpr bool STEADY = decltype(steady)::value;
        const bool more = STEADY || t + 1 < nk;
        const bool refill = STEADY || t + S < nk;
        const unsigned cur = lds_base + (unsigned)((t & (S - 1)) * R_STAGE);
        const unsigned nxt = lds_base + (unsigned)(((t + 1) & (S - 1)) * R_STAGE);
        QUARTER(fa0, fb0, fa1, fb1, cur, 1);
        QUARTER(fa1, fb1, fa0, fb0, cur, 2);
        QUARTER(fa0, fb0, fa1, fb1, cur, 3);
        if (more)
        {
            // the loads of step t + 1; stages t + 2 .. t + S - 1 may stay in flight
            if (STEADY)
                WAIT_VMCNT((S - 2) * 8);
            else
                wait_stages(nk - 2 - t < S - 2 ? nk - 2 - t : S - 2);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa1[0]), "+v"(fa1[1]), "+v"(fb1[0]), "+v"(fb1[1]));
        if (more) __builtin_amdgcn_s_barrier(); // every wavefront has read the last of stage t and seen its own loads of stage t + 1
        PIN;
        const unsigned pa = nxt + (unsigned)rd_a[0], pb = nxt + (unsigned)rd_b[0];
        mma1(0, 0, fa1, fb1); PIN; if (more) LDS_READ(fa0[0], pa, 0); PIN; if (refill) { issue_one(t + S, 0, 0); issue_one(t + S, 0, 1); } PIN;
        mma1(0, 1, fa1, fb1); PIN; if (more) LDS_READ(fb0[0], pb, 0); PIN; if (refill) { issue_one(t + S, 1, 0); issue_one(t + S, 1, 1); } PIN;
        mma1(1, 0, fa1, fb1); PIN; if (more) LDS_READ(fb0[1], pb, 4096); PIN; if (refill) { issue_one(t + S, 2, 0); issue_one(t + S, 2, 1); } PIN;
        mma1(1, 1, fa1, fb1); PIN; if (more) LDS_READ(fa0[1], pa, 4096); PIN; if (refill) { issue_one(t + S, 3, 0); issue_one(t + S, 3, 1); } PIN;
    };
    int t = 0;
    for (; t + S < nk; t++) k_step(t, std::true_type{});
    for (; t < nk; t++) k_step(t, std::false_type{});
#undef QUARTER
#undef REQUEST_QUARTER

    // ---- fused epilogue: dequantise, bias, scale, store fp32
    EARLY_ARRIVED;
#undef EARLY_ARRIVED
    float colscale[2], colc[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
    {
        colscale[j] = PER_COL ? div_rn(1.f, early_sb[j]) : 0.f;
        colc[j] = BT == 4 ? mul_rn(early_c[j], beta) : 0.f;
    }
    float* rowscale_lds = reinterpret_cast<float*>(smem);
    {
        const float rs = PER_COL ? div_rn(1.f, early_sa) : div_rn(1.f, mul_rn(early_sa, early_sb[0]));
        __builtin_amdgcn_s_barrier(); // every wavefront has left the K loop: the stages are free
        if (threadIdx.x < QT) rowscale_lds[threadIdx.x] = rs;
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
    {
#pragma unroll
        for (int r = 0; r < 16; r++)
        {
            const int row_in_tile = wm * 64 + 4 * lhi + i * 32 + 8 * (r >> 2) + (r & 3);
            const float rowscale = rowscale_lds[row_in_tile];
            float* orow = out + (size_t)(tile_m * QT + row_in_tile) * ldo + col_base;
            float f2[2];
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                float f = mul_rn((float)acc[i][j][r], rowscale);
                if (PER_COL) f = mul_rn(f, colscale[j]);
                if (BT == 4) f = add_rn(f, colc[j]);
                f2[j] = mul_rn(f, alpha);
            }
            *reinterpret_cast<float2*>(orow) = make_float2(f2[0], f2[1]);
        }
    }
}

template<int KSTEP>
static int launch_128x128(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K, const GemmEpilogue& epi, hipStream_t stream)
{
    const int tm = M / QT, tn = N / QT, nk = K / KSTEP;
    dim3 grid(tm * tn), block(256);
#define LAUNCH(PC, BTV)                                                                                                                              \
    do                                                                                                                                               \
    {                                                                                                                                                \
        if (KSTEP == 128)                                                                                                                            \
            hipLaunchKernelGGL((gemm_int8_128x128_k128_kernel<PC, BTV>), grid, block, 0, stream, aq, aq_stride, bq, bq_stride, nk, tm, tn,           \
                               epi.a_scales, epi.b_scales, epi.c, epi.alpha, epi.beta, epi.out, epi.out_stride);                                     \
        else                                                                                                                                         \
            hipLaunchKernelGGL((gemm_int8_128x128_kernel<PC, BTV, 4>), grid, block, 0, stream, aq, aq_stride, bq, bq_stride, nk, tm, tn,             \
                               epi.a_scales, epi.b_scales, epi.c, epi.alpha, epi.beta, epi.out, epi.out_stride);                                     \
    } while (0)
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
    return launch_status("gemm_int8_128x128_kernel");
}

// Problems between the few-row kernels and the 256x256 kernel: M and N multiples of 128 (the caller decides from how many tiles up).
// K % 128 == 0 takes the form with 128-byte K steps, other K % 64 == 0 the form with 64-byte steps.
// NCNNHIP_GEMM_RING128 (read at every call): 0 switches both off, 64 forces the 64-byte form.
int launch_gemm_int8_ring128(const int8_t* aq, size_t aq_stride, const int8_t* bq, size_t bq_stride, int M, int N, int K, const GemmEpilogue& epi,
                             hipStream_t stream, bool* handled)
{
    *handled = false;
    if (M % QT || N % QT || K % PK || aq_stride % 16 || bq_stride % 16 || !al16(aq) || !al16(bq)) return NCNNHIP_OK;
    if (epi.transpose || epi.acc_out || !(epi.bt == -1 || epi.bt == 4)) return NCNNHIP_OK;
    if (epi.out_stride % 2 || (reinterpret_cast<uintptr_t>(epi.out) & 7)) return NCNNHIP_OK; // the epilogue stores 8 bytes per lane
    if ((unsigned long long)QT * aq_stride + 256 > 0xffffffffull || (unsigned long long)QT * bq_stride + 256 > 0xffffffffull) return NCNNHIP_OK; // 32-bit lane offsets
    const char* e = getenv("NCNNHIP_GEMM_RING128");
    const int mode = e ? atoi(e) : 128;
    if (mode == 0) return NCNNHIP_OK;
    *handled = true;
    if (K % RK == 0 && mode != 64) return launch_128x128<128>(aq, aq_stride, bq, bq_stride, M, N, K, epi, stream);
    return launch_128x128<64>(aq, aq_stride, bq, bq_stride, M, N, K, epi, stream);
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
