// int8 Convolution (group 1, zero border) on channels-last blobs for layers with MANY output pixels (batched nets):
// the weights of a block of output channels stay in LDS for the life of the workgroup and the input reaches LDS once.
//
// GEMM view: D[channel][pixel] = sum_k W[channel][k] * X[pixel][k], k = (tap, input channel).  Output channels are the
// A operand (rows) and pixels the B operand (columns) of v_mfma_i32_32x32x32_i8, so a lane's accumulators are 16
// channels of ONE pixel, four runs of four consecutive channels: requantised, a run is one dword, two lane-half swaps
// turn a lane's four dwords into 16 consecutive bytes of its pixel, and the results go from registers to global memory
// without passing through LDS (fp32 results: each run is one 16-byte store).
//
// A workgroup (4 wavefronts) owns BN output channels -- all K bytes of their packed weight rows are fetched into LDS
// once, rows padded by 16 bytes so that the 128-bit fragment reads of 16 consecutive rows fall on different banks --
// and walks pixel tiles of BM pixels.  The input of a tile is fetched ONCE into LDS as "pixels x channels", again with
// 16 bytes of padding per pixel, by direct global->LDS loads whose per-lane source address is where the im2col
// arithmetic happens:
//   * kernels with taps: a tile is R whole output rows (counted over the stack of images), its patch the rows of the
//     VIRTUAL padded image stack (every image with its zero border around it, images stacked) those rows touch.  A
//     wavefront fetches whole rows: which image row that is, whether it exists, and where it starts are scalar
//     arithmetic; a lane's column offset and whether its column is a border column never change, so a fetch costs a
//     couple of vector instructions.  Border columns are never written (they were cleared once), border rows come from
//     a line of zeros.  In that stack an output pixel's tap is at base(pixel) + (ky * dilation * Wp + kx * dilation),
//     the same offset for every pixel, so the K loop adds one scalar per tap to each fragment address and selects
//     nothing.  A 3x3 layer reads each input value from global memory once instead of nine times.
//   * 1x1 kernels: a tile is BM consecutive pixels, the patch those pixels (stride applied by the source address).
// Inside a tile the K loop touches LDS only: no barrier, no wait on memory.  The next tile's patch is requested into
// the other patch buffer before the K loop of this one (when two patches fit), so a workgroup waits for memory once.
// Two workgroups share a compute unit (at most half its LDS and 256 registers each): one's vector work -- patch
// addresses, the requantising epilogue -- issues in the shadow of the other's matrix instructions.
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "conv_nhwc.h"
#include "mfma_tile.h"

#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))

namespace ncnnhip {

static __device__ __attribute__((aligned(64))) int8_t g_resident_zero_line[64];

typedef float v4f __attribute__((ext_vector_type(4)));

struct ResidentPlan
{
    int H, W, Cp, kw, kh, dw, dh, sw, sh, pad_top, pad_left, outw, outh, npix, batch, cout, out_cp, Ktot;
    int Hp, Wp, plane; // the virtual padded image; output pixels per image
    int ntaps;
    int nh;            // 32-byte K pieces per tap
    int n5, nw;        // 16-byte slots per patch pixel / per weight row in LDS (odd)
    int data_chunks_a; // 16-byte chunks of a pixel that hold data
    int data_chunks_w; // ... of a weight row
    int R;             // kernels with taps: output rows (over the stack of images) per tile
    int total_rows;    // batch * outh
    int rows_cap;      // rows of the virtual stack a patch buffer holds
    int row_slots;     // Wp * n5: 16-byte slots of one patch row
    int row_iters;     // wavefront loads per patch row
    int w_slots;       // BN * nw
    int tiles, groups, n_cg;
    int lds_tab, lds_w, lds_patch0, lds_patch1; // byte offsets into dynamic LDS
    unsigned magic_n5, magic_nw, magic_hp, magic_outw, magic_outh, magic_plane, magic_ncg;
};

// n / d by multiplication with magic = 2^32 / d + 1 (exact while n * d < 2^32, which the launch checks); d == 1 has magic 0
__device__ __forceinline__ unsigned mdiv(unsigned n, unsigned magic)
{
    return magic ? __umulhi(n, magic) : n;
}

__device__ __forceinline__ void lds_read128(v4i& dst, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1" : "=v"(dst) : "v"(addr));
}
__device__ __forceinline__ void lds_read128f(v4f& dst, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1" : "=v"(dst) : "v"(addr));
}

// s_waitcnt lgkmcnt(PENDING) that the fragment registers pass through: the products that use them depend on it and
// cannot be scheduled above it
template<int PENDING>
__device__ __forceinline__ void wait_fragments(v4i (&fa)[1], v4i (&fw)[1])
{
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(fa[0]), "+v"(fw[0]) : "n"(PENDING));
}
template<int PENDING>
__device__ __forceinline__ void wait_fragments(v4i (&fa)[1], v4i (&fw)[2])
{
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(fa[0]), "+v"(fw[0]), "+v"(fw[1]) : "n"(PENDING));
}
template<int PENDING>
__device__ __forceinline__ void wait_fragments(v4i (&fa)[2], v4i (&fw)[1])
{
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fw[0]) : "n"(PENDING));
}
template<int PENDING>
__device__ __forceinline__ void wait_fragments(v4i (&fa)[2], v4i (&fw)[2])
{
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fw[0]), "+v"(fw[1]) : "n"(PENDING));
}

// Round half away from zero and pack: values already clamped to [-127, 127] (so the rounding cannot leave that range)
// become bytes.  y = trunc(c + copysign(0.5, c)) with the add rounded toward zero (see float2int8_as_float in
// common.h); one switch of the rounding mode for all the adds of a call.  Two words advance together so that no
// sub-dword write is followed directly by an access to the same register (the chip wants one wait state there).
__device__ __forceinline__ void round_pack_2x4(float (&c)[8], uint32_t& w0, uint32_t& w1)
{
    float t;
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
                 "v_and_or_b32 %10, %0, %11, 0.5\n\tv_add_f32 %0, %0, %10\n\t"
                 "v_and_or_b32 %10, %1, %11, 0.5\n\tv_add_f32 %1, %1, %10\n\t"
                 "v_and_or_b32 %10, %2, %11, 0.5\n\tv_add_f32 %2, %2, %10\n\t"
                 "v_and_or_b32 %10, %3, %11, 0.5\n\tv_add_f32 %3, %3, %10\n\t"
                 "v_and_or_b32 %10, %4, %11, 0.5\n\tv_add_f32 %4, %4, %10\n\t"
                 "v_and_or_b32 %10, %5, %11, 0.5\n\tv_add_f32 %5, %5, %10\n\t"
                 "v_and_or_b32 %10, %6, %11, 0.5\n\tv_add_f32 %6, %6, %10\n\t"
                 "v_and_or_b32 %10, %7, %11, 0.5\n\tv_add_f32 %7, %7, %10\n\t"
                 "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0\n\t"
                 "v_cvt_i32_f32_sdwa %8, %0 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %9, %4 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %8, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %9, %5 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %8, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %9, %6 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %8, %3 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %9, %7 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 1"
                 : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3]), "+v"(c[4]), "+v"(c[5]), "+v"(c[6]), "+v"(c[7]), "=&v"(w0), "=&v"(w1), "=&v"(t)
                 : "s"(0x80000000u));
}
__device__ __forceinline__ void round_pack_1x4(float (&c)[4], uint32_t& w0)
{
    float t;
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
                 "v_and_or_b32 %5, %0, %6, 0.5\n\tv_add_f32 %0, %0, %5\n\t"
                 "v_and_or_b32 %5, %1, %6, 0.5\n\tv_add_f32 %1, %1, %5\n\t"
                 "v_and_or_b32 %5, %2, %6, 0.5\n\tv_add_f32 %2, %2, %5\n\t"
                 "v_and_or_b32 %5, %3, %6, 0.5\n\tv_add_f32 %3, %3, %5\n\t"
                 "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0\n\t"
                 "v_cvt_i32_f32_sdwa %4, %0 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_i32_f32_sdwa %4, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_i32_f32_sdwa %4, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_i32_f32_sdwa %4, %3 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 1"
                 : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3]), "=&v"(w0), "=&v"(t)
                 : "s"(0x80000000u));
}

// the five table rows of one group of four channels (input scale, bias, output scale, clamp bounds), and the wait that
// hands them over: PENDING later LDS reads may stay in flight
struct ChannelTables
{
    v4f si, bi, so, lo, hi;
};
template<int BN>
__device__ __forceinline__ void request_tables(ChannelTables& t, unsigned addr)
{
    lds_read128f(t.si, addr);
    lds_read128f(t.bi, addr + BN * 4);
    lds_read128f(t.so, addr + 2 * BN * 4);
    lds_read128f(t.lo, addr + 3 * BN * 4);
    lds_read128f(t.hi, addr + 4 * BN * 4);
}
template<int PENDING>
__device__ __forceinline__ void wait_tables(ChannelTables& t)
{
    asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(t.si), "+v"(t.bi), "+v"(t.so), "+v"(t.lo), "+v"(t.hi) : "n"(PENDING));
}

constexpr int RESIDENT_MAX_ROW_ITERS = 8; // wavefront loads per patch row (a lane keeps one column offset for each)

// OUT 0: requantised int8; 1: fp32 with the optional fused tail (residual, ReLU, quantised copy)
template<int TM, int TN, int WN, int OUT>
__global__ __launch_bounds__(256, 2) void conv_resident_kernel(const int8_t* __restrict__ wpk, const int8_t* __restrict__ x, ResidentPlan P, ConvEpilogue epi, ConvFusion fusion)
{
    constexpr int WM = 4 / WN;
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    extern __shared__ __attribute__((aligned(1024))) int8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, lhi = lane >> 5;
    const unsigned lds0 = (unsigned)(uintptr_t)(AS3 int8_t*)lds;
    const int8_t* zero = g_resident_zero_line;

    // ---- which channel block, which pixel tiles.  Workgroup ids are dealt round-robin to the 8 XCDs: remapped so that
    // an XCD works on neighbouring tiles (they share border rows of the input, and all channel blocks of a tile its
    // pixels, in that XCD's L2)
    int b = blockIdx.x;
    {
        const int T = gridDim.x, xcd = b & 7, idx = b >> 3, rem = T & 7;
        b = xcd * (T >> 3) + (xcd < rem ? xcd : rem) + idx;
    }
    const int grp = (int)mdiv((unsigned)b, P.magic_ncg);
    const int cg = b - grp * P.n_cg;
    const int col0 = cg * BN;
    const int ppitch = P.n5 * 16, wpitch = P.nw * 16;

    // ---- the epilogue's per-channel tables are requested first (bare loads from clamped indices: nothing looks at the
    // values before the first tile's operands have landed, so their latency costs nothing)
    const bool to_int8 = OUT == 0;
    float raw_si = 0.f, raw_bi = 0.f, raw_so = 0.f;
    {
        int ch = col0 + (tid < BN ? tid : 0);
        if (ch >= P.cout) ch = P.cout - 1;
        raw_si = epi.scale_in[ch];
        raw_bi = (epi.bias ? epi.bias : epi.scale_in)[ch];
        raw_so = (to_int8 ? epi.scale_out : epi.scale_in)[ch];
    }

    // ---- what a lane needs to know about the patch never changes from tile to tile
    // kernels with taps: load j of a patch row covers slots j*64 + lane of that row; the lane's column, its byte offset
    // from the start of the image row, and whether it is an image column at all (border columns are never written)
    unsigned col_off[RESIDENT_MAX_ROW_ITERS];
    unsigned col_ok = 0; // bit j
    // the lane's pixels of a tile: row inside the tile and (virtual) column
    int pix_r[TM], pix_ox[TM];
    bool pix_in[TM];
    {
#pragma unroll
        for (int j = 0; j < RESIDENT_MAX_ROW_ITERS; j++)
        {
            const unsigned s = (unsigned)(j * 64 + lane);
            const unsigned px = mdiv(s, P.magic_n5);
            const int chunk = (int)(s - px * (unsigned)P.n5);
            const int ix = (int)px - P.pad_left;
            const bool ok = j < P.row_iters && (int)s < P.row_slots && chunk < P.data_chunks_a && (unsigned)ix < (unsigned)P.W;
            col_off[j] = ok ? (unsigned)(ix * P.Cp + chunk * 16) : 0u;
            col_ok |= ok ? 1u << j : 0u;
        }
#pragma unroll
        for (int a = 0; a < TM; a++)
        {
            const int j = (wm * TM + a) * 32 + l32;
            const int r = (int)mdiv((unsigned)j, P.magic_outw);
            pix_in[a] = r < P.R;
            pix_r[a] = pix_in[a] ? r : 0;
            pix_ox[a] = pix_in[a] ? j - r * P.outw : 0;
        }
        // border columns of both patch buffers are cleared once: the fetches never write them
        const int border = P.Wp - P.W;
        const int cells = P.rows_cap * border * (P.lds_patch1 != P.lds_patch0 ? 2 : 1);
        for (int c = tid; c < cells; c += 256)
        {
            const int row = c / border, k = c - row * border;
            const int bufsel = row >= P.rows_cap ? 1 : 0;
            const int rr = row - bufsel * P.rows_cap;
            const int px = k < P.pad_left ? k : P.W + k; // left border, then right border
            int8_t* dst = lds + (bufsel ? P.lds_patch1 : P.lds_patch0) + (rr * P.Wp + px) * ppitch;
            for (int q = 0; q < P.n5; q++) *reinterpret_cast<v4i*>(dst + q * 16) = v4i{0, 0, 0, 0};
        }
    }

    // virtual row of output row g (rows counted over the stack of images)
    auto virtual_row = [&](int g) -> int {
        const int img = (int)mdiv((unsigned)g, P.magic_outh);
        return img * P.Hp + (g - img * P.outh) * P.sh;
    };

    // ---- requests a tile's patch into LDS at byte offset dst; returns the first virtual row it holds
    auto fill_patch = [&](int tile, int dst) -> int {
        const int g0 = tile * P.R;
        int g1 = g0 + P.R - 1;
        if (g1 >= P.total_rows) g1 = P.total_rows - 1;
        const int v0 = virtual_row(g0);
        int nrows = virtual_row(g1) + (P.kh - 1) * P.dh - v0 + 1;
        if (nrows > P.rows_cap) nrows = P.rows_cap; // (the launch sized the buffer for the tallest tile)
        for (int k = wave; k < nrows; k += 4)
        {
            const int v = v0 + k;
            const int img = (int)mdiv((unsigned)v, P.magic_hp);
            const int iy = v - img * P.Hp - P.pad_top;
            const bool row_ok = (unsigned)iy < (unsigned)P.H && img < P.batch; // else a border row: zeros
            const int8_t* base = row_ok ? x + (size_t)(img * P.H + iy) * P.W * P.Cp : zero;
            int8_t* row_lds = lds + dst + k * (P.row_slots * 16);
#pragma unroll
            for (int j = 0; j < RESIDENT_MAX_ROW_ITERS; j++)
            {
                if (j < P.row_iters && ((col_ok >> j) & 1u))
                {
                    const unsigned off = row_ok ? col_off[j] : (unsigned)((lane & 3) * 16);
                    __builtin_amdgcn_global_load_lds((const AS1 void*)(base + off), (AS3 void*)(row_lds + j * 1024), 16, 0, 0);
                }
            }
        }
        return v0;
    };

    // ---- the first tile's patch (nobody else has asked for these lines: they come from furthest away), then the
    // weights of this channel block: every K byte of BN rows, requested once
    int tile = grp;
    {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier(); // the cleared border columns are in place before any fetch lands next to them
        asm volatile("" ::: "memory");
    }
    int v0 = fill_patch(tile, P.lds_patch0);
    {
        const int iters = (P.w_slots + 255) >> 8;
        for (int it = 0; it < iters; it++)
        {
            const unsigned q = (unsigned)(it * 256 + tid);
            const unsigned row = mdiv(q, P.magic_nw);
            const int chunk = (int)(q - row * (unsigned)P.nw);
            int ch = col0 + (int)row;
            if (ch >= P.cout) ch = P.cout - 1; // a valid row; its products land in channels whose tables are zero
            const int8_t* src = chunk < P.data_chunks_w ? wpk + (size_t)ch * P.Ktot + chunk * 16 : zero;
            if ((int)q < P.w_slots) __builtin_amdgcn_global_load_lds((const AS1 void*)src, (AS3 void*)(lds + P.lds_w + (it * 4 + wave) * 1024), 16, 0, 0);
        }
    }

    // ---- everything this wavefront asked for has landed.  Tables into LDS: input scale, bias, output scale and the
    // requantising clamp [lo, hi] that also holds a ReLU or a clip when that is provably the same value (see below)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    bool tame = true, nonneg = true;
    if (tid < BN)
    {
        const bool real = col0 + tid < P.cout;
        const float si = real ? raw_si : 0.f;
        const float bi = (real && epi.bias) ? raw_bi : -0.f; // x + -0 = x for every x
        const float so = (real && to_int8) ? raw_so : 0.f;
        float lo = -127.f, hi = 127.f;
        // Finite tables keep every value finite; an output scale that is not negative makes x -> RN(x * s) monotonic, so
        // it commutes with the max of a ReLU and the min / max of a clip, and nested clamps are one clamp; a product
        // that stays below 2^31 never takes float2int8's out-of-range answer.
        bool ok = fabsf(si) < 0x1p90f && fabsf(bi) < 0x1p120f && so >= 0.f && so < INFINITY;
        if (epi.act.type == 3)
        {
            const float clip_abs = fmaxf(fabsf(epi.act.p0), fabsf(epi.act.p1));
            ok = ok && fabsf(epi.act.p0) < INFINITY && fabsf(epi.act.p1) < INFINITY && epi.act.p0 <= epi.act.p1 && mul_rn(clip_abs, so) < 2147483648.f;
            lo = __builtin_amdgcn_fmed3f(mul_rn(epi.act.p0, so), -127.f, 127.f);
            hi = __builtin_amdgcn_fmed3f(mul_rn(epi.act.p1, so), -127.f, 127.f);
        }
        else
        {
            // |acc| <= 2^31
            ok = ok && mul_rn(add_rn(mul_rn(2147483648.f, fabsf(si)), fabsf(bi)), so) < 1073741824.f;
            if (epi.act.type == 1) lo = 0.f;
        }
        tame = ok;
        nonneg = lo >= 0.f; // a clamp without a negative bound: the rounding is one conversion (pack8_nonneg / pack4_nonneg)
        float* tab = reinterpret_cast<float*>(lds + P.lds_tab);
        tab[tid] = si;
        tab[BN + tid] = bi;
        tab[2 * BN + tid] = so;
        tab[3 * BN + tid] = lo;
        tab[4 * BN + tid] = hi;
    }
    {
        const int failed = __syncthreads_or((tame ? 0 : 1) | (nonneg ? 0 : 2)); // (also: everybody's share of the operands and the tables are in LDS)
        tame = !(failed & 1);
        nonneg = tame && !(failed & 2);
    }

    // ---- fragment addresses that do not depend on the tile
    unsigned w_base[TN];
#pragma unroll
    for (int c = 0; c < TN; c++) w_base[c] = lds0 + (unsigned)(P.lds_w + ((wn * TN + c) * 32 + l32) * wpitch + lhi * 16);
    const unsigned tab_base = lds0 + (unsigned)(P.lds_tab + (wn * TN * 32 + 4 * lhi) * 4);
    const int halves = P.ntaps * P.nh;
    const bool dbuf = P.lds_patch1 != P.lds_patch0;

    int buf = 0;
    for (;; tile += P.groups)
    {
        const int patch_off = buf ? P.lds_patch1 : P.lds_patch0;
        const int next = tile + P.groups;
        int v0_next = 0;
        if (dbuf && next < P.tiles) v0_next = fill_patch(next, buf ? P.lds_patch0 : P.lds_patch1);

        // this lane's pixels: where their first tap lies in the patch, and which output pixel they are (npix: none)
        unsigned a_base[TM];
        int p_out[TM];
        bool full;
        {
            const int g0 = tile * P.R;
#pragma unroll
            for (int a = 0; a < TM; a++)
            {
                int g = g0 + pix_r[a];
                const bool in = pix_in[a] && g < P.total_rows;
                if (g >= P.total_rows) g = g0; // a valid row; nothing of it is stored
                const int vr = virtual_row(g) - v0;
                a_base[a] = lds0 + (unsigned)(patch_off + (vr * P.Wp + pix_ox[a] * P.sw) * ppitch + lhi * 16);
                p_out[a] = in ? g * P.outw + pix_ox[a] : P.npix;
            }
            full = P.R * P.outw == BM && g0 + P.R <= P.total_rows;
        }

        v16i acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
            for (int c = 0; c < TN; c++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[a][c][r] = 0;

        // ---- K loop: 32 bytes of K per piece, three pieces per trip, the fragments of the next two pieces requested
        // before the products of this one.  The body is straight-line code (scalar arithmetic decides how far the pixel fragments
        // move: 32 bytes inside a tap, to the next tap's offset at its end): fragments that are still on their way from
        // LDS must not meet a branch, where the compiler would be free to copy their registers.  The last trips request
        // pieces that do not exist (addresses at or beyond the end of the operands, never multiplied), so that every
        // trip is the same; what is left of the pieces after the last whole trip is multiplied behind the loop.
        {
            unsigned a_cur[TM], w_cur[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) a_cur[a] = a_base[a];
#pragma unroll
            for (int c = 0; c < TN; c++) w_cur[c] = w_base[c];
            // how far the pixel fragments move from one piece to the next: 32 bytes inside a tap, to the next tap of
            // the kernel row at its end, to the first tap of the next kernel row at the end of a row (two counters)
            const int step_tap = P.dw * ppitch - (P.nh - 1) * 32;
            const int step_row = (P.dh * P.Wp - (P.kw - 1) * P.dw) * ppitch - (P.nh - 1) * 32;
            int h_left = P.nh, kx_left = P.kw;
            auto advance = [&]() {
                int delta = 32;
                if (--h_left == 0)
                {
                    h_left = P.nh;
                    delta = step_tap;
                    if (--kx_left == 0)
                    {
                        kx_left = P.kw;
                        delta = step_row;
                    }
                }
#pragma unroll
                for (int a = 0; a < TM; a++) a_cur[a] += (unsigned)delta;
#pragma unroll
                for (int c = 0; c < TN; c++) w_cur[c] += 32;
            };
            v4i fa0[TM], fw0[TN], fa1[TM], fw1[TN], fa2[TM], fw2[TN];
            auto request = [&](v4i (&fa)[TM], v4i (&fw)[TN]) {
#pragma unroll
                for (int a = 0; a < TM; a++) lds_read128(fa[a], a_cur[a]);
#pragma unroll
                for (int c = 0; c < TN; c++) lds_read128(fw[c], w_cur[c]);
            };
            auto multiply = [&](v4i (&fa)[TM], v4i (&fw)[TN]) {
#pragma unroll
                for (int a = 0; a < TM; a++)
#pragma unroll
                    for (int c = 0; c < TN; c++) acc[a][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[c], fa[a], acc[a][c], 0, 0, 0);
            };
            // three fragment sets: the reads of pieces i + 1 and i + 2 are in flight while piece i is multiplied (one
            // wavefront per SIMD has nobody else to cover an LDS round trip, which costs about two pieces' products)
            constexpr int F = TM + TN;
            int left = halves;
            request(fa0, fw0);
            advance();
            request(fa1, fw1);
            for (; left >= 3; left -= 3)
            {
                advance();
                request(fa2, fw2);
                wait_fragments<2 * F>(fa0, fw0); // LDS answers in order: with two later pieces' reads behind them, this piece's are done
                multiply(fa0, fw0);
                advance();
                request(fa0, fw0);
                wait_fragments<2 * F>(fa1, fw1);
                multiply(fa1, fw1);
                advance();
                request(fa1, fw1);
                wait_fragments<2 * F>(fa2, fw2);
                multiply(fa2, fw2);
            }
            // the two sets on their way hold the next two pieces (or addresses past the end, never multiplied)
            wait_fragments<0>(fa0, fw0);
            wait_fragments<0>(fa1, fw1);
            if (left >= 1) multiply(fa0, fw0);
            if (left == 2) multiply(fa1, fw1);
        }

        if (!dbuf && next < P.tiles)
        {
            // one patch buffer: everybody has finished reading it; the next tile's patch travels during the epilogue
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            v0_next = fill_patch(next, P.lds_patch0);
        }

        // ---- epilogue, registers -> global memory.  Register r of block (a, c): pixel l32 of pixel block a, channel
        // c*32 + 8*(r/4) + 4*lhi + r%4 of the wavefront's channels.
        const int ch_wave = col0 + wn * TN * 32;
        if (OUT == 0)
        {
            int8_t* out = static_cast<int8_t*>(epi.out);
            auto finish = [&](auto tame_tag, auto act_tag) {
                constexpr bool TAME = decltype(tame_tag)::value;
                constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
                for (int c = 0; c < TN; c++)
                {
                    uint32_t word[TM][4];
#pragma unroll
                    for (int g = 0; g < 4; g++)
                    {
                        v4f si, bi, so, lo, hi;
                        const unsigned ta = tab_base + (unsigned)((c * 32 + 8 * g) * 4);
                        lds_read128f(si, ta);
                        lds_read128f(bi, ta + BN * 4);
                        lds_read128f(so, ta + 2 * BN * 4);
                        if (TAME)
                        {
                            lds_read128f(lo, ta + 3 * BN * 4);
                            lds_read128f(hi, ta + 4 * BN * 4);
                        }
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        asm volatile("" : "+v"(si), "+v"(bi), "+v"(so));
                        if (TAME) asm volatile("" : "+v"(lo), "+v"(hi));
#pragma unroll
                        for (int a = 0; a < TM; a++)
                        {
                            float f[4];
#pragma unroll
                            for (int e = 0; e < 4; e++)
                            {
                                float v = add_rn(mul_rn((float)acc[a][c][4 * g + e], si[e]), bi[e]);
                                if (!TAME)
                                {
                                    if (ACT == 1)
                                        v = fmaxf(v, 0.f);
                                    else if (ACT == 3)
                                    {
                                        if (v < epi.act.p0) v = epi.act.p0;
                                        if (v > epi.act.p1) v = epi.act.p1;
                                    }
                                }
                                f[e] = mul_rn(v, so[e]);
                            }
                            if (TAME)
                            {
                                const float los[4] = {lo[0], lo[1], lo[2], lo[3]}, his[4] = {hi[0], hi[1], hi[2], hi[3]};
                                float2int8_as_float_bounded_lanes_x4(f[0], f[1], f[2], f[3], los, his);
                            }
                            else
                                float2int8_as_float_x4(f[0], f[1], f[2], f[3]);
                            word[a][g] = pack4_quantised(f[0], f[1], f[2], f[3]);
                        }
                    }
                    // lanes l and l + 32 hold the two halves of every 8-channel run of one pixel: after the swaps the
                    // lower lane has channels 0..15 of the 32-channel block, the upper one 16..31, as 16 consecutive bytes
                    asm volatile("s_nop 1"); // a lane-half swap right behind a sub-dword write needs two wait states
#pragma unroll
                    for (int a = 0; a < TM; a++)
                    {
                        const auto s02 = __builtin_amdgcn_permlane32_swap(word[a][0], word[a][2], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(word[a][1], word[a][3], false, false);
                        const v4i pk = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
                        const int p = p_out[a];
                        const int ch = ch_wave + c * 32 + lhi * 16;
                        if (p < P.npix && ch < P.out_cp) *reinterpret_cast<v4i*>(out + (size_t)p * P.out_cp + ch) = pk;
                    }
                }
            };
            if (tame)
            {
                // The common case, trimmed: the tables of the next group of four channels are requested before the
                // arithmetic of this one, and all of a group's values (four channels of TM pixels) are rounded under one
                // switch of the rounding mode.
                constexpr int NG = TN * 4;
                uint32_t word[TM][NG];
                ChannelTables tab0, tab1;
                request_tables<BN>(tab0, tab_base);
#pragma unroll
                for (int idx = 0; idx < NG; idx++)
                {
                    ChannelTables& cur = (idx & 1) ? tab1 : tab0;
                    ChannelTables& nxt = (idx & 1) ? tab0 : tab1;
                    const int c = idx >> 2, g = idx & 3;
                    if (idx + 1 < NG)
                    {
                        request_tables<BN>(nxt, tab_base + (unsigned)((((idx + 1) >> 2) * 32 + 8 * ((idx + 1) & 3)) * 4));
                        wait_tables<5>(cur);
                    }
                    else
                        wait_tables<0>(cur);
                    float v[TM * 4];
#pragma unroll
                    for (int a = 0; a < TM; a++)
#pragma unroll
                        for (int e = 0; e < 4; e++)
                        {
                            const float f = mul_rn(add_rn(mul_rn((float)acc[a][c][4 * g + e], cur.si[e]), cur.bi[e]), cur.so[e]);
                            v[a * 4 + e] = __builtin_amdgcn_fmed3f(f, cur.lo[e], cur.hi[e]);
                        }
                    if (nonneg)
                    {
                        if constexpr (TM == 2)
                            pack8_nonneg(v, word[0][idx], word[1][idx]);
                        else
                            word[0][idx] = pack4_nonneg(v[0], v[1], v[2], v[3]);
                    }
                    else if constexpr (TM == 2)
                        round_pack_2x4(v, word[0][idx], word[1][idx]);
                    else
                        round_pack_1x4(v, word[0][idx]);
                }
#pragma unroll
                for (int c = 0; c < TN; c++)
#pragma unroll
                    for (int a = 0; a < TM; a++)
                    {
                        const auto s02 = __builtin_amdgcn_permlane32_swap(word[a][c * 4], word[a][c * 4 + 2], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(word[a][c * 4 + 1], word[a][c * 4 + 3], false, false);
                        const v4i pk = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
                        const int p = p_out[a];
                        const int ch = ch_wave + c * 32 + lhi * 16;
                        if (p < P.npix && ch < P.out_cp) *reinterpret_cast<v4i*>(out + (size_t)p * P.out_cp + ch) = pk;
                    }
            }
            else if (epi.act.type == 1)
                finish(std::false_type{}, std::integral_constant<int, 1>{});
            else if (epi.act.type == 3)
                finish(std::false_type{}, std::integral_constant<int, 3>{});
            else
                finish(std::false_type{}, std::integral_constant<int, 0>{});
        }
        else
        {
            float* out = static_cast<float*>(epi.out);
            const bool with_residual = fusion.residual != 0;
#pragma unroll
            for (int c = 0; c < TN; c++)
            {
                uint32_t word[TM][4];
                // the residual of the whole 32-channel block first, all loads in flight together (clamped addresses,
                // nothing selected until the values are used)
                v4f res[TM][4];
                if (with_residual)
                {
#pragma unroll
                    for (int a = 0; a < TM; a++)
#pragma unroll
                        for (int g = 0; g < 4; g++)
                        {
                            int p = p_out[a];
                            int ch = ch_wave + c * 32 + 8 * g + 4 * lhi;
                            if (p >= P.npix) p = P.npix - 1;
                            if (ch >= P.out_cp) ch = P.out_cp - 4;
                            res[a][g] = *reinterpret_cast<const v4f*>(fusion.residual + (size_t)p * P.out_cp + ch);
                        }
                }
#pragma unroll
                for (int g = 0; g < 4; g++)
                {
                    v4f si, bi;
                    const unsigned ta = tab_base + (unsigned)((c * 32 + 8 * g) * 4);
                    lds_read128f(si, ta);
                    lds_read128f(bi, ta + BN * 4);
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    asm volatile("" : "+v"(si), "+v"(bi));
#pragma unroll
                    for (int a = 0; a < TM; a++)
                    {
                        v4f v;
#pragma unroll
                        for (int e = 0; e < 4; e++)
                        {
                            float t = add_rn(mul_rn((float)acc[a][c][4 * g + e], si[e]), bi[e]);
                            if (epi.act.type == 1)
                                t = fmaxf(t, 0.f);
                            else if (epi.act.type == 3)
                            {
                                if (t < epi.act.p0) t = epi.act.p0;
                                if (t > epi.act.p1) t = epi.act.p1;
                            }
                            if (with_residual) t = add_rn(t, res[a][g][e]);
                            if (fusion.relu_after) t = t < 0.f ? 0.f : t; // the ReLU LAYER's statement (src/layer/relu.cpp:36-37): a NaN stays
                            v[e] = t;
                        }
                        const int p = p_out[a];
                        const int ch = ch_wave + c * 32 + 8 * g + 4 * lhi;
                        if (p < P.npix && ch < P.out_cp) *reinterpret_cast<v4f*>(out + (size_t)p * P.out_cp + ch) = v;
                        if (fusion.q8_out)
                        {
                            float q0 = mul_rn(v[0], fusion.q8_scale), q1 = mul_rn(v[1], fusion.q8_scale), q2 = mul_rn(v[2], fusion.q8_scale), q3 = mul_rn(v[3], fusion.q8_scale);
                            float2int8_as_float_x4(q0, q1, q2, q3);
                            word[a][g] = pack4_quantised(q0, q1, q2, q3);
                        }
                    }
                }
                if (fusion.q8_out)
                {
                    asm volatile("s_nop 1"); // a lane-half swap right behind a sub-dword write needs two wait states
#pragma unroll
                    for (int a = 0; a < TM; a++)
                    {
                        const auto s02 = __builtin_amdgcn_permlane32_swap(word[a][0], word[a][2], false, false);
                        const auto s13 = __builtin_amdgcn_permlane32_swap(word[a][1], word[a][3], false, false);
                        const v4i pk = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
                        const int p = p_out[a];
                        const int ch = ch_wave + c * 32 + lhi * 16;
                        if (p < P.npix && ch < P.out_cp) *reinterpret_cast<v4i*>(fusion.q8_out + (size_t)p * P.out_cp + ch) = pk;
                    }
                }
            }
        }
        if (next >= P.tiles) break;
        // The next tile's patch has landed -- this wavefront's share, then everybody's (the barrier also says that nobody
        // still reads the patch buffer refilled next).  Memory instructions complete in the order they were issued and
        // the patch was requested before this tile's stores, so those may stay in flight: a full tile issues STORES of
        // them per wavefront (a ragged one may issue fewer, and waits for everything).
        constexpr int STORES = OUT == 0 ? TM * TN : TM * TN * 5;
        if (full && col0 + BN <= P.out_cp && (OUT == 0 || fusion.q8_out))
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(STORES) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        v0 = v0_next;
        if (dbuf) buf ^= 1;
    }
}

static inline unsigned magic_of(unsigned d)
{
    return d > 1 ? (unsigned)((1ull << 32) / d + 1) : 0u; // d == 1 is special-cased by the callers that can meet it
}

struct ResidentConfig
{
    int tm, tn, wn;
};

static const size_t RESIDENT_LDS_LIMIT = (160u << 10) - 1024; // dynamic LDS a workgroup may ask for (the kernel holds 1 KiB statically)

// fills the plan for one tile configuration; false when the layer does not fit it
static bool resident_plan_for(const NhwcGeom& g, const ConvEpilogue& epi, int out_cp, const ResidentConfig& cfg, ResidentPlan& P, size_t& lds_bytes)
{
    const int wm = 4 / cfg.wn;
    const int BM = wm * cfg.tm * 32, BN = cfg.wn * cfg.tn * 32;
    P.H = g.H, P.W = g.W, P.Cp = g.Cp, P.kw = g.kw, P.kh = g.kh, P.dw = g.dw, P.dh = g.dh, P.sw = g.sw, P.sh = g.sh;
    P.pad_top = g.pad_top, P.pad_left = g.pad_left, P.outw = g.outw, P.outh = g.outh, P.npix = g.npix, P.batch = epi.batch;
    P.cout = g.cout, P.out_cp = out_cp, P.Ktot = g.K, P.ntaps = g.ntaps;
    P.plane = g.outw * g.outh;
    P.total_rows = epi.batch * g.outh;
    if (g.ntaps > 1 && g.Cp % 64 != 0) return false; // a tap's bytes are whole 32-byte pieces, and rows of taps are contiguous
    P.nh = (g.Cp + 31) / 32;
    P.data_chunks_a = g.Cp / 16;
    P.n5 = P.nh * 2 + 1;
    const int row_bytes = g.ntaps > 1 ? g.ntaps * g.Cp : P.nh * 32;
    if (row_bytes > g.K) return false;
    P.data_chunks_w = row_bytes / 16;
    P.nw = P.data_chunks_w + 1;
    P.w_slots = BN * P.nw;
    // the virtual padded image: every tap of every output pixel lies inside it
    P.Hp = std::max(g.H + g.pad_top, (g.outh - 1) * g.sh + (g.kh - 1) * g.dh + 1);
    P.Wp = std::max(g.W + g.pad_left, (g.outw - 1) * g.sw + (g.kw - 1) * g.dw + 1);
    size_t patch_bytes;
    int patch_loads; // per wavefront
    {
        P.R = std::min(BM / g.outw, P.total_rows);
        if (P.R < 1) return false; // an output row is wider than a tile
        P.tiles = ceil_div(P.total_rows, P.R);
        // rows of the stack R consecutive output rows can span: a tile that runs into the next image also holds the
        // rows between the two (tiles that divide an image never do)
        const int crossings = g.outh % P.R == 0 ? 0 : (P.R - 1 + g.outh - 1) / g.outh;
        P.rows_cap = (P.R - 1) * g.sh + crossings * std::max(0, P.Hp - g.outh * g.sh) + (g.kh - 1) * g.dh + 1;
        P.row_slots = P.Wp * P.n5;
        P.row_iters = ceil_div(P.row_slots, 64);
        if (P.row_iters > RESIDENT_MAX_ROW_ITERS) return false;
        patch_bytes = (size_t)P.rows_cap * P.row_slots * 16;
        patch_loads = ceil_div(P.rows_cap, 4) * P.row_iters;
    }
    if (ceil_div(P.w_slots, 256) + patch_loads + 3 > 60) return false; // loads in flight per wavefront before the first tile (the counter holds 63)
    const size_t tab_bytes = 5 * BN * 4;
    P.n_cg = ceil_div(out_cp, BN);
    P.lds_tab = 0;
    P.lds_w = (int)((tab_bytes + 255) & ~(size_t)255);
    P.lds_patch0 = P.lds_w + (int)(((size_t)P.w_slots * 16 + 255) & ~(size_t)255);
    patch_bytes = (patch_bytes + 255) & ~(size_t)255;
    const size_t one = (size_t)P.lds_patch0 + patch_bytes;
    if (one > RESIDENT_LDS_LIMIT) return false;
    // as many workgroups as the chip holds at once (two per compute unit where LDS allows); a workgroup that walks
    // several tiles gets a second patch buffer when that fits
    auto places = [&](size_t bytes) { return 256 * (int)std::min<size_t>(2, (RESIDENT_LDS_LIMIT + 1024) / (bytes + 1024)); };
    const int jobs_cg = std::max(1, places(one) / P.n_cg);
    const bool two = P.tiles > jobs_cg && places(one + patch_bytes) == places(one);
    lds_bytes = two ? one + patch_bytes : one;
    P.groups = std::min(P.tiles, std::max(1, places(lds_bytes) / P.n_cg));
    P.lds_patch1 = two ? P.lds_patch0 + (int)patch_bytes : P.lds_patch0;
    // divisions by multiplication: exact while dividend * divisor < 2^32
    const long long vrows = (long long)(epi.batch + 1) * P.Hp + P.rows_cap;
    if (vrows * P.Hp >= (1ll << 32) || ((long long)g.npix + BM) * P.plane >= (1ll << 32) || (long long)(P.total_rows + P.R) * g.outh >= (1ll << 32) ||
        (256ll + 64 * RESIDENT_MAX_ROW_ITERS) * P.n5 >= (1ll << 32) || ((long long)P.w_slots + 256) * P.nw >= (1ll << 32) ||
        (long long)P.groups * P.n_cg * P.n_cg >= (1ll << 32) || (long long)BM * g.outw >= (1ll << 32))
        return false;
    if ((long long)g.W * g.Cp >= (1ll << 31)) return false; // a lane's offset inside an image row is formed in 32 bits
    P.magic_n5 = magic_of((unsigned)P.n5);
    P.magic_nw = magic_of((unsigned)P.nw);
    P.magic_hp = magic_of((unsigned)P.Hp);
    P.magic_outw = magic_of((unsigned)P.outw);
    P.magic_outh = magic_of((unsigned)P.outh);
    P.magic_plane = magic_of((unsigned)P.plane);
    P.magic_ncg = magic_of((unsigned)P.n_cg);
    return true;
}

typedef void (*ResidentKernel)(const int8_t*, const int8_t*, ResidentPlan, ConvEpilogue, ConvFusion);

template<int TM, int TN, int WN>
static ResidentKernel resident_kernel_for(int out)
{
    return out == 0 ? conv_resident_kernel<TM, TN, WN, 0> : conv_resident_kernel<TM, TN, WN, 1>;
}

// tile configurations: {pixel blocks per wavefront, channel blocks per wavefront, wavefronts along the channels}
static const ResidentConfig RESIDENT_CONFIGS[] = {{2, 2, 1}, {1, 2, 1}, {2, 1, 1}, {1, 1, 1}, {1, 1, 2}, {2, 1, 2}, {1, 2, 2}, {2, 2, 2}};
constexpr int RESIDENT_NCONFIGS = sizeof(RESIDENT_CONFIGS) / sizeof(RESIDENT_CONFIGS[0]);

static ResidentKernel resident_kernel(int cfg, int out)
{
    switch (cfg)
    {
    case 0: return resident_kernel_for<2, 2, 1>(out);
    case 1: return resident_kernel_for<1, 2, 1>(out);
    case 2: return resident_kernel_for<2, 1, 1>(out);
    case 3: return resident_kernel_for<1, 1, 1>(out);
    case 4: return resident_kernel_for<1, 1, 2>(out);
    case 5: return resident_kernel_for<2, 1, 2>(out);
    case 6: return resident_kernel_for<1, 2, 2>(out);
    default: return resident_kernel_for<2, 2, 2>(out);
    }
}

static bool resident_basics(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp)
{
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(epi.out) | reinterpret_cast<uintptr_t>(fusion.residual) | reinterpret_cast<uintptr_t>(fusion.q8_out);
    const bool act_ok = epi.act.type == 0 || epi.act.type == 1 || epi.act.type == 3;
    const bool plain = !fusion.residual && !fusion.relu_after && !fusion.q8_out;
    return g.pad_word == 0 && g.tapK == g.Cp && g.Cp % 16 == 0 && out_cp % 16 == 0 && (ptrs & 15) == 0 && act_ok && !epi.acc_out && (!epi.scale_out || plain);
}

// The configuration this layer runs with, or -1: the estimate below prices each one that fits and keeps the cheapest.
static int resident_choose(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp, ResidentPlan& best_plan, size_t& best_lds)
{
    if (!resident_basics(g, epi, fusion, out_cp)) return -1;
    int forced = -1;
    if (const char* e = getenv("NCNNHIP_RESIDENT_CFG")) forced = atoi(e);
    int best = -1;
    double best_cost = 0;
    for (int i = 0; i < RESIDENT_NCONFIGS; i++)
    {
        if (forced >= 0 && i != forced) continue;
        ResidentPlan P;
        size_t lds_bytes;
        if (!resident_plan_for(g, epi, out_cp, RESIDENT_CONFIGS[i], P, lds_bytes)) continue;
        const ResidentConfig& c = RESIDENT_CONFIGS[i];
        // Cycles of the busiest compute unit.  A wavefront's tile costs matrix-core time (its blocks x K pieces x 32) and
        // vector time (the epilogue's instructions for its 16 outputs per block and lane, patch addresses); two workgroups
        // on a compute unit overlap the two, one alone runs them one after the other.  In front of that, the bytes the
        // unit has to fetch before its first product.
        const int halves = P.ntaps * P.nh;
        const double mfma = (double)c.tm * c.tn * halves * 32, valu = (double)c.tm * c.tn * 16 * 36 + 400;
        const double rounds = (double)ceil_div(P.tiles, P.groups);
        const int per_cu = ceil_div(P.groups * P.n_cg, 256);
        const double tile = per_cu >= 2 ? 1.2 * per_cu * std::max(mfma, valu) : mfma + valu;
        const double prologue = 0.5 * (double)(P.w_slots + P.rows_cap * P.row_slots) * per_cu;
        const double cost = rounds * tile + prologue;
        if (best < 0 || cost < best_cost)
        {
            best = i;
            best_cost = cost;
            best_plan = P;
            best_lds = lds_bytes;
        }
    }
    return best;
}

// Which layers take this kernel: kernels with taps (a 1x1 layer reads nothing twice and is bound by HBM or by its epilogue
// either way: measured no faster here) from 40000 output pixels up.  Launched alone, the kernel is as fast or faster than the
// pipelined kernel from 1536 pixels up (the 3x3 layers of a ResNet-50 at batch 16 to 128: 56 x 56 maps 8 to 25 % faster,
// 28 x 28 4 to 7 %, 14 x 14 15 % at batch 16 and 2 to 4 % slower beyond).  Inside a whole pass, where launches follow one
// another without a gap, the long-lived workgroups of the smaller layers hold their CUs' LDS until the last tile is done and
// the next launch starts later than behind the pipelined kernel's short ones: with every 3x3 layer on this kernel a ResNet-50
// pass is 2 % slower at batch 32 and 1 % at batch 128 (equal at batch 16); from 40000 pixels up (the 56 x 56 maps from batch
// 16, the 28 x 28 maps from batch 64) the passes are as fast as without it and those layers are the ones that gain most alone.
// Environment, read at every launch: NCNNHIP_RESIDENT_OFF (any value) switches the kernel off, NCNNHIP_RESIDENT_MIN sets
// the pixel threshold, NCNNHIP_RESIDENT_CFG forces one tile configuration (0..7): for measurements and tests.
bool conv_resident_fits(const NhwcGeom& g, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp)
{
    if (g.ntaps < 2) return false; // first: most layers of a network are 1x1 and need not look the environment up
    if (getenv("NCNNHIP_RESIDENT_OFF")) return false;
    long long min_pixels = 40000;
    if (const char* e = getenv("NCNNHIP_RESIDENT_MIN")) min_pixels = atoll(e);
    if (g.npix < min_pixels) return false;
    ResidentPlan P;
    size_t lds_bytes;
    return resident_choose(g, epi, fusion, out_cp, P, lds_bytes) >= 0;
}

int launch_conv_resident(const NhwcGeom& g, const int8_t* wpk, const int8_t* x, const ConvEpilogue& epi, const ConvFusion& fusion, int out_cp, hipStream_t stream)
{
    NCNNHIP_REQUIRE(((reinterpret_cast<uintptr_t>(wpk) | reinterpret_cast<uintptr_t>(x)) & 15) == 0, "convolution: operands must be 16-byte aligned");
    ResidentPlan P;
    size_t lds_bytes = 0;
    const int cfg = resident_choose(g, epi, fusion, out_cp, P, lds_bytes);
    NCNNHIP_REQUIRE(cfg >= 0, "convolution: this layer does not fit the weights-resident kernel");
    const int out = epi.scale_out ? 0 : 1;
    ResidentKernel kernel = resident_kernel(cfg, out);
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once
    static std::mutex mtx;
    static bool allowed[RESIDENT_NCONFIGS][2];
    {
        std::lock_guard<std::mutex> lock(mtx);
        if (!allowed[cfg][out])
        {
            NCNNHIP_CHECK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RESIDENT_LDS_LIMIT));
            allowed[cfg][out] = true;
        }
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)(P.groups * P.n_cg)), dim3(256), lds_bytes, stream, wpk, x, P, epi, fusion);
    return launch_status("conv_resident_kernel");
}

} // namespace ncnnhip

