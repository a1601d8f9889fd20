// General-shape int8 x int8 -> int32 tile contraction on the gfx950 matrix cores.
//
// D[i][j] = sum_k A[i][k] * B[j][k], both operands K-contiguous ("NT" form), any M/N/K.
// One workgroup (256 threads = 4 wavefronts in a 2x2 arrangement) owns a BM x BN output tile and
// walks K in steps of 64 bytes.  Operand tiles are staged in LDS as [row][64 bytes] with an
// 80-byte row pitch: a 16-lane group of 128-bit LDS reads then touches 64 distinct banks.
// Each wavefront issues v_mfma_i32_32x32x32_i8: lane l supplies 16 consecutive K bytes of operand
// row (l % 32), K sub-range (l / 32) * 16; accumulator register r of lane l is output element
// (8*(r/4) + 4*(l/32) + r%4, l%32) of the 32x32 block.
//
// The operand sources and the epilogue are policy objects so that Gemm, InnerProduct and the
// implicit-GEMM convolution share this file.  This is the any-shape kernel; the large aligned
// Gemm has its own pipelined kernel in gemm_int8.hip.
#ifndef NCNNHIP_MFMA_TILE_H
#define NCNNHIP_MFMA_TILE_H

#include "common.h"

namespace ncnnhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int TILE_K = 64;
constexpr int LDS_PITCH = 80;

// ---- operand source: dense row-major int8 matrix [rows][K] -------------------------------
struct DenseOperand
{
    const int8_t* base;
    size_t stride;
    int rows;
    int K;
    int vec; // rows start 16-byte aligned and stride % 16 == 0

    template<int ROWS>
    __device__ __forceinline__ void prepare(int) {}

    // fills lds[ROWS][LDS_PITCH] with rows row0.. and K range k0..k0+63, zero beyond the matrix
    template<int ROWS>
    __device__ __forceinline__ void load_tile(int8_t* lds, int row0, int k0) const
    {
#pragma unroll
        for (int c = threadIdx.x; c < ROWS * 4; c += 256)
        {
            const int r = c >> 2;
            const int kc = (c & 3) * 16;
            const int gr = row0 + r;
            const int gk = k0 + kc;
            v4i v = {0, 0, 0, 0};
            if (gr < rows && gk < K)
            {
                const int8_t* p = base + (size_t)gr * stride + gk;
                if (vec && gk + 16 <= K)
                {
                    v = *reinterpret_cast<const v4i*>(p);
                }
                else
                {
                    const int nb = K - gk < 16 ? K - gk : 16;
                    int8_t tmp[16];
#pragma unroll
                    for (int i = 0; i < 16; i++) tmp[i] = i < nb ? p[i] : (int8_t)0;
                    v = *reinterpret_cast<v4i*>(tmp);
                }
            }
            *reinterpret_cast<v4i*>(lds + r * LDS_PITCH + kc) = v;
        }
    }
};

// ---- operand source: im2col view of an int8 activation blob ------------------------------
// Row n of the virtual matrix is output pixel n = (img*outh + oy)*outw + ox, column
// k = (q*kh + ky)*kw + kx of group `g` (channel g*cin_g + q).  Out-of-image taps read the border
// byte; rows/columns beyond the matrix read 0.
struct Im2colOperand
{
    const int8_t* x;
    size_t cstep, nstep;
    int w, h;
    int cin_g;
    int kw, kh, dw, dh, sw, sh;
    int pad_top, pad_left;
    int outw, outh;
    int npix; // batch*outh*outw
    int K;    // cin_g*kh*kw
    int group_channel0;
    int pad_byte;

    // per-thread constants for the pixel this thread gathers
    const int8_t* pix_base;
    int iy0, ix0;
    int pix_ok;

    template<int ROWS>
    __device__ __forceinline__ void prepare(int row0)
    {
        const int n = row0 + (threadIdx.x % ROWS);
        pix_ok = n < npix;
        const int nn = pix_ok ? n : 0;
        const int img = nn / (outw * outh);
        const int rem = nn - img * (outw * outh);
        const int oy = rem / outw;
        const int ox = rem - oy * outw;
        iy0 = oy * sh - pad_top;
        ix0 = ox * sw - pad_left;
        pix_base = x + (size_t)img * nstep + (size_t)group_channel0 * cstep;
    }

    // ktab[k] = {channel offset + tap offset, (dy << 16) | dx}, or dy = 0x7fff for k >= K
    __device__ __forceinline__ void fill_ktab(int2* ktab, int k0) const
    {
        if (threadIdx.x < TILE_K)
        {
            const int k = k0 + threadIdx.x;
            int2 e;
            if (k < K)
            {
                const int taps = kw * kh;
                const int q = k / taps;
                const int t = k - q * taps;
                const int ky = t / kw;
                const int kx = t - ky * kw;
                const int dy = ky * dh, dx = kx * dw;
                e.x = (int)(q * cstep) + dy * w + dx;
                e.y = (dy << 16) | dx;
            }
            else
            {
                e.x = 0;
                e.y = 0x7fff << 16;
            }
            ktab[threadIdx.x] = e;
        }
    }

    template<int ROWS>
    __device__ __forceinline__ void load_tile(int8_t* lds, const int2* ktab) const
    {
        constexpr int KSLOTS = 256 / ROWS; // threads sharing one pixel row
        const int r = threadIdx.x % ROWS;
        const int ks = threadIdx.x / ROWS;
        const int base_off = iy0 * w + ix0;
#pragma unroll 4
        for (int kk = ks; kk < TILE_K; kk += KSLOTS)
        {
            const int2 e = ktab[kk];
            const int dy = e.y >> 16, dx = e.y & 0xffff;
            int v = 0;
            if (pix_ok && dy != 0x7fff)
            {
                const int iy = iy0 + dy, ix = ix0 + dx;
                v = ((unsigned)iy < (unsigned)h && (unsigned)ix < (unsigned)w) ? (int)pix_base[base_off + e.x] : pad_byte;
            }
            lds[r * LDS_PITCH + kk] = (int8_t)v;
        }
    }
};

// ---- the tile kernel body ----------------------------------------------------------------
// SrcA::load_tile<BM>(lds, row0, k0); SrcB is either DenseOperand or Im2colOperand.
template<int BM, int BN, typename SrcB, typename Epilogue>
__device__ __forceinline__ void mfma_tile_body(DenseOperand srcA, SrcB srcB, Epilogue epi, int M, int N, int K, int row0, int col0)
{
    constexpr int TM = BM / 64;
    constexpr int TN = BN / 64;
    __shared__ __attribute__((aligned(16))) int8_t As[BM * LDS_PITCH];
    __shared__ __attribute__((aligned(16))) int8_t Bs[BN * LDS_PITCH];
    __shared__ int2 ktab[TILE_K];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    srcB.template prepare<BN>(col0);

    for (int k0 = 0; k0 < K; k0 += TILE_K)
    {
        srcA.template load_tile<BM>(As, row0, k0);
        if constexpr (__is_same(SrcB, Im2colOperand))
        {
            srcB.fill_ktab(ktab, k0);
            __syncthreads();
            srcB.template load_tile<BN>(Bs, ktab);
        }
        else
        {
            srcB.template load_tile<BN>(Bs, col0, k0);
        }
        __syncthreads();

#pragma unroll
        for (int ks = 0; ks < TILE_K; ks += 32)
        {
            v4i a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                a[i] = *reinterpret_cast<const v4i*>(As + (wm * (BM / 2) + i * 32 + l32) * LDS_PITCH + ks + lhi * 16);
#pragma unroll
            for (int j = 0; j < TN; j++)
                b[j] = *reinterpret_cast<const v4i*>(Bs + (wn * (BN / 2) + j * 32 + l32) * LDS_PITCH + ks + lhi * 16);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int gi = row0 + wm * (BM / 2) + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                const int gj = col0 + wn * (BN / 2) + j * 32 + l32;
                if (gi < M && gj < N) epi(gi, gj, acc[i][j][r]);
            }
}

} // namespace ncnnhip

#endif // NCNNHIP_MFMA_TILE_H
