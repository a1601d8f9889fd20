// Shared host/device helpers for the gfx950 kernels.
#ifndef NCNNHIP_COMMON_H
#define NCNNHIP_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "ncnnhip.h"

namespace ncnnhip {

// ---- error plumbing (host) --------------------------------------------------------------
void set_error(const char* fmt, ...);
int map_hip_error(hipError_t e, const char* what);

#define NCNNHIP_CHECK(expr)                                          \
    do                                                               \
    {                                                                \
        hipError_t _e = (expr);                                      \
        if (_e != hipSuccess) return ::ncnnhip::map_hip_error(_e, #expr); \
    } while (0)

#define NCNNHIP_REQUIRE(cond, ...)                \
    do                                            \
    {                                             \
        if (!(cond))                              \
        {                                         \
            ::ncnnhip::set_error(__VA_ARGS__);    \
            return NCNNHIP_ERROR;                 \
        }                                         \
    } while (0)

static inline hipStream_t as_stream(void* s)
{
    return reinterpret_cast<hipStream_t>(s);
}

static inline int launch_status(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return map_hip_error(e, what);
    return NCNNHIP_OK;
}

// ---- device arithmetic: every float op is a single rounded IEEE binary32 op -------------
// (the intrinsics keep the compiler from contracting mul+add into an FMA)

__device__ __forceinline__ float mul_rn(float a, float b)
{
    return __fmul_rn(a, b);
}
__device__ __forceinline__ float add_rn(float a, float b)
{
    return __fadd_rn(a, b);
}
__device__ __forceinline__ float div_rn(float a, float b)
{
    return __fdiv_rn(a, b);
}

// round half away from zero, saturate to [-127,127]; NaN and |v| >= 2^31 give -127 like the
// x86 float->int conversion the reference runs on (INT_MIN, then clamped).
__device__ __forceinline__ int float2int8(float v)
{
    float r = roundf(v);
    if (!(fabsf(r) < 2147483648.f)) return -127;
    int q = (int)r;
    q = q > 127 ? 127 : q;
    q = q < -127 ? -127 : q;
    return q;
}

// A float whose truncation toward zero is float2int8(v); every user converts it with (int), i.e. v_cvt_i32_f32.
//   clamp first: round-half-away(clamp(v, -127, 127)) == clamp(round-half-away(v), -127, 127)
//   round as trunc(c + copysign(0.5, c)) with the ADD rounded toward zero: a nearest-even add would turn
//   0.49999997 + 0.5 into 1.0; rounded toward zero the sum never reaches the next integer unless c + 0.5 does exactly
//   (integers below 2^24 are representable, so RTZ(c + 0.5) >= floor(c + 0.5)).  The rounding mode lives in the wave's
//   MODE register (bits 1:0, 3 = toward zero): it is switched for that one add and back inside one asm statement.
//   NaN and |v| >= 2^31 give -127 like the x86 conversion of the reference (INT_MIN, then clamped).
// 5 VALU instructions (med3, bfi, add, cmp, cndmask) instead of 10 for trunc + remainder test + clamp.
__device__ __forceinline__ float float2int8_as_float(float v)
{
    const float c = __builtin_amdgcn_fmed3f(v, -127.f, 127.f);
    const float h = copysignf(0.5f, c);
    float y;
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
                 "v_add_f32 %0, %1, %2\n\t"
                 "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
                 : "=v"(y)
                 : "v"(c), "v"(h));
    return fabsf(v) < 2147483648.f ? y : -127.f;
}

// four at a time: one switch of the rounding mode and back for four adds
__device__ __forceinline__ void float2int8_as_float_x4(float& v0, float& v1, float& v2, float& v3)
{
    const float c0 = __builtin_amdgcn_fmed3f(v0, -127.f, 127.f), c1 = __builtin_amdgcn_fmed3f(v1, -127.f, 127.f);
    const float c2 = __builtin_amdgcn_fmed3f(v2, -127.f, 127.f), c3 = __builtin_amdgcn_fmed3f(v3, -127.f, 127.f);
    const float h0 = copysignf(0.5f, c0), h1 = copysignf(0.5f, c1), h2 = copysignf(0.5f, c2), h3 = copysignf(0.5f, c3);
    float y0, y1, y2, y3;
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
                 "v_add_f32 %0, %4, %8\n\t"
                 "v_add_f32 %1, %5, %9\n\t"
                 "v_add_f32 %2, %6, %10\n\t"
                 "v_add_f32 %3, %7, %11\n\t"
                 "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
                 : "=&v"(y0), "=&v"(y1), "=&v"(y2), "=&v"(y3)
                 : "v"(c0), "v"(c1), "v"(c2), "v"(c3), "v"(h0), "v"(h1), "v"(h2), "v"(h3));
    v0 = fabsf(v0) < 2147483648.f ? y0 : -127.f;
    v1 = fabsf(v1) < 2147483648.f ? y1 : -127.f;
    v2 = fabsf(v2) < 2147483648.f ? y2 : -127.f;
    v3 = fabsf(v3) < 2147483648.f ? y3 : -127.f;
}

// Clip (activation type 3) for a value known not to be NaN.  The reference writes `if (v < lo) v = lo; if (v > hi)
// v = hi;` (src/layer/fused_activation.h:25-33); for every v that is finite or infinite, and any lo and hi (a NaN bound
// leaves v alone in both forms, lo > hi ends at hi in both), max-then-min gives the same value.
__device__ __forceinline__ float clip_not_nan(float v, float lo, float hi)
{
    return fminf(fmaxf(v, lo), hi);
}

// float2int8_as_float_x4 for values the caller knows to lie inside (-2^31, 2^31): the out-of-range answer of -127
// cannot occur, so the compare and select that produce it are left out.  [lo, hi] is the clamp, inside [-127, 127]:
// a narrower one folds a preceding clip into it (see clip_folds_into_requantise).
__device__ __forceinline__ void float2int8_as_float_bounded_x4(float& v0, float& v1, float& v2, float& v3, float lo = -127.f, float hi = 127.f)
{
    const float c0 = __builtin_amdgcn_fmed3f(v0, lo, hi), c1 = __builtin_amdgcn_fmed3f(v1, lo, hi);
    const float c2 = __builtin_amdgcn_fmed3f(v2, lo, hi), c3 = __builtin_amdgcn_fmed3f(v3, lo, hi);
    const float h0 = copysignf(0.5f, c0), h1 = copysignf(0.5f, c1), h2 = copysignf(0.5f, c2), h3 = copysignf(0.5f, c3);
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
                 "v_add_f32 %0, %4, %8\n\t"
                 "v_add_f32 %1, %5, %9\n\t"
                 "v_add_f32 %2, %6, %10\n\t"
                 "v_add_f32 %3, %7, %11\n\t"
                 "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
                 : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
                 : "v"(c0), "v"(c1), "v"(c2), "v"(c3), "v"(h0), "v"(h1), "v"(h2), "v"(h3));
}

// Four already-quantised values (integers in [-127, 127] held as floats) -> four bytes, first value lowest: each
// conversion writes its low byte straight into its place in the word (sub-dword destination select), four
// instructions instead of four conversions plus the masks, shifts and ors.  A vector instruction that reads a
// register right after a sub-dword write to it needs one wait state on this chip, and the compiler does not look
// inside asm: hence the s_nop after each write (the last one covers whatever the compiler schedules next).
__device__ __forceinline__ uint32_t pack4_quantised(float a, float b, float c, float d)
{
    uint32_t r;
    asm volatile("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_i32_f32_sdwa %0, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_i32_f32_sdwa %0, %3 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_i32_f32_sdwa %0, %4 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0"
                 : "=&v"(r)
                 : "v"(a), "v"(b), "v"(c), "v"(d));
    return r;
}

// Sixteen values -> four words; the four words advance together, so no write is read by the next instruction and
// only the end needs wait states: two, which also covers a lane-row swap (v_permlane*_swap) as the next reader.
__device__ __forceinline__ void pack16_quantised(const float (&v)[16], uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3)
{
    asm volatile("v_cvt_i32_f32_sdwa %0, %4 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %1, %8 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %2, %12 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %3, %16 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %0, %5 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %1, %9 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %2, %13 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %3, %17 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %0, %6 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %1, %10 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %2, %14 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %3, %18 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %0, %7 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %1, %11 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %2, %15 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_i32_f32_sdwa %3, %19 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 1"
                 : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
                 : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "v"(v[8]), "v"(v[9]), "v"(v[10]),
                   "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]));
}

// Values already clamped into [0, 127] (a clamp whose lower bound is not negative: ReLU, ReLU6 and their like folded into the
// requantising clamp): rounding half away from zero is floor(c + 0.5) there, which v_cvt_rpi_i32_f32 computes exactly -- no
// intermediate sum is rounded (0.49999997 gives 0; compared on the device with floor((double)c + 0.5) for every float within
// 64 ulp of an integer or a half below 8 and a sweep of [0.125, 128)).  One instruction per value instead of three (sign-copied
// half, add rounded toward zero, truncating conversion), and no switch of the rounding mode.  Same wait states as above.
__device__ __forceinline__ uint32_t pack4_nonneg(float a, float b, float c, float d)
{
    uint32_t r;
    asm volatile("v_cvt_rpi_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %3 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %4 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 0"
                 : "=&v"(r)
                 : "v"(a), "v"(b), "v"(c), "v"(d));
    return r;
}
__device__ __forceinline__ void pack8_nonneg(const float (&v)[8], uint32_t& r0, uint32_t& r1)
{
    asm volatile("v_cvt_rpi_i32_f32_sdwa %0, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %6 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %3 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %7 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %4 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %8 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %5 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %9 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 1"
                 : "=&v"(r0), "=&v"(r1)
                 : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
}
__device__ __forceinline__ void pack16_nonneg(const float (&v)[16], uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3)
{
    asm volatile("v_cvt_rpi_i32_f32_sdwa %0, %4 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %8 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %2, %12 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %3, %16 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %5 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %9 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %2, %13 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %3, %17 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %6 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %10 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %2, %14 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %3, %18 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %0, %7 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %1, %11 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %2, %15 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "v_cvt_rpi_i32_f32_sdwa %3, %19 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
                 "s_nop 1"
                 : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
                 : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "v"(v[8]), "v"(v[9]), "v"(v[10]),
                   "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]));
}

// the same with one clamp per value (four different channels)
__device__ __forceinline__ void float2int8_as_float_bounded_lanes_x4(float& v0, float& v1, float& v2, float& v3, const float (&lo)[4], const float (&hi)[4])
{
    const float c0 = __builtin_amdgcn_fmed3f(v0, lo[0], hi[0]), c1 = __builtin_amdgcn_fmed3f(v1, lo[1], hi[1]);
    const float c2 = __builtin_amdgcn_fmed3f(v2, lo[2], hi[2]), c3 = __builtin_amdgcn_fmed3f(v3, lo[3], hi[3]);
    const float h0 = copysignf(0.5f, c0), h1 = copysignf(0.5f, c1), h2 = copysignf(0.5f, c2), h3 = copysignf(0.5f, c3);
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
                 "v_add_f32 %0, %4, %8\n\t"
                 "v_add_f32 %1, %5, %9\n\t"
                 "v_add_f32 %2, %6, %10\n\t"
                 "v_add_f32 %3, %7, %11\n\t"
                 "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
                 : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
                 : "v"(c0), "v"(c1), "v"(c2), "v"(c3), "v"(h0), "v"(h1), "v"(h2), "v"(h3));
}

// Clip, then multiply by the output scale, then clamp to [-127, 127] (what a clipping layer that requantises does per
// value: src/layer/fused_activation.h:25-33, then float2int8 of v * scale_out) equals multiply first and clamp once to
//   [ clamp(p0 * s), clamp(p1 * s) ]
// when p0 <= p1, s >= 0 and everything is finite: x -> RN(x * s) never decreases, so it commutes with min and max,
// and two nested clamps are one clamp to the clamped bounds.  Saves the max and the min per value.
__device__ __forceinline__ bool clip_folds_into_requantise(float p0, float p1, float s)
{
    return p0 <= p1 && s >= 0.f && s < INFINITY;
}

__device__ __forceinline__ float apply_activation(float v, const ncnnhip_activation& a)
{
    switch (a.type)
    {
    case 1:
        v = fmaxf(v, 0.f);
        break;
    case 2:
        v = v > 0.f ? v : mul_rn(v, a.p0);
        break;
    case 3:
        if (v < a.p0) v = a.p0;
        if (v > a.p1) v = a.p1;
        break;
    case 4:
        v = fminf(v, 88.3762626647949f);
        v = fmaxf(v, -88.3762626647949f);
        v = div_rn(1.f, add_rn(1.f, expf(-v)));
        break;
    case 5:
        v = mul_rn(v, tanhf(logf(add_rn(expf(v), 1.f))));
        break;
    case 6:
    {
        float lower = div_rn(-a.p1, a.p0);
        float upper = add_rn(div_rn(1.f, a.p0), lower);
        if (v < lower)
            v = 0.f;
        else if (v > upper)
            ;
        else
            v = mul_rn(v, add_rn(mul_rn(v, a.p0), a.p1));
        break;
    }
    default:
        break;
    }
    return v;
}

// n / d for 0 <= n < 2^20 and d >= 1: both are exact as floats and the float quotient (reciprocal good to an ulp or
// two, one multiply) is within 2^20 * 2^-21 = one half of the true one, so its truncation is off by at most one, which
// the remainder shows.  Seven instructions where the compiler's general 32-bit division takes about twenty-five.
__device__ __forceinline__ int small_div(int n, int d)
{
    int q = (int)((float)n * __builtin_amdgcn_rcpf((float)d));
    const int r = n - q * d;
    if (r < 0)
        q--;
    else if (r >= d)
        q++;
    return q;
}

static inline int ceil_div(long long a, long long b)
{
    return (int)((a + b - 1) / b);
}

} // namespace ncnnhip

#endif // NCNNHIP_COMMON_H
