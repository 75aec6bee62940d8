// Shared device/host helpers for the gfx950 kernels of libqmll.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qmll.h"

#define QMLL_WAVE 64

// thread-local text of the last failure, returned by qmll_last_error()
void qmll_set_error(const char* fmt, ...);

#define QMLL_REQUIRE(cond, code, ...)          \
    do {                                        \
        if (!(cond)) {                          \
            qmll_set_error(__VA_ARGS__);        \
            return (code);                      \
        }                                       \
    } while (0)

// call after every launch: a failed launch is reported, never swallowed
#define QMLL_CHECK_LAUNCH(name)                                                         \
    do {                                                                                \
        hipError_t e__ = hipGetLastError();                                             \
        if (e__ != hipSuccess) {                                                        \
            qmll_set_error("%s: launch failed: %s", name, hipGetErrorString(e__));      \
            return QMLL_ERR_LAUNCH;                                                     \
        }                                                                               \
    } while (0)

static inline bool qmll_is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
static inline int qmll_log2(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

#ifdef __HIPCC__

__device__ __forceinline__ int lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// value held by lane (lane ^ MASK); MASK is a power of two below 64
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
    int vi = __float_as_int(v);
    int r;
    if constexpr (MASK == 1) {
        r = __builtin_amdgcn_update_dpp(0, vi, 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
    } else if constexpr (MASK == 2) {
        r = __builtin_amdgcn_update_dpp(0, vi, 0x4E, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
    } else if constexpr (MASK == 8) {
        r = __builtin_amdgcn_update_dpp(0, vi, 0x128, 0xf, 0xf, false);  // row_ror:8
    } else if constexpr (MASK == 4) {
        // lanes 0-3 / 8-11 of a row take lane+4 (row_shl:4, banks 0 and 2), the others lane-4
        r = __builtin_amdgcn_update_dpp(0, vi, 0x104, 0xf, 0x5, false);
        r = __builtin_amdgcn_update_dpp(r, vi, 0x114, 0xf, 0xA, false);
    } else if constexpr (MASK == 16) {
        r = __builtin_amdgcn_ds_swizzle(vi, 0x401F);                     // bit mode: and 0x1f, xor 16
    } else {
        r = __shfl_xor(vi, MASK, 64);
    }
    return __int_as_float(r);
}

// sum over the 64 lanes, result in every lane
__device__ __forceinline__ float wave_sum(float v) {
    v += lane_xor<1>(v);
    v += lane_xor<2>(v);
    v += lane_xor<4>(v);
    v += lane_xor<8>(v);
    v += lane_xor<16>(v);
    v += lane_xor<32>(v);
    return v;
}

// Large-argument fallback, kept out of line so the unrolled feature loops stay small.
__device__ __attribute__((noinline)) inline void sincos_large(float x, float* s, float* c) { sincosf(x, s, c); }

// sin and cos of an fp32 argument to ~1 ulp (7e-8 absolute, measured over |x| < 1000): a
// 3-term Cody-Waite reduction by pi/2 with FMA, then minimax polynomials on [-pi/4, pi/4].
// Arguments beyond 3.2e4 take the library routine.
__device__ __forceinline__ void sincos_f32(float x, float* s, float* c) {
    float kf = rintf(x * 0.63661977236758134308f);
    int k = (int)kf;
    float r = fmaf(kf, -1.57079601287841796875f, x);          // pi/2 split in three fp32 parts
    r = fmaf(kf, -3.1391647326017846353352069854736328125e-07f, r);
    r = fmaf(kf, -5.3903029534742383e-15f, r);
    float r2 = r * r;
    // sin(r) ~ r + r^3 * P(r^2), cos(r) ~ 1 - r^2/2 + r^4 * Q(r^2)
    float ps = fmaf(r2, 2.86567956e-6f, -1.98559923e-4f);
    ps = fmaf(ps, r2, 8.33338592e-3f);
    ps = fmaf(ps, r2, -1.66666672e-1f);
    float sr = fmaf(ps * r2, r, r);
    float pc = fmaf(r2, 2.44677067e-5f, -1.38877297e-3f);
    pc = fmaf(pc, r2, 4.16666567e-2f);
    pc = fmaf(pc, r2, -0.5f);
    float cr = fmaf(pc, r2, 1.0f);
    const bool swap = k & 1;
    float ss = swap ? cr : sr;
    float cc = swap ? sr : cr;
    // quadrant signs: sin flips for k mod 4 in {2,3}, cos for {1,2}
    ss = __int_as_float(__float_as_int(ss) ^ ((k & 2) << 30));
    cc = __int_as_float(__float_as_int(cc) ^ (((k + 1) & 2) << 30));
    if (__builtin_expect(fabsf(x) > 32000.0f, 0)) sincos_large(x, &ss, &cc);
    *s = ss;
    *c = cc;
}

// sin and cos on the transcendental unit (v_sin_f32 / v_cos_f32 take revolutions): the
// argument is first reduced to |r| <= pi by a Cody-Waite step with 2 pi split in two fp32
// parts (exact for |x| <= 3.2e4), so the conversion to revolutions loses nothing.  Measured
// against fp64 over |x| < 1500: 3.7e-7 maximum, 7.5e-8 rms absolute error.  Two
// transcendental issues and five plain instructions replace the 17 of a polynomial pair.
__device__ __forceinline__ void sincos_hw(float x, float* s, float* c) {
    const float t = fmaf(x, 0.15915494309189535f, 12582912.0f);   // + 1.5 * 2^23: rounds x / 2 pi
    const float kf = t - 12582912.0f;
    float r = fmaf(kf, -6.2831840515136719f, x);
    r = fmaf(kf, -1.2556659e-06f, r);
    const float u = r * 0.15915494309189535f;
    *s = __builtin_amdgcn_sinf(u);
    *c = __builtin_amdgcn_cosf(u);
}

// cosine / sine alone, any argument: the library routine takes over beyond the range of
// the two-part reduction
__device__ __forceinline__ float cos_hw(float x) {
    float s, c;
    sincos_hw(x, &s, &c);
    if (__builtin_expect(fabsf(x) > 32000.0f, 0)) sincos_large(x, &s, &c);
    return c;
}
__device__ __forceinline__ float sin_hw(float x) {
    float s, c;
    sincos_hw(x, &s, &c);
    if (__builtin_expect(fabsf(x) > 32000.0f, 0)) sincos_large(x, &s, &c);
    return s;
}

// ---- fp32 operands for the half-precision matrix cores --------------------------------------
// An fp32 value as two fp16 parts, hi = the value rounded to fp16 and lo = the rounded rest (22 bits
// together): a product of two such values is hi.hi + hi.lo + lo.hi on v_mfma_f32_32x32x16_f16,
// accumulated in fp32.  fp16 has five exponent bits, so the caller first scales by a power of two
// (exact) that takes the largest entry of the operand to [2^13, 2^14); the matrix cores keep fp16
// subnormals, so smaller entries lose only bits below 2^-38 of the largest.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void split_f16(float v, _Float16& hi, _Float16& lo) {
    // v as it was rounded to fp32: when v is a product, the compiler may otherwise contract the
    // multiply into one of the two conversions (v_fma_mix) and not the other, and the two parts then
    // refer to different roundings of v near a tie (an error of one fp16 unit in the last place)
    asm("" : "+v"(v));
    hi = (_Float16)v;
    lo = (_Float16)(v - (float)hi);
}

// |v| for finite v, 0 for an infinity or a NaN: the operand scales below are taken from the largest
// FINITE entry, so that a non-finite entry spoils its own row only (its parts become Inf / NaN) and
// not the rows that share its scale (which an infinite maximum would scale down to nothing)
__device__ __forceinline__ float finite_abs(float v) {
    const float a = fabsf(v);
    return a <= 3.4028234663852886e38f ? a : 0.0f;
}
__device__ __forceinline__ bool not_finite(float m) { return !(m <= 3.4028234663852886e38f); }

// 2^k with k clamped to what a float holds
__device__ __forceinline__ float pow2i(int k) { return __int_as_float((min(max(k, -126), 127) + 127) << 23); }

// k such that m 2^k lies in [2^13, 2^14) (m > 0 finite), 0 for m = 0; at most 126, so that 2^k and
// 2^-k are both floats (operands below 2^-113 then sit lower in fp16's range)
__device__ __forceinline__ int scale_exponent(float m) {
    if (!(m > 0.0f)) return 0;
    const int e = (int)((__float_as_uint(m) >> 23) & 0xff) - 127;      // floor(log2 m) for normal m
    return min(13 - max(e, -126), 126);
}

#endif  // __HIPCC__
