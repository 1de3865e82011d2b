// The radial kernel functions applied to the accumulator of a tile (gfx950).
//
// Rows are packed scaled by operand_scale(kernel)/sigma with their half norms h = -1/2 |x~|^2, so that the
// MFMA chain plus the two half norms leaves e = x~.c~ + hA + hB = -1/2 |x~ - c~|^2 in the accumulator.  The
// scale is chosen per kernel so that the epilogue needs no multiplication to get at its argument
// (D = |x/sigma - c/sigma|, L = log2 e):
//
//   Gaussian   (falkon/kernels/distance_kernel.py:140-159): scale sqrt(L), e = -L D^2/2, K = exp2(e); the
//              reference's clamp of the squared distance at 1e-20 is K <= 1; (in double precision the scale is
//              sqrt(2048 L) and K = exp2(e / 2048), see kGaussExpBits;)
//   Laplacian  (distance_kernel.py:182-205): scale sqrt(2) L, -e = (L D)^2 =: q^2, K = exp(-D) = exp2(-q);
//   Matern 3/2 (distance_kernel.py:243-254): scale sqrt(6) L, q = L s with s = sqrt(3) D,
//              K = (1 + s) exp(-s) = (1 + q/L) exp2(-q);
//   Matern 5/2 (distance_kernel.py:255-267): scale sqrt(10) L, q = L s with s = sqrt(5) D,
//              K = (1 + s + s^2/3) exp(-s) = (1 + q/L + q^2/(3 L^2)) exp2(-q).
//   Laplacian derivative weight (FLK_LAPLACIAN_DU): packed like the Laplacian, K = exp(-D)/D = L exp2(-q)/q, and 0
//              where D^2 <= 1e-20 (where the reference's clamp stops the gradient).
//   The reference clamps D^2 at 1e-20 before the square root (distance_kernel.py:100): q^2 is clamped at
//   (scale^2 / 2) * 1e-20.  Matern nu = 1/2 is the Laplacian and nu = inf the Gaussian (distance_kernel.py:235-238).
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/falkon_amd.h"

namespace flk {

constexpr double kLog2e = 1.4426950408889634;
constexpr double kSqrtLog2e = 1.2011224087864498;
constexpr double kSqrt2 = 1.4142135623730951;
constexpr double kSqrt3 = 1.7320508075688772;
constexpr double kSqrt5 = 2.23606797749979;

// The Gaussian's exponent in double precision is carried times 2^kGaussExpBits (the packed rows take the square root of
// that factor, the half norms the factor itself, at no cost): the accumulator then holds E = 2048 e, whose integer and
// fractional parts are what the table-based exponential needs (exp2_table_scaled), one conversion and one v_fract_f64
// instead of the three additions that round e to a multiple of 1/2048.
constexpr int kGaussExpBits = 11;
constexpr double kGaussExpScale = 2048.0;
constexpr double kSqrtGaussExpScale = 45.254833995939045;       // sqrt(2048)

// factor on x / sigma when a matrix is packed for the kernel (packed_f64: the packed operand is double precision)
inline double operand_scale(int kf, bool packed_f64) {
    switch (kf) {
        case FLK_LAPLACIAN:
        case FLK_LAPLACIAN_DU: return kLog2e * kSqrt2;
        case FLK_MATERN32:  return kSqrt3 * kLog2e * kSqrt2;
        case FLK_MATERN52:  return kSqrt5 * kLog2e * kSqrt2;
        default:            return packed_f64 ? kSqrtLog2e * kSqrtGaussExpScale : kSqrtLog2e;
    }
}

// 2^e in double precision for e <= 0 (gfx950 has no fp64 exponential instruction; this replaces the library routine,
// which also serves positive, huge and non-finite arguments: 8 % off the small-d fp64 products).  e = n + f with
// n = rint(e) read from the low word of e + 1.5 * 2^52 and f = e - n in [-1/2, 1/2] exact; 2^f from the degree-11
// interpolant at the Chebyshev nodes (relative error 3.2e-18 before rounding; 2^0 = 1 exactly); v_ldexp_f64 applies
// 2^n and rounds results below 2^-1022 correctly.  Arguments below -1100 are raised to it (the result is 0 from
// -1075 on), so that n always fits the low word.  (Scaling through the exponent field instead of v_ldexp_f64, with
// results below 2^-1021 flushed to zero, measured no faster.)
// max(e, about -1100) for the exponentials below, done on the high word as an unsigned integer (one 32-bit
// instruction): among negative doubles a larger high word is a more negative number, so capping it at the high word
// of -1100.0 raises everything below to [-1100.2, -1100], leaves the rest alone, and turns a negative NaN into -1100 too
// (non-finite rows are handled through their half norms, not through the kernel values).  The fp64 maximum would
// cost two instructions: the compiler has to quieten its operand first, as it does not know that an MFMA result
// cannot be a signalling NaN.  (Inline assembly on an accumulator register is no way around that: the wait states
// an MFMA result needs before a vector instruction may read it are not inserted for assembly.)
__device__ __forceinline__ double raise_to_exp_range(double e) {
    const unsigned long long bits = (unsigned long long)__double_as_longlong(e);
    const unsigned hi = min((unsigned)(bits >> 32), 0xC0913000u);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | (bits & 0xffffffffull)));
}

__device__ __forceinline__ double exp2_nonpositive(double e) {
    constexpr double kRound = 6755399441055744.0;       // 1.5 * 2^52: adding it rounds to the nearest integer
    e = raise_to_exp_range(e);
    const double t = e + kRound;
    const int n = (int)(unsigned)__double_as_longlong(t);  // the integer, in two's complement, is the low word
    const double f = e - (t - kRound);
    double p = 0x1.e9ec1fcb69a7fp-32;
    p = fma(p, f, 0x1.e6228acd1c6e5p-28);
    p = fma(p, f, 0x1.b524ebd13a55fp-24);
    p = fma(p, f, 0x1.62bfc2c86d700p-20);
    p = fma(p, f, 0x1.ffcbfc6da6ed1p-17);
    p = fma(p, f, 0x1.430913112c61bp-13);
    p = fma(p, f, 0x1.5d87fe78a3f9cp-10);
    p = fma(p, f, 0x1.3b2ab6fb9f1a5p-7);
    p = fma(p, f, 0x1.c6b08d704a0c6p-5);
    p = fma(p, f, 0x1.ebfbdff82c5aep-3);
    p = fma(p, f, 0x1.62e42fefa39efp-1);
    p = fma(p, f, 1.0);
    return __builtin_ldexp(p, n);
}

// The same through a table: 2^e = 2^n * 2^(k/2048) * 2^f with N = rint(2048 e) = 2048 n + k (k the low 11 bits of
// N, n = N >> 11) and |f| <= 2^-12, where the cubic Taylor polynomial of 2^f is exact to 3.4e-17.  tab[k] = 2^(k/2048)
// lives in LDS (16 KB per workgroup, exp2_table_fill): ten fp64 and three 32-bit instructions in place of eighteen fp64
// ones, and the LDS read runs beside the vector ALU.  For e <= 0 like exp2_nonpositive (a positive e up to 2^20 works
// too); arguments below -1100 are raised to it.
constexpr int kExpTableBits = 11;
constexpr int kExpTableSize = 1 << kExpTableBits;

// All threads of the workgroup call this once, followed by a workgroup barrier, before exp2_table is used.
__device__ __forceinline__ void exp2_table_fill(double *tab, int tid, int nthreads) {
    for (int k = tid; k < kExpTableSize; k += nthreads)
        tab[k] = 2.0 * exp2_nonpositive((double)(k - kExpTableSize) * (1.0 / kExpTableSize));
}

template <bool ON_FMA = true>
__device__ __forceinline__ double exp2_table(double e, const double *tab) {
    // adding 1.5 * 2^41 (ulp 2^-11) rounds e to the nearest multiple of 1/2048 and leaves N = rint(2048 e), in two's
    // complement, in the low word of the sum; no multiplication is involved
    constexpr double kRound = 3298534883328.0;               // 1.5 * 2^41
    // (the instruction itself: the builtin would quieten a signalling NaN first, one more fp64 instruction per value)
    const double c = raise_to_exp_range(e);
    const double t = c + kRound;
    const int N = (int)(unsigned)__double_as_longlong(t);
    // ON_FMA: two of the additions and the product with the table entry are issued as v_fma_f64 (x * 1 + y,
    // x * y + 0): on gfx950 that instruction measures 6.0 cycles per wave against 7.5 for v_add_f64 and 7.7 for
    // v_mul_f64.  (They depend on t, so they come after the compiler's own first read of e, which carries the MFMA
    // wait states.)  It pays where the MFMA chain is long enough to schedule around the fixed instructions (mmv at
    // N = 5e5, M = 2e4: d = 28 12.5 -> 12.1 ms, but d = 9 7.6 -> 8.4): the callers choose.
    double r, f, y;
    if constexpr (ON_FMA) {
        asm("v_fma_f64 %0, %1, 1.0, %2" : "=v"(r) : "v"(t), "s"(-kRound));
        asm("v_fma_f64 %0, %1, -1.0, %2" : "=v"(f) : "v"(r), "v"(c));
    } else {
        r = t - kRound;
        f = c - r;
    }                                                                // f: exact, |f| <= 2^-12
    double p = fma(0x1.c6b08d704a0bfp-5, f, 0x1.ebfbdff82c58ep-3);   // ln2^3 / 6, ln2^2 / 2
    p = fma(p, f, 0x1.62e42fefa39efp-1);                             // ln2
    p = fma(p, f, 1.0);
    const double entry = tab[N & (kExpTableSize - 1)];
    if constexpr (ON_FMA) asm("v_fma_f64 %0, %1, %2, 0" : "=v"(y) : "v"(p), "v"(entry));
    else y = p * entry;
    return __builtin_ldexp(y, N >> kExpTableBits);
}

// 2^(E / 2048) for E <= 0 from the same table: N = ceil(E) (v_cvt_i32_f64 truncates towards zero and saturates, so no
// clamp is needed: from -2^31 on the result is 0), x = E - N = -fract(-E) in (-1, 0], 2^(E/2048) = 2^(N >> 11) *
// tab[N & 2047] * 2^(x/2048); the last factor is 1 + fx (a1 + fx (a2 + fx a3)) with fx = -x, the cubic through the
// Chebyshev nodes of (2^y - 1) / y on [-2^-11, 0] (relative error 1.7e-17 before rounding, exactly 1 at x = 0).
// Eight fp64 and three 32-bit instructions per value.  E must not be positive: ceil and fract would disagree there.
template <bool ON_FMA = true>
__device__ __forceinline__ double exp2_table_scaled(double E, const double *tab) {
    const int N = (int)E;
    const double fx = __builtin_amdgcn_fract(-E);
    double p = fma(-0x1.c6a1c7b96fda5p-38, fx, 0x1.ebfbdfcbdb733p-25);
    p = fma(p, fx, -0x1.62e42fefa38b4p-12);
    p = fma(p, fx, 1.0);
    const double entry = tab[N & (kExpTableSize - 1)];
    double y;
    if constexpr (ON_FMA) asm("v_fma_f64 %0, %1, %2, 0" : "=v"(y) : "v"(p), "v"(entry));
    else y = p * entry;
    return __builtin_ldexp(y, N >> kExpTableBits);
}

// How a kernel function evaluates 2^x in double precision: by polynomial, or from the table in LDS.  scaled(E) is
// 2^(E / 2048) for E <= 0, the Gaussian's form.
struct Exp2Poly {
    __device__ __forceinline__ double operator()(double e) const { return exp2_nonpositive(e); }
    __device__ __forceinline__ double scaled(double E) const { return exp2_nonpositive(E * (1.0 / kGaussExpScale)); }
};
template <bool ON_FMA> struct Exp2Table {
    const double *tab;
    __device__ __forceinline__ double operator()(double e) const { return exp2_table<ON_FMA>(e, tab); }
    __device__ __forceinline__ double scaled(double E) const { return exp2_table_scaled<ON_FMA>(E, tab); }
};

template <int KF> struct KernelFn;

// Gaussian: the median-of-three with 0 and 1 folds into the clamp bit of v_exp_f32, so the clamp is free
template <> struct KernelFn<FLK_GAUSSIAN> {
    static __device__ __forceinline__ float value(float e) {
        return __builtin_amdgcn_fmed3f(__builtin_amdgcn_exp2f(e), 0.0f, 1.0f);
    }
    // (double precision: the accumulator holds 2048 e, see kGaussExpBits)
    template <class E> static __device__ __forceinline__ double value(double e, E ex) {
        return ex.scaled(fmin(e, 0.0));
    }
};

// q = sqrt(max(-e, clamp)): the scaled distance, with the reference's clamp carried over to q^2
template <int KF> constexpr double distance_clamp() {
    return (KF == FLK_MATERN32 ? 3.0 : KF == FLK_MATERN52 ? 5.0 : 1.0) * kLog2e * kLog2e * 1e-20;
}
template <int KF> __device__ __forceinline__ float scaled_distance(float e) {
    return __builtin_amdgcn_sqrtf(fmaxf(-e, (float)distance_clamp<KF>()));
}
// Square root of a positive, finite, normal double (the clamp keeps the argument at 1e-20 or above): the hardware's
// reciprocal square root as the seed, one coupled step for the root g and half its reciprocal h, and one correction
// by the residual x - g^2.  The library's sqrt runs the same steps plus a second correction (exact rounding), a
// rescaling of subnormal arguments and a fix-up for 0 and infinity: eight more fp64-rate instructions per value,
// which none of the arguments here need (an infinite squared distance gives NaN here, not K = 0).
__device__ __forceinline__ double sqrt_clamped(double x) {
    const double y = __builtin_amdgcn_rsq(x);
    double g = x * y, h = 0.5 * y;
    const double r = fma(-h, g, 0.5);
    g = fma(g, r, g);
    h = fma(h, r, h);
    return fma(fma(-g, g, x), h, g);
}
template <int KF> __device__ __forceinline__ double scaled_distance(double e) {
    return sqrt_clamped(fmax(-e, distance_clamp<KF>()));
}

template <> struct KernelFn<FLK_LAPLACIAN> {
    static __device__ __forceinline__ float value(float e) {
        return __builtin_amdgcn_exp2f(-scaled_distance<FLK_LAPLACIAN>(e));
    }
    template <class E> static __device__ __forceinline__ double value(double e, E ex) {
        return ex(-scaled_distance<FLK_LAPLACIAN>(e));
    }
};

template <> struct KernelFn<FLK_LAPLACIAN_DU> {
    static __device__ __forceinline__ float value(float e) {
        const float q = scaled_distance<FLK_LAPLACIAN_DU>(e);
        const float k = __builtin_amdgcn_exp2f(-q) * ((float)kLog2e * __builtin_amdgcn_rcpf(q));
        return -e > (float)distance_clamp<FLK_LAPLACIAN_DU>() ? k : 0.0f;
    }
    template <class E> static __device__ __forceinline__ double value(double e, E ex) {
        const double q = scaled_distance<FLK_LAPLACIAN_DU>(e);
        return -e > distance_clamp<FLK_LAPLACIAN_DU>() ? ex(-q) * kLog2e / q : 0.0;
    }
};

template <> struct KernelFn<FLK_MATERN32> {
    static __device__ __forceinline__ float value(float e) {
        const float q = scaled_distance<FLK_MATERN32>(e);
        return __builtin_fmaf(q, (float)(1.0 / kLog2e), 1.0f) * __builtin_amdgcn_exp2f(-q);
    }
    template <class E> static __device__ __forceinline__ double value(double e, E ex) {
        const double q = scaled_distance<FLK_MATERN32>(e);
        return fma(q, 1.0 / kLog2e, 1.0) * ex(-q);
    }
};

template <> struct KernelFn<FLK_MATERN52> {
    static __device__ __forceinline__ float value(float e) {
        const float q = scaled_distance<FLK_MATERN52>(e);
        const float poly = __builtin_fmaf(q, __builtin_fmaf(q, (float)(1.0 / (3.0 * kLog2e * kLog2e)), (float)(1.0 / kLog2e)), 1.0f);
        return poly * __builtin_amdgcn_exp2f(-q);
    }
    template <class E> static __device__ __forceinline__ double value(double e, E ex) {
        const double q = scaled_distance<FLK_MATERN52>(e);
        return fma(q, fma(q, 1.0 / (3.0 * kLog2e * kLog2e), 1.0 / kLog2e), 1.0) * ex(-q);
    }
};

template <int KF> __device__ __forceinline__ float kernel_value(float e) { return KernelFn<KF>::value(e); }
template <int KF> __device__ __forceinline__ double kernel_value(double e) { return KernelFn<KF>::value(e, Exp2Poly{}); }
// the same with 2^x read from the table in LDS (exp2_table_fill)
template <int KF, bool ON_FMA = true> __device__ __forceinline__ double kernel_value(double e, const double *tab) {
    return KernelFn<KF>::value(e, Exp2Table<ON_FMA>{tab});
}

}  // namespace flk
