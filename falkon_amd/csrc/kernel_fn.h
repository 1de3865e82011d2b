// The radial kernel functions applied to the accumulator of a tile (gfx950).
//
// Rows are packed scaled by operand_scale(kernel)/sigma with their half norms h = -1/2 |x~|^2, so that the
// MFMA chain plus the two half norms leaves e = x~.c~ + hA + hB = -1/2 |x~ - c~|^2 in the accumulator:
//
//   Gaussian   (falkon/kernels/distance_kernel.py:140-159): operand_scale = sqrt(log2 e), K = exp2(e), and the
//              reference's clamp of the squared distance at 1e-20 is K <= 1;
//   the others (operand_scale = 1, e = -D^2/2 with D = |x/sigma - c/sigma|, D^2 clamped at 1e-20 as in
//              distance_kernel.py:100 before the square root):
//     Laplacian    (distance_kernel.py:182-205):  K = exp(-D)
//     Matern nu=3/2 (distance_kernel.py:243-254): K = (1 + s) exp(-s),            s = sqrt(3) D
//     Matern nu=5/2 (distance_kernel.py:255-267): K = (1 + s + s^2/3) exp(-s),    s = sqrt(5) D
//   Matern nu = 1/2 is the Laplacian and nu = inf the Gaussian (distance_kernel.py:235-238).
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/falkon_amd.h"

namespace flk {

constexpr double kLog2e = 1.4426950408889634;

template <int KF> __device__ __forceinline__ float kernel_value(float e);
template <int KF> __device__ __forceinline__ double kernel_value(double e);

// Gaussian: the median-of-three with 0 and 1 folds into the clamp bit of v_exp_f32, so the clamp is free
template <> __device__ __forceinline__ float kernel_value<FLK_GAUSSIAN>(float e) {
    return __builtin_amdgcn_fmed3f(__builtin_amdgcn_exp2f(e), 0.0f, 1.0f);
}
template <> __device__ __forceinline__ double kernel_value<FLK_GAUSSIAN>(double e) { return exp2(fmin(e, 0.0)); }

// distance D from e = -D^2/2, with the reference's clamp
__device__ __forceinline__ float clamped_distance(float e) { return __builtin_amdgcn_sqrtf(fmaxf(-2.0f * e, 1e-20f)); }
__device__ __forceinline__ double clamped_distance(double e) { return sqrt(fmax(-2.0 * e, 1e-20)); }

template <> __device__ __forceinline__ float kernel_value<FLK_LAPLACIAN>(float e) {
    return __builtin_amdgcn_exp2f(clamped_distance(e) * (float)(-kLog2e));
}
template <> __device__ __forceinline__ double kernel_value<FLK_LAPLACIAN>(double e) {
    return exp2(clamped_distance(e) * -kLog2e);
}

template <> __device__ __forceinline__ float kernel_value<FLK_MATERN32>(float e) {
    const float s = clamped_distance(e) * 1.7320508075688772f;
    return (1.0f + s) * __builtin_amdgcn_exp2f(s * (float)(-kLog2e));
}
template <> __device__ __forceinline__ double kernel_value<FLK_MATERN32>(double e) {
    const double s = clamped_distance(e) * 1.7320508075688772;
    return (1.0 + s) * exp2(s * -kLog2e);
}

template <> __device__ __forceinline__ float kernel_value<FLK_MATERN52>(float e) {
    const float s = clamped_distance(e) * 2.23606797749979f;
    const float poly = __builtin_fmaf(s, __builtin_fmaf(s, 1.0f / 3.0f, 1.0f), 1.0f);
    return poly * __builtin_amdgcn_exp2f(s * (float)(-kLog2e));
}
template <> __device__ __forceinline__ double kernel_value<FLK_MATERN52>(double e) {
    const double s = clamped_distance(e) * 2.23606797749979;
    return fma(s, fma(s, 1.0 / 3.0, 1.0), 1.0) * exp2(s * -kLog2e);
}

}  // namespace flk
