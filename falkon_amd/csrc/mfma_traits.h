// MFMA tile traits shared by the LDS-tiled product kernel and the kernel-matrix kernel (gfx950).
#pragma once
#include <hip/hip_runtime.h>

namespace flk {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef double doublex2 __attribute__((ext_vector_type(2)));

template <typename T> struct LTraits;

template <> struct LTraits<float> {
    static constexpr int BLK = 32, KG = 2, ACCN = 16, NG = 4, VPL = 4;  // VPL: elements per 16-byte vector
    typedef floatx16 acc_t;
    typedef floatx4 vec4_t;
    typedef floatx4 v16_t;     // one 16-byte load
    static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // offset (within the block, in matrix rows) of the g-th group of 4 consecutive accumulator rows
    static __device__ __forceinline__ int group_off(int g, int lg) { return 8 * g + 4 * lg; }
    static __device__ __forceinline__ int out_row(int j) { return j; }
    // matrix row (within its block) of accumulator register r in lane group lg
    static __device__ __forceinline__ int acc_row(int r, int lg) { return 8 * (r >> 2) + 4 * lg + (r & 3); }
};

template <> struct LTraits<double> {
    static constexpr int BLK = 16, KG = 4, ACCN = 4, NG = 1, VPL = 2;
    typedef doublex4 acc_t;
    typedef doublex4 vec4_t;
    typedef doublex2 v16_t;
    static __device__ __forceinline__ acc_t mfma(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int group_off(int g, int lg) { return 4 * lg; }
    static __device__ __forceinline__ int out_row(int j) { return 4 * (j & 3) + (j >> 2); }
    static __device__ __forceinline__ int acc_row(int r, int lg) { return 4 * lg + r; }
};

}  // namespace flk
