// Shared by the register-resident kernels that contract many right-hand sides on the matrix cores (fp32:
// mmv_small_f32_wide.hip; bf16x3 mode: mmv_split_wide.hip): the forms of a pass, the staged right-hand sides of an A
// block, the contraction steps and the final store.
#pragma once
#include <hip/hip_runtime.h>

namespace flk {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// The staged values of an A block are hn(32) | vec[32 rows][COLS + 1] (the odd row stride makes the reads conflict
// free); the columns of the 32-groups come first, then the 16-group, then the 8-group
template <int COLS> struct WideGeo {
    static_assert(COLS % 8 == 0 && COLS >= 8 && COLS <= 64 && COLS != 56, "8, 16, 24, 32, 40, 48 or 64 columns");
    static constexpr int kCols = COLS;
    static constexpr int kN32 = COLS / 32, kH16 = (COLS % 32) / 16, kQ8 = (COLS % 16) / 8;
    static constexpr int kOff16 = 32 * kN32, kOff8 = kOff16 + 16 * kH16;
    static constexpr int kStride = kCols + 1;
    static constexpr int kStage = 32 + 32 * kStride;
    static constexpr int kFetch = 1 + kCols / 8;         // dwords a thread fetches per A block
};
constexpr int kWideMaxCols = 64;

// Output accumulators of the resident blocks (the members a form does not use are never touched)
template <int FR, int COLS> struct WideAcc {
    floatx16 g32[FR][WideGeo<COLS>::kN32 > 0 ? WideGeo<COLS>::kN32 : 1];
    floatx16 h16[FR];
    floatx4 q8[FR][2];
};

template <int COLS> struct WideRowVals { float x[WideGeo<COLS>::kFetch]; };

// The row values of an A block (half norms and right-hand side entries) are the same for the four waves of a
// workgroup, which walk the same reduction chunk: the workgroup fetches them once, thread t the half norm of row
// t % 32 and the entries vec[row t % 32][t / 32 + 8 c], c = 0 .. COLS / 8 - 1 (128-byte runs of the planes), and stages
// them in one LDS buffer that every wave reads its MFMA operands from.  (With a private copy per wave the loads per lane
// and block cost 9 % of the launch: N = 1e6, M = 2e4, d = 28, 32 columns, 21.3 ms against 19.4 with those loads
// removed.)
template <int COLS>
__device__ __forceinline__ void wide_fetch(WideRowVals<COLS> &rv, const float *__restrict__ hA,
                                           const float *__restrict__ vecp, int64_t vec_ld, int64_t ab, int tid) {
    const int r = tid & 31, p0 = tid >> 5;
    rv.x[0] = hA[ab * 32 + r];
#pragma unroll
    for (int c = 0; c < COLS / 8; c++) rv.x[1 + c] = vecp[(int64_t)(p0 + 8 * c) * vec_ld + ab * 32 + r];
}
template <int COLS>
__device__ __forceinline__ void wide_stage(const WideRowVals<COLS> &rv, float *lds, int tid) {
    const int r = tid & 31, p0 = tid >> 5;
    if (p0 == 0) lds[r] = rv.x[0];
#pragma unroll
    for (int c = 0; c < COLS / 8; c++) lds[32 + r * WideGeo<COLS>::kStride + p0 + 8 * c] = rv.x[1 + c];
}
// Workgroup barrier that drains the wave's LDS traffic only (not its global loads, which are meant to stay in flight)
__device__ __forceinline__ void wide_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// B operands of one contraction step: one value per 32-group, one for the 16-group, two for the 8-group
template <int COLS> struct WideB {
    float g32[WideGeo<COLS>::kN32 > 0 ? WideGeo<COLS>::kN32 : 1];
    float h16;
    float q8[2];
};
template <int COLS>
__device__ __forceinline__ void wide_read_b(WideB<COLS> &b, const float *lds, int row, int j) {
    using G = WideGeo<COLS>;
    const float *p = lds + 32 + row * G::kStride;
#pragma unroll
    for (int g = 0; g < G::kN32; g++) b.g32[g] = p[32 * g + j];
    if constexpr (G::kH16 != 0) b.h16 = p[G::kOff16 + (j & 15)];
    if constexpr (G::kQ8 != 0) {
        b.q8[0] = p[G::kOff8 + (j & 3)];
        b.q8[1] = p[G::kOff8 + 4 + (j & 3)];
    }
}
// compiler fence on the operands of a step (otherwise every read is hoisted to the front)
template <int COLS>
__device__ __forceinline__ void wide_fence_b(WideB<COLS> &b, const float *lds) {
    using G = WideGeo<COLS>;
#pragma unroll
    for (int g = 0; g < G::kN32; g++) asm volatile("" : "+v"(b.g32[g]) : "v"(lds) : "memory");
    if constexpr (G::kH16 != 0) asm volatile("" : "+v"(b.h16) : "v"(lds) : "memory");
    if constexpr (G::kQ8 != 0) {
        asm volatile("" : "+v"(b.q8[0]) : "v"(lds) : "memory");
        asm volatile("" : "+v"(b.q8[1]) : "v"(lds) : "memory");
    }
}

// out[q] += (kernel values in the accumulator registers acc[q]) contracted with the staged right-hand sides of the A
// block at lds, on the matrix cores; the B operands are read one step ahead, fenced
template <int FR, int COLS>
__device__ __forceinline__ void wide_contract(const floatx16 (&acc)[FR], const float *lds, int j, int h,
                                              WideAcc<FR, COLS> &out) {
    using G = WideGeo<COLS>;
    WideB<COLS> bval, bnext;
    wide_read_b<COLS>(bval, lds, 4 * h, j);
    bnext = bval;
#pragma unroll
    for (int s2 = 0; s2 < 16; s2++) {
        if (s2 + 1 < 16) wide_read_b<COLS>(bnext, lds, 8 * ((s2 + 1) >> 2) + 4 * h + ((s2 + 1) & 3), j);
#pragma unroll
        for (int g = 0; g < G::kN32; g++)
#pragma unroll
            for (int q = 0; q < FR; q++)
                out.g32[q][g] = __builtin_amdgcn_mfma_f32_32x32x2f32(acc[q][s2], bval.g32[g], out.g32[q][g], 0, 0, 0);
        if constexpr (G::kH16 != 0) {
#pragma unroll
            for (int q = 0; q < FR; q++)
                out.h16[q] = __builtin_amdgcn_mfma_f32_16x16x1f32(acc[q][s2], bval.h16, out.h16[q], 0, 0, 0);
        }
        if constexpr (G::kQ8 != 0) {
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int q = 0; q < FR; q++)
                    out.q8[q][u] = __builtin_amdgcn_mfma_f32_4x4x1f32(acc[q][s2], bval.q8[u], out.q8[q][u], 0, 0, 0);
        }
        wide_fence_b<COLS>(bval, lds);
        bval = bnext;
    }
}

template <int FR, int COLS>
__device__ __forceinline__ void wide_zero(WideAcc<FR, COLS> &out) {
    using G = WideGeo<COLS>;
#pragma unroll
    for (int q = 0; q < FR; q++) {
#pragma unroll
        for (int g = 0; g < G::kN32; g++)
#pragma unroll
            for (int r = 0; r < 16; r++) out.g32[q][g][r] = 0.f;
        if constexpr (G::kH16 != 0) {
#pragma unroll
            for (int r = 0; r < 16; r++) out.h16[q][r] = 0.f;
        }
        if constexpr (G::kQ8 != 0) {
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int r = 0; r < 4; r++) out.q8[q][u][r] = 0.f;
        }
    }
}

// partial[by][t][block bb0 + q] = the wave's sums, for the first tcols columns
template <int FR, int COLS>
__device__ __forceinline__ void wide_store(const WideAcc<FR, COLS> &out, float *__restrict__ partial, unsigned by, int tcols,
                                           int64_t nb_pad, int64_t bb0, int64_t nb_blocks, int lane) {
    using G = WideGeo<COLS>;
    const int j = lane & 31, h = lane >> 5;
    // 32-groups: lane = column t, registers = output rows (both lane halves hold different rows): no cross-lane step
#pragma unroll
    for (int g = 0; g < G::kN32; g++) {
        if (j + 32 * g < tcols) {
#pragma unroll
            for (int q = 0; q < FR; q++) {
                if (bb0 + q < nb_blocks) {
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        partial[((int64_t)by * tcols + j + 32 * g) * nb_pad + (bb0 + q) * 32 + 8 * (r >> 2) + 4 * h + (r & 3)] =
                            out.g32[q][g][r];
                }
            }
        }
    }
    if constexpr (G::kH16 != 0) {
        // column lane % 16; registers 4 b + r and 4 (b + 2) + r together are output row 16 b + 4 (lane / 16) + r
        const int t = G::kOff16 + (lane & 15), mq = lane >> 4;
        if (t < tcols) {
#pragma unroll
            for (int q = 0; q < FR; q++) {
                if (bb0 + q < nb_blocks) {
#pragma unroll
                    for (int b = 0; b < 2; b++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            partial[((int64_t)by * tcols + t) * nb_pad + (bb0 + q) * 32 + 16 * b + 4 * mq + r] =
                                out.h16[q][4 * b + r] + out.h16[q][4 * (b + 2) + r];
                }
            }
        }
    }
    if constexpr (G::kQ8 != 0) {
        // lane l and lane l + 32 hold partial sums of output rows 4 ((l / 4) % 8) + r, column 4 u + l % 4
        const int t4 = G::kOff8 + (lane & 3), jb = 4 * ((lane >> 2) & 7);
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float sum = out.q8[q][u][r] + __shfl_xor(out.q8[q][u][r], 32);
                    if (lane < 32 && 4 * u + t4 < tcols && bb0 + q < nb_blocks)
                        partial[((int64_t)by * tcols + 4 * u + t4) * nb_pad + (bb0 + q) * 32 + jb + r] = sum;
                }
    }
}

}  // namespace flk
