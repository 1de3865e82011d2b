// Register-resident fp64 product kernel for many right-hand sides (up to 16 or 32 per pass), gfx950.
// Compiled once per kernel function (-DFLK_KF=0..4).
//
// Same walk as mmv_small_f64_kernel (a wave keeps FR blocks of 16 output rows in registers and streams blocks of 16
// reduction rows; K is never stored), but the contraction against vec runs on the matrix cores as well.  The fp64
// kernel value costs about a hundred cycles per lane (software exponential), so recomputing K for every four
// columns, as the FMA kernel does, is what many right-hand sides pay for; here 16 columns share one evaluation.
// Once the kernel values have replaced the exponents, accumulator register r of lane l (B position j = l % 16, A row
// 4 q + r, q = l / 16) is exactly the A operand of a 16x16x4 MFMA step whose B operand is vec[4 q + r][t = l % 16]:
//   out2[position 4 r2 + q][t] += sum_i K[i][j] vec[i][t],
// four more MFMAs per 16 x 16 tile whatever the number of columns, and register r2 of a lane ends up holding output
// row 4 q + r2 of column t (positions map to rows as in the packed block), so there is no cross-lane step.
// With NC = 2 a second group of 16 columns rides on the same kernel values (four more MFMAs per tile and group).
// Measured, dfmmv at N = 5e5, M = 2e4: 32 columns in one pass against two passes of 16: d = 9 35.1 ms against 49.1,
// d = 28 45.3 against 69.3, d = 64 69.2 against 116.7; 17 columns 35 / 45 / 69 ms against 39.1 / 58.9 / 106.6 for a
// 16-column pass followed by a one-column pass.  With NC = 4 (33 to 64 columns) the resident
// blocks per wave are halved (registers: 16 output accumulators per block and group).
#include "flk_common.h"
#include "kernel_fn.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

typedef double doublex4 __attribute__((ext_vector_type(4)));

constexpr int kWide64Waves = 4;
constexpr int kWide64Cols = 16;                             // one group of columns; NC groups share an evaluation of K
constexpr int kWide64MaxGroups = 4;
template <int NC> struct Wide64Geo {
    static constexpr int kCols = 16 * NC;
    static constexpr int kStride = kCols + 1;               // row stride of the staged vec values
    static constexpr int kStage = 16 + 16 * kStride;        // hn(16) | vec[16 rows][16 NC + 1]
    static constexpr bool kShared = NC >= 3;                // one stage per workgroup instead of one per wave (below)
    static constexpr int kFetch = kShared ? 1 + NC : 1 + kCols / 4;   // doubles a thread fetches per A block
};

template <int NC> struct Wide64RowVals { double x[Wide64Geo<NC>::kFetch]; };

template <int DP>
__device__ __forceinline__ void wide64_load_a(double (&a)[DP], const double *__restrict__ P, int64_t blk, int j, int q) {
    const double *p = P + (blk * (4 * DP) + (int64_t)q * DP) * 16 + j;
#pragma unroll
    for (int s = 0; s < DP; s++) a[s] = p[s * 16];
}

// lane l fetches hA[row l % 16] and vec[row l % 16][4c + l / 16], c = 0..4 NC - 1: 128-byte runs of the planes
template <int NC>
__device__ __forceinline__ void wide64_fetch(Wide64RowVals<NC> &rv, const double *__restrict__ hA,
                                             const double *__restrict__ vecp, int64_t vec_ld, int64_t ab, int lane) {
    const int r = lane & 15, hh = lane >> 4;
    rv.x[0] = hA[ab * 16 + r];
#pragma unroll
    for (int c = 0; c < Wide64Geo<NC>::kCols / 4; c++) rv.x[1 + c] = vecp[(int64_t)(4 * c + hh) * vec_ld + ab * 16 + r];
}
template <int NC>
__device__ __forceinline__ void wide64_stage(const Wide64RowVals<NC> &rv, double *lds, int lane) {
    const int r = lane & 15, hh = lane >> 4;
    if (hh == 0) lds[r] = rv.x[0];
#pragma unroll
    for (int c = 0; c < Wide64Geo<NC>::kCols / 4; c++) lds[16 + r * Wide64Geo<NC>::kStride + 4 * c + hh] = rv.x[1 + c];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// The row values of an A block (half norms and right-hand side entries) are the same for the four waves of a
// workgroup, which walk the same reduction chunk: the workgroup fetches them once, thread t the half norm of row
// t % 16 and the entries vec[row t % 16][t / 16 + 16 c], c = 0 .. NC - 1 (128-byte runs of the planes), and stages
// them in one LDS buffer that every wave reads its MFMA operands from, at the price of a workgroup barrier per A block.
// Used with four column groups, where a private copy per wave costs 17 loads per lane and block (dfmmv at N = 5e5,
// M = 2e4, 64 columns: d = 40 85.9 -> 75.8 ms, d = 64 105.1 -> 98.6); with one or two groups the private copies are as
// fast or faster (16 columns, d = 64: 58.4 ms against 61.2) and stay.
template <int NC>
__device__ __forceinline__ void wide64_fetch_wg(Wide64RowVals<NC> &rv, const double *__restrict__ hA,
                                             const double *__restrict__ vecp, int64_t vec_ld, int64_t ab, int tid) {
    const int r = tid & 15, p0 = tid >> 4;
    rv.x[0] = hA[ab * 16 + r];
#pragma unroll
    for (int c = 0; c < NC; c++) rv.x[1 + c] = vecp[(int64_t)(p0 + 16 * c) * vec_ld + ab * 16 + r];
}
template <int NC>
__device__ __forceinline__ void wide64_stage_wg(const Wide64RowVals<NC> &rv, double *lds, int tid) {
    const int r = tid & 15, p0 = tid >> 4;
    if (p0 == 0) lds[r] = rv.x[0];
#pragma unroll
    for (int c = 0; c < NC; c++) lds[16 + r * Wide64Geo<NC>::kStride + p0 + 16 * c] = rv.x[1 + c];
}
// Workgroup barrier that drains the wave's LDS traffic only (not its global loads, which are meant to stay in flight)
__device__ __forceinline__ void wide64_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int DP, int FR, int KF, int NC>
__device__ __forceinline__ void wide64_tile_step(const double (&a)[DP], const double *lds, int j, int q,
                                                 const double (&breg)[FR][DP], const double (&hb)[FR],
                                                 doublex4 (&out2)[FR][NC], const double *exp_tab) {
    constexpr int kWide64Stride = Wide64Geo<NC>::kStride;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const doublex4 hn = *(const doublex4 *)(lds + 4 * q);          // rows 4q .. 4q + 3 of the A block
    doublex4 acc[FR];
#pragma unroll
    for (int c = 0; c < FR; c++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[c][r] = hn[r] + hb[c];
#pragma unroll
    for (int s = 0; s < DP; s++)
#pragma unroll
        for (int c = 0; c < FR; c++) acc[c] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[s], breg[c][s], acc[c], 0, 0, 0);
#pragma unroll
    for (int c = 0; c < FR; c++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[c][r] = kernel_value<KF, (DP > 4)>(acc[c][r], exp_tab);
    const double *vb = lds + 16 + (4 * q) * kWide64Stride + j;     // vec[4q + r][t = j]
#pragma unroll
    for (int r = 0; r < 4; r++) {
#pragma unroll
        for (int g = 0; g < NC; g++) {
            const double bval = vb[r * kWide64Stride + 16 * g];
#pragma unroll
            for (int c = 0; c < FR; c++)
                out2[c][g] = __builtin_amdgcn_mfma_f64_16x16x4f64(acc[c][r], bval, out2[c][g], 0, 0, 0);
        }
    }
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int DP, int FR, int KF, int NC>
__global__ void __launch_bounds__(256, 2)
    mmv_small_f64_wide_kernel(const double *__restrict__ PA, const double *__restrict__ hA,
                              const double *__restrict__ vecp, int64_t vec_ld, const double *__restrict__ PB,
                              const double *__restrict__ hB, int64_t na_blocks, int64_t nb_blocks,
                              int64_t a_chunk_blocks, double *__restrict__ partial, int64_t nb_pad, int tcols,
                              bool y_fastest) {
    // vecp must hold 16 NC planes (zeros beyond the caller's columns); the first tcols columns are stored
    constexpr bool kShared = Wide64Geo<NC>::kShared;
    __shared__ __attribute__((aligned(32))) double stage[kShared ? 1 : kWide64Waves][2][Wide64Geo<NC>::kStage];
    // gfx950 has no fp64 exponential: 2^(k/2048) from a table in LDS, filled here (kernel_fn.h)
    __shared__ double exp_tab[kExpTableSize];
    exp2_table_fill(exp_tab, threadIdx.x, 256);
    __syncthreads();
    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int j = lane & 15, q = lane >> 4;
    const int jrow = 4 * (j & 3) + (j >> 2);  // matrix row (within its block) held at position j
    const int64_t bb0 = ((int64_t)bx * kWide64Waves + wave) * FR;
    // private stages: a wave whose blocks all lie past the end leaves (no workgroup barriers from here on); shared
    // stage: it keeps going on the last block, for the barriers, and stores nothing
    if (!kShared && bb0 >= nb_blocks) return;
    const int64_t a0 = (int64_t)by * a_chunk_blocks;
    int64_t a1 = a0 + a_chunk_blocks;
    if (a1 > na_blocks) a1 = na_blocks;

    double breg[FR][DP];
    double hb[FR];
#pragma unroll
    for (int c = 0; c < FR; c++) {
        const int64_t bb = bb0 + c < nb_blocks ? bb0 + c : nb_blocks - 1;
        wide64_load_a<DP>(breg[c], PB, bb, j, q);
        hb[c] = hB[bb * 16 + jrow];
    }
    doublex4 out2[FR][NC];
#pragma unroll
    for (int c = 0; c < FR; c++)
#pragma unroll
        for (int g = 0; g < NC; g++)
#pragma unroll
            for (int r = 0; r < 4; r++) out2[c][g][r] = 0.0;

    double fa0[DP], fa1[DP];
    Wide64RowVals<NC> rv;
    double *lds0 = stage[kShared ? 0 : wave][0], *lds1 = stage[kShared ? 0 : wave][1];
    if constexpr (kShared) {
        if (a0 < a1) {
            wide64_load_a<DP>(fa0, PA, a0, j, q);
            wide64_fetch_wg<NC>(rv, hA, vecp, vec_ld, a0, tid);
            wide64_stage_wg<NC>(rv, lds0, tid);
        }
        wide64_barrier();
        // One barrier per A block: a stage is written after the barrier that follows its last reader and read after
        // the barrier that follows its writers.  The conditions are the same for every wave of the workgroup.
        for (int64_t ab = a0; ab < a1; ab += 2) {
            const bool has1 = ab + 1 < a1;
            if (has1) { wide64_load_a<DP>(fa1, PA, ab + 1, j, q); wide64_fetch_wg<NC>(rv, hA, vecp, vec_ld, ab + 1, tid); }
            wide64_tile_step<DP, FR, KF, NC>(fa0, lds0, j, q, breg, hb, out2, exp_tab);
            if (has1) wide64_stage_wg<NC>(rv, lds1, tid);
            wide64_barrier();
            if (has1) {
                const bool has2 = ab + 2 < a1;
                if (has2) { wide64_load_a<DP>(fa0, PA, ab + 2, j, q); wide64_fetch_wg<NC>(rv, hA, vecp, vec_ld, ab + 2, tid); }
                wide64_tile_step<DP, FR, KF, NC>(fa1, lds1, j, q, breg, hb, out2, exp_tab);
                if (has2) wide64_stage_wg<NC>(rv, lds0, tid);
            }
            wide64_barrier();
        }
    } else {
        if (a0 < a1) {
            wide64_load_a<DP>(fa0, PA, a0, j, q);
            wide64_fetch<NC>(rv, hA, vecp, vec_ld, a0, lane);
            wide64_stage<NC>(rv, lds0, lane);
        }
        for (int64_t ab = a0; ab < a1; ab += 2) {
            const bool has1 = ab + 1 < a1;
            if (has1) { wide64_load_a<DP>(fa1, PA, ab + 1, j, q); wide64_fetch<NC>(rv, hA, vecp, vec_ld, ab + 1, lane); }
            wide64_tile_step<DP, FR, KF, NC>(fa0, lds0, j, q, breg, hb, out2, exp_tab);
            if (has1) {
                wide64_stage<NC>(rv, lds1, lane);
                const bool has2 = ab + 2 < a1;
                if (has2) { wide64_load_a<DP>(fa0, PA, ab + 2, j, q); wide64_fetch<NC>(rv, hA, vecp, vec_ld, ab + 2, lane); }
                wide64_tile_step<DP, FR, KF, NC>(fa1, lds1, j, q, breg, hb, out2, exp_tab);
                if (has2) wide64_stage<NC>(rv, lds0, lane);
            }
        }
    }
    // lane = column t = j, registers = output rows 4q .. 4q + 3 of each block
#pragma unroll
    for (int g = 0; g < NC; g++) {
        if (j + 16 * g < tcols) {
#pragma unroll
            for (int c = 0; c < FR; c++)
                if (bb0 + c < nb_blocks)
                    *(doublex4 *)(&partial[((int64_t)by * tcols + j + 16 * g) * nb_pad + (bb0 + c) * 16 + 4 * q]) = out2[c][g];
        }
    }
}

template <int DP, int FR, int NC>
static int launch_wide64_one(const PackedView &A, const PackedView &B, const double *vecp, int64_t vec_ld, int tcols,
                             int64_t a_chunk_blocks, int splits, double *partial, hipStream_t st) {
    const int64_t per_wg = kWide64Waves * FR;
    dim3 grid((unsigned)((B.nblk + per_wg - 1) / per_wg), (unsigned)splits);
    hipLaunchKernelGGL((mmv_small_f64_wide_kernel<DP, FR, FLK_KF, NC>), grid, dim3(256), 0, st, (const double *)A.data,
                       (const double *)A.hnorm, vecp, vec_ld, (const double *)B.data, (const double *)B.hnorm, A.nblk,
                       B.nblk, a_chunk_blocks, partial, B.npad, tcols, B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_small_f64_wide_kernel");
    return FLK_OK;
}

int FLK_CAT(launch_mmv_small_f64_wide_kf, FLK_KF)(const PackedView &A, const PackedView &B, const double *vecp,
                                                  int64_t vec_ld, int tcols, int64_t a_chunk_blocks, int splits,
                                                  double *partial, hipStream_t st) {
    if (tcols < 1 || tcols > kWide64Cols * kWide64MaxGroups)
        return fail(FLK_EINVAL, "mmv_small wide: column chunk %d not in 1..64", tcols);
    if (A.dpad != B.dpad) return fail(FLK_EINVAL, "mmv_small: operands packed with different feature counts");
    const int dp = (int)(A.dpad / 4);
#define FLK_WIDE64(DPV, FRV)                                                                                             \
    case DPV:                                                                                                           \
        if (tcols > 3 * kWide64Cols)                                                                                    \
            return launch_wide64_one<DPV, (FRV) / 2, 4>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st); \
        if (tcols > 2 * kWide64Cols)                                                                                    \
            return launch_wide64_one<DPV, (FRV) / 2, 3>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st); \
        return tcols > kWide64Cols                                                                                      \
                   ? launch_wide64_one<DPV, FRV, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st)     \
                   : launch_wide64_one<DPV, FRV, 1>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
    switch (dp) {
        FLK_WIDE64(1, 4) FLK_WIDE64(2, 4) FLK_WIDE64(3, 4) FLK_WIDE64(4, 4) FLK_WIDE64(5, 4) FLK_WIDE64(6, 4)
        FLK_WIDE64(7, 4) FLK_WIDE64(8, 4) FLK_WIDE64(9, 2) FLK_WIDE64(10, 2) FLK_WIDE64(11, 2) FLK_WIDE64(12, 2)
        FLK_WIDE64(13, 2) FLK_WIDE64(14, 2) FLK_WIDE64(15, 2) FLK_WIDE64(16, 2)
    }
#undef FLK_WIDE64
    return fail(FLK_EUNSUPPORTED, "mmv_small wide<f64>: padded feature count %lld not in 4..64", (long long)A.dpad);
}

}  // namespace flk
