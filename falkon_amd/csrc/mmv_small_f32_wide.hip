// Register-resident fp32 product kernel for many right-hand sides (up to 32 or 64 per pass), gfx950.
// Compiled once per kernel function (-DFLK_KF=0..4).
//
// Same walk as mmv_small_f32_kernel (a wave keeps FR blocks of 32 output rows in registers and streams blocks of 32
// reduction rows; K is never stored), but the contraction against vec runs on the matrix cores as well: once the
// kernel values have replaced the exponents in the accumulator registers, register s of a lane is exactly the A
// operand of an fp32 32x32x2 MFMA step (row i = 8*(s/4) + 4*(lane/32) + s%4 of the A block, column j = lane % 32),
// so  out2[j][t] += sum_i K[i][j] vec[i][t]  is 16 more MFMAs per fragment whatever the number of columns, with
// vec[i][t] (t = lane % 32) as the B operand.  Per-lane FMAs cost 16 per column and fragment: beyond eight columns
// (four for the two-fragment kernels) this kernel is the cheaper one.  NC = 2 serves 64 columns per evaluation of K
// (two groups of 32, 32 contraction MFMAs per fragment, two resident fragments per wave): between 33 and 64 columns
// the cross term and the exponential are then computed once instead of twice.
#include "mmv_small_f32_kernel.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

// NC groups of 32 columns: the staged values of an A block are hn(32) | vec[32 rows][columns + 1] (the odd row stride
// makes the reads conflict free)
// (NC = 0 stands for the 16-column form, one half group, and NC = -1 for the 8-column form)
template <int NC> struct WideGeo {
    static constexpr int kCols = NC == -1 ? 8 : NC == 0 ? 16 : 32 * NC;
    static constexpr int kStride = kCols + 1;
    static constexpr int kStage = 32 + 32 * kStride;
    static constexpr int kFetch = 1 + kCols / 8;         // dwords a thread fetches per A block
};
constexpr int kWideCols = 32;                            // of one group
constexpr int kWideHalfCols = 16;                        // of the 16-column form
constexpr int kWideNarrowCols = 8;                       // of the 8-column form

// Output accumulators of a resident block: one 16-register set per group of 32 columns (one for the 16-column form);
// the 8-column form keeps two sets of four registers (columns 0 .. 3 and 4 .. 7)
template <int NC> struct WideOut {
    typedef floatx16 type;
    static constexpr int kSets = NC == 0 ? 1 : NC;
    static constexpr int kRegs = 16;
};
template <> struct WideOut<-1> {
    typedef floatx4 type;
    static constexpr int kSets = 2;
    static constexpr int kRegs = 4;
};
constexpr int kWideMaxGroups = 2;

template <int NC> struct WideRowVals { float x[WideGeo<NC>::kFetch]; };

// The row values of an A block (half norms and right-hand side entries) are the same for the four waves of a
// workgroup, which walk the same reduction chunk: the workgroup fetches them once, thread t the half norm of row
// t % 32 and the entries vec[row t % 32][t / 32 + 8 c], c = 0 .. 4 NC - 1 (128-byte runs of the planes), and stages
// them in one LDS buffer that every wave reads its MFMA operands from.  (With a private copy per wave the 16 NC + 1
// loads per lane and block cost 9 % of the launch: N = 1e6, M = 2e4, d = 28, 32 columns, 21.3 ms against 19.4 with
// those loads removed.)
template <int NC>
__device__ __forceinline__ void wide_fetch(WideRowVals<NC> &rv, const float *__restrict__ hA,
                                           const float *__restrict__ vecp, int64_t vec_ld, int64_t ab, int tid) {
    const int r = tid & 31, p0 = tid >> 5;
    rv.x[0] = hA[ab * 32 + r];
#pragma unroll
    for (int c = 0; c < WideGeo<NC>::kCols / 8; c++) rv.x[1 + c] = vecp[(int64_t)(p0 + 8 * c) * vec_ld + ab * 32 + r];
}
template <int NC>
__device__ __forceinline__ void wide_stage(const WideRowVals<NC> &rv, float *lds, int tid) {
    const int r = tid & 31, p0 = tid >> 5;
    if (p0 == 0) lds[r] = rv.x[0];
#pragma unroll
    for (int c = 0; c < WideGeo<NC>::kCols / 8; c++) lds[32 + r * WideGeo<NC>::kStride + p0 + 8 * c] = rv.x[1 + c];
}
// Workgroup barrier that drains the wave's LDS traffic only (not its global loads, which are meant to stay in flight)
__device__ __forceinline__ void wide_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int DP, int FR, bool FOLD, int KF, int NC>
__device__ __forceinline__ void wide_tile_step(const float (&a)[DP], const float *lds, int j, int h,
                                               const float (&breg)[FR][DP], const float (&hb)[FR],
                                               typename WideOut<NC>::type (&out2)[FR][WideOut<NC>::kSets]) {
    constexpr int kWideStride = WideGeo<NC>::kStride;
    floatx4 hn[4];
#pragma unroll
    for (int g = 0; g < 4; g++) hn[g] = *(const floatx4 *)(lds + 8 * g + 4 * h);
    floatx16 acc[FR];
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[q][r] = FOLD ? hn[r >> 2][r & 3] : hn[r >> 2][r & 3] + hb[q];
#pragma unroll
    for (int s = 0; s < DP; s++)
#pragma unroll
        for (int q = 0; q < FR; q++) acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], breg[q][s], acc[q], 0, 0, 0);
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[q][r] = kernel_value<KF>(acc[q][r]);
    // All kernel values first, then the contraction: left alone the compiler sinks every v_exp_f32 to just in front of
    // the MFMA that consumes it, and each of those MFMAs then waits for the exponential's result.
    __builtin_amdgcn_sched_barrier(0);
    // contraction on the matrix cores; the B operand is read one step ahead, fenced (otherwise every read is
    // hoisted to the front)
    if constexpr (NC == -1) {
        // Up to 8 columns: two 16-block 4x4x1 steps (8 cycles each; the 16x16x1 step below takes 32, 16 per-lane FMAs per
        // column 64).  As A operand, register s2 of lane l is K[i][j] with j = l % 32 and i the row of step s2 in lane
        // half h: block b = l / 4 holds the output rows 4 (b % 8) .. + 3 against that row of half b / 8.  The B operand
        // of block b is vec[that row][4 u + l % 4] for the column set u, and output (row 4 (b % 8) + r, column
        // 4 u + l % 4) accumulates in register r of set u in lane l: the two lane halves hold partial sums of the
        // same outputs, added at the store.
        const float *vb = lds + 32 + (j & 3);
        float bval[2] = {vb[(4 * h) * kWideStride], vb[(4 * h) * kWideStride + 4]}, bnext[2] = {0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < 16; s2++) {
            if (s2 + 1 < 16) {
#pragma unroll
                for (int u = 0; u < 2; u++)
                    bnext[u] = vb[(8 * ((s2 + 1) >> 2) + 4 * h + ((s2 + 1) & 3)) * kWideStride + 4 * u];
            }
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int q = 0; q < FR; q++)
                    out2[q][u] = __builtin_amdgcn_mfma_f32_4x4x1f32(acc[q][s2], bval[u], out2[q][u], 0, 0, 0);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                asm volatile("" : "+v"(bval[u]) : "v"(vb) : "memory");
                bval[u] = bnext[u];
            }
        }
    } else if constexpr (NC == 0) {
        // Up to 16 columns: the four-block 16x16x1 step, half the cycles of a 32x32x2 step that would leave half of its
        // columns unused.  Its blocks are the lane quarters: as A operand, register s2 of lane l is K[i][j] with
        // j = l % 32 and i the row of step s2 in lane half h, i.e. block b = l / 16 holds the output rows 16 (b & 1) ..
        // + 15 against row i of half b >> 1; the B operand of block b is vec[that row][t = l % 16], which is what the
        // lanes of that quarter read.  Block b accumulates in registers 4 b .. 4 b + 3 (output row 16 (b & 1) +
        // 4 (lane / 16) + r, column lane % 16): blocks b and b + 2 are partial sums of the same outputs.
        const float *vb = lds + 32 + (j & 15);
        float bval = vb[(4 * h) * kWideStride], bnext = 0.f;
#pragma unroll
        for (int s2 = 0; s2 < 16; s2++) {
            if (s2 + 1 < 16) bnext = vb[(8 * ((s2 + 1) >> 2) + 4 * h + ((s2 + 1) & 3)) * kWideStride];
#pragma unroll
            for (int q = 0; q < FR; q++)
                out2[q][0] = __builtin_amdgcn_mfma_f32_16x16x1f32(acc[q][s2], bval, out2[q][0], 0, 0, 0);
            asm volatile("" : "+v"(bval) : "v"(vb) : "memory");
            bval = bnext;
        }
    } else {
        const float *vb = lds + 32 + j;
        float bval[NC], bnext[NC];
#pragma unroll
        for (int g = 0; g < NC; g++) { bval[g] = vb[(4 * h) * kWideStride + 32 * g]; bnext[g] = 0.f; }
#pragma unroll
        for (int s2 = 0; s2 < 16; s2++) {
            if (s2 + 1 < 16) {
#pragma unroll
                for (int g = 0; g < NC; g++)
                    bnext[g] = vb[(8 * ((s2 + 1) >> 2) + 4 * h + ((s2 + 1) & 3)) * kWideStride + 32 * g];
            }
#pragma unroll
            for (int g = 0; g < NC; g++)
#pragma unroll
                for (int q = 0; q < FR; q++)
                    out2[q][g] = __builtin_amdgcn_mfma_f32_32x32x2f32(acc[q][s2], bval[g], out2[q][g], 0, 0, 0);
#pragma unroll
            for (int g = 0; g < NC; g++) {
                asm volatile("" : "+v"(bval[g]) : "v"(vb) : "memory");
                bval[g] = bnext[g];
            }
        }
    }
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int DP, int FR, bool FOLD, int KF, int NC>
__global__ void __launch_bounds__(256, 2)
    mmv_small_f32_wide_kernel(const float *__restrict__ PA, const float *__restrict__ hA, const float *__restrict__ vecp,
                              int64_t vec_ld, const float *__restrict__ PB, const float *__restrict__ hB,
                              int64_t na_blocks, int64_t nb_blocks, int64_t a_chunk_blocks, float *__restrict__ partial,
                              int64_t nb_pad, int tcols, bool y_fastest) {
    // vecp must hold 32 NC planes (16 for NC = 0, 8 for NC = -1; zeros beyond the caller's columns); the first tcols
    // columns are stored
    __shared__ __attribute__((aligned(16))) float stage[2][WideGeo<NC>::kStage];   // shared by the four waves
    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int j = lane & 31, h = lane >> 5;
    // (a wave whose blocks all lie past the end keeps going on the last block, for the barriers; it stores nothing)
    const int64_t bb0 = ((int64_t)bx * kWavesPerWg + wave) * FR;
    const int64_t a0 = (int64_t)by * a_chunk_blocks;
    int64_t a1 = a0 + a_chunk_blocks;
    if (a1 > na_blocks) a1 = na_blocks;

    float breg[FR][DP];
    float hb[FR];
#pragma unroll
    for (int q = 0; q < FR; q++) {
        int64_t bb = bb0 + q < nb_blocks ? bb0 + q : nb_blocks - 1;
        load_a<DP>(breg[q], PB, bb, j, h);
        hb[q] = hB[bb * 32 + j];
        if (FOLD) breg[q][DP - 1] = h ? hb[q] : breg[q][DP - 1];
    }
    typename WideOut<NC>::type out2[FR][WideOut<NC>::kSets];
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int g = 0; g < WideOut<NC>::kSets; g++)
#pragma unroll
            for (int r = 0; r < WideOut<NC>::kRegs; r++) out2[q][g][r] = 0.f;

    float fa0[DP], fa1[DP];
    WideRowVals<NC> rv;
    float *lds0 = stage[0], *lds1 = stage[1];
    if (a0 < a1) {
        load_a<DP>(fa0, PA, a0, j, h);
        wide_fetch<NC>(rv, hA, vecp, vec_ld, a0, tid);
        wide_stage<NC>(rv, lds0, tid);
    }
    wide_barrier();
    // One barrier per A block: a stage is written after the barrier that follows its last reader and read after the
    // barrier that follows its writers.  The conditions are the same for every wave of the workgroup.
    for (int64_t ab = a0; ab < a1; ab += 2) {
        const bool has1 = ab + 1 < a1;
        if (has1) { load_a<DP>(fa1, PA, ab + 1, j, h); wide_fetch<NC>(rv, hA, vecp, vec_ld, ab + 1, tid); }
        wide_tile_step<DP, FR, FOLD, KF, NC>(fa0, lds0, j, h, breg, hb, out2);
        if (has1) wide_stage<NC>(rv, lds1, tid);
        wide_barrier();
        if (has1) {
            const bool has2 = ab + 2 < a1;
            if (has2) { load_a<DP>(fa0, PA, ab + 2, j, h); wide_fetch<NC>(rv, hA, vecp, vec_ld, ab + 2, tid); }
            wide_tile_step<DP, FR, FOLD, KF, NC>(fa1, lds1, j, h, breg, hb, out2);
            if (has2) wide_stage<NC>(rv, lds0, tid);
        }
        wide_barrier();
    }
    if constexpr (NC == -1) {
        // lane l and lane l + 32 hold partial sums of output rows 4 ((l / 4) % 8) + r, column 4 u + l % 4
        const int t4 = lane & 3, jb = 4 * ((lane >> 2) & 7);
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float sum = out2[q][u][r] + __shfl_xor(out2[q][u][r], 32);
                    if (lane < 32 && 4 * u + t4 < tcols && bb0 + q < nb_blocks)
                        partial[((int64_t)by * tcols + 4 * u + t4) * nb_pad + (bb0 + q) * 32 + jb + r] = sum;
                }
    } else if constexpr (NC == 0) {
        // lane = column t = lane % 16; registers 4 b + r and 4 (b + 2) + r together are output row 16 b + 4 (lane / 16) + r
        const int t = lane & 15, mq = lane >> 4;
        if (t < tcols) {
#pragma unroll
            for (int q = 0; q < FR; q++) {
                if (bb0 + q < nb_blocks) {
#pragma unroll
                    for (int b = 0; b < 2; b++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            partial[((int64_t)by * tcols + t) * nb_pad + (bb0 + q) * 32 + 16 * b + 4 * mq + r] =
                                out2[q][0][4 * b + r] + out2[q][0][4 * (b + 2) + r];
                }
            }
        }
    } else {
        // lane = column t, registers = output rows (both lane halves hold different rows): no cross-lane step
#pragma unroll
        for (int g = 0; g < NC; g++) {
            if (j + 32 * g < tcols) {
#pragma unroll
                for (int q = 0; q < FR; q++) {
                    if (bb0 + q < nb_blocks) {
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            partial[((int64_t)by * tcols + j + 32 * g) * nb_pad + (bb0 + q) * 32 + 8 * (r >> 2) + 4 * h + (r & 3)] =
                                out2[q][g][r];
                    }
                }
            }
        }
    }
}

template <int DP, int FR, bool FOLD, int NC = 1>
static int launch_wide_one(const PackedView &A, const PackedView &B, const float *vecp, int64_t vec_ld, int tcols,
                           int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
    const int64_t per_wg = kWavesPerWg * FR;
    dim3 grid((unsigned)((B.nblk + per_wg - 1) / per_wg), (unsigned)splits);
    hipLaunchKernelGGL((mmv_small_f32_wide_kernel<DP, FR, FOLD, FLK_KF, NC>), grid, dim3(256), 0, st, (const float *)A.data,
                       (const float *)A.hnorm, vecp, vec_ld, (const float *)B.data, (const float *)B.hnorm, A.nblk,
                       B.nblk, a_chunk_blocks, partial, B.npad, tcols, B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_small_f32_wide_kernel");
    return FLK_OK;
}

int FLK_CAT(launch_mmv_small_f32_wide_kf, FLK_KF)(const PackedView &A, const PackedView &B, const float *vecp,
                                                  int64_t vec_ld, int tcols, int64_t a_chunk_blocks, int splits,
                                                  float *partial, hipStream_t st) {
    if (tcols < 1 || tcols > kWideCols * kWideMaxGroups)
        return fail(FLK_EINVAL, "mmv_small wide: column chunk %d not in 1..64", tcols);
    const int dp = (int)(A.dpad / 2);
    const bool fold = f32_fold_applies(A.d);
    if (tcols > kWideCols) {
        // 33 to 64 columns: two groups of 32 on one evaluation of K; two resident fragments per wave (64 output
        // accumulators per fragment; from 56 padded features on a few registers spill, which still beats one fragment:
        // d = 64, 64 columns: 84.3 ms per dfmmv against 84.9, d = 40: 67.3 against 73.8)
#define FLK_WIDE2(DPV)                                                                                              \
    case DPV:                                                                                                      \
        return fold ? launch_wide_one<DPV, 2, true, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st) \
                    : launch_wide_one<DPV, 2, false, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
#define FLK_WIDE2_PLAIN(DPV) \
    case DPV: return launch_wide_one<DPV, 2, false, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        switch (dp) {
            FLK_WIDE2(1) FLK_WIDE2(2) FLK_WIDE2(3) FLK_WIDE2(4) FLK_WIDE2(5) FLK_WIDE2(6) FLK_WIDE2(7) FLK_WIDE2(8)
            FLK_WIDE2(9) FLK_WIDE2(10) FLK_WIDE2(11) FLK_WIDE2(12) FLK_WIDE2(13) FLK_WIDE2(14) FLK_WIDE2(15) FLK_WIDE2(16)
            FLK_WIDE2_PLAIN(17) FLK_WIDE2_PLAIN(18) FLK_WIDE2_PLAIN(19) FLK_WIDE2_PLAIN(20) FLK_WIDE2_PLAIN(21)
            FLK_WIDE2_PLAIN(22) FLK_WIDE2_PLAIN(23) FLK_WIDE2_PLAIN(24) FLK_WIDE2_PLAIN(25) FLK_WIDE2_PLAIN(26)
            FLK_WIDE2_PLAIN(27) FLK_WIDE2_PLAIN(28) FLK_WIDE2_PLAIN(29) FLK_WIDE2_PLAIN(30) FLK_WIDE2_PLAIN(31)
            FLK_WIDE2_PLAIN(32)
        }
#undef FLK_WIDE2
#undef FLK_WIDE2_PLAIN
        return fail(FLK_EUNSUPPORTED, "mmv_small wide: padded feature count %lld not in 2..64", (long long)A.dpad);
    }
    // up to 8 columns: the 8-column form (vecp holds 8 planes); up to 16: the 16-column form (16 planes); 17 to 32: one
    // group of 32
    const bool half = tcols <= kWideHalfCols, narrow = tcols <= kWideNarrowCols;
#define FLK_WIDE_ONE(DPV, FRV, FOLDV)                                                                              \
    (narrow ? launch_wide_one<DPV, FRV, FOLDV, -1>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st)  \
     : half ? launch_wide_one<DPV, FRV, FOLDV, 0>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st)   \
            : launch_wide_one<DPV, FRV, FOLDV, 1>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st))
#define FLK_WIDE(DPV, FRV) \
    case DPV: return fold ? FLK_WIDE_ONE(DPV, FRV, true) : FLK_WIDE_ONE(DPV, FRV, false);
#define FLK_WIDE_PLAIN(DPV, FRV) \
    case DPV: return FLK_WIDE_ONE(DPV, FRV, false);
    switch (dp) {
        FLK_WIDE(1, 4) FLK_WIDE(2, 4) FLK_WIDE(3, 4) FLK_WIDE(4, 4) FLK_WIDE(5, 4) FLK_WIDE(6, 4) FLK_WIDE(7, 4)
        FLK_WIDE(8, 4) FLK_WIDE(9, 2) FLK_WIDE(10, 2) FLK_WIDE(11, 2) FLK_WIDE(12, 2) FLK_WIDE(13, 2) FLK_WIDE(14, 2)
        FLK_WIDE(15, 2) FLK_WIDE(16, 2)
        FLK_WIDE_PLAIN(17, 2) FLK_WIDE_PLAIN(18, 2) FLK_WIDE_PLAIN(19, 2) FLK_WIDE_PLAIN(20, 2) FLK_WIDE_PLAIN(21, 2)
        FLK_WIDE_PLAIN(22, 2) FLK_WIDE_PLAIN(23, 2) FLK_WIDE_PLAIN(24, 2) FLK_WIDE_PLAIN(25, 2) FLK_WIDE_PLAIN(26, 2)
        FLK_WIDE_PLAIN(27, 2) FLK_WIDE_PLAIN(28, 2) FLK_WIDE_PLAIN(29, 2) FLK_WIDE_PLAIN(30, 2) FLK_WIDE_PLAIN(31, 2)
        FLK_WIDE_PLAIN(32, 2)
    }
#undef FLK_WIDE
#undef FLK_WIDE_PLAIN
#undef FLK_WIDE_ONE
    return fail(FLK_EUNSUPPORTED, "mmv_small wide: padded feature count %lld not in 2..64", (long long)A.dpad);
}

}  // namespace flk
