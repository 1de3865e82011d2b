// Register-resident fp32 product kernel for many right-hand sides (8 to 64 per pass), gfx950.
// Compiled once per kernel function (-DFLK_KF=0..4).
//
// Same walk as mmv_small_f32_kernel (a wave keeps FR blocks of 32 output rows in registers and streams blocks of 32
// reduction rows; K is never stored), but the contraction against vec runs on the matrix cores as well: once the
// kernel values have replaced the exponents in the accumulator registers, register s of a lane is exactly the A
// operand of an fp32 MFMA step (row i = 8*(s/4) + 4*(lane/32) + s%4 of the A block, column j = lane % 32), so
// out[j][t] += sum_i K[i][j] vec[i][t]  is 16 more steps per fragment, with vec[i][t] as the B operand.  The columns of
// a pass are served by up to three kinds of step that share the kernel values:
//   groups of 32 columns, the 32x32x2 step (64 cycles): t = lane % 32, each lane ends up with 16 output rows of one
//     column;
//   one group of 16, the four-block 16x16x1 step (32 cycles): block b = lane / 16 pairs the output rows 16 (b & 1) ..
//     + 15 with the row of lane half b >> 1, its B operand is vec[that row][lane % 16], which is what the lanes of that
//     quarter read, and it accumulates in registers 4 b .. 4 b + 3 (output row 16 (b & 1) + 4 (lane / 16) + r, column
//     lane % 16): blocks b and b + 2 are partial sums of the same outputs, added at the store;
//   one group of 8, two 16-block 4x4x1 steps (8 cycles each): block b = lane / 4 pairs the output rows 4 (b % 8) .. + 3
//     with the row of lane half b / 8, the B operand is vec[that row][4 u + lane % 4] for the column set u, and output
//     (row 4 (b % 8) + r, column 4 u + lane % 4) accumulates in register r of set u: the two lane halves hold partial
//     sums of the same outputs, added at the store.
// A pass takes 8, 16, 24, 32, 40, 48 or 64 columns: 32 N32 + 16 H16 + 8 Q8.  Per-lane FMAs cost 16 per column and
// fragment: beyond four to six columns this kernel is the cheaper one.
#include "mmv_small_f32_kernel.h"
#include "mmv_wide_common.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

template <int DP, int FR, bool FOLD, int KF, int COLS>
__device__ __forceinline__ void wide_tile_step(const float (&a)[DP], const float *lds, int j, int h,
                                               const float (&breg)[FR][DP], const float (&hb)[FR],
                                               WideAcc<FR, COLS> &out) {
    using G = WideGeo<COLS>;
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
    wide_contract<FR, COLS>(acc, lds, j, h, out);
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int DP, int FR, bool FOLD, int KF, int COLS>
__global__ void __launch_bounds__(256, 2)
    mmv_small_f32_wide_kernel(const float *__restrict__ PA, const float *__restrict__ hA, const float *__restrict__ vecp,
                              int64_t vec_ld, const float *__restrict__ PB, const float *__restrict__ hB,
                              int64_t na_blocks, int64_t nb_blocks, int64_t a_chunk_blocks, float *__restrict__ partial,
                              int64_t nb_pad, int tcols, bool y_fastest) {
    using G = WideGeo<COLS>;
    // vecp must hold COLS planes (zeros beyond the caller's columns); the first tcols columns are stored
    __shared__ __attribute__((aligned(16))) float stage[2][G::kStage];   // shared by the four waves
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
    WideAcc<FR, COLS> out;
    wide_zero<FR, COLS>(out);

    float fa0[DP], fa1[DP];
    WideRowVals<COLS> rv;
    float *lds0 = stage[0], *lds1 = stage[1];
    if (a0 < a1) {
        load_a<DP>(fa0, PA, a0, j, h);
        wide_fetch<COLS>(rv, hA, vecp, vec_ld, a0, tid);
        wide_stage<COLS>(rv, lds0, tid);
    }
    wide_barrier();
    // One barrier per A block: a stage is written after the barrier that follows its last reader and read after the
    // barrier that follows its writers.  The conditions are the same for every wave of the workgroup.
    for (int64_t ab = a0; ab < a1; ab += 2) {
        const bool has1 = ab + 1 < a1;
        if (has1) { load_a<DP>(fa1, PA, ab + 1, j, h); wide_fetch<COLS>(rv, hA, vecp, vec_ld, ab + 1, tid); }
        wide_tile_step<DP, FR, FOLD, KF, COLS>(fa0, lds0, j, h, breg, hb, out);
        if (has1) wide_stage<COLS>(rv, lds1, tid);
        wide_barrier();
        if (has1) {
            const bool has2 = ab + 2 < a1;
            if (has2) { load_a<DP>(fa0, PA, ab + 2, j, h); wide_fetch<COLS>(rv, hA, vecp, vec_ld, ab + 2, tid); }
            wide_tile_step<DP, FR, FOLD, KF, COLS>(fa1, lds1, j, h, breg, hb, out);
            if (has2) wide_stage<COLS>(rv, lds0, tid);
        }
        wide_barrier();
    }

    wide_store<FR, COLS>(out, partial, by, tcols, nb_pad, bb0, nb_blocks, lane);
}

template <int DP, int FR, bool FOLD, int COLS>
static int launch_wide_one(const PackedView &A, const PackedView &B, const float *vecp, int64_t vec_ld, int tcols,
                           int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
    const int64_t per_wg = kWavesPerWg * FR;
    dim3 grid((unsigned)((B.nblk + per_wg - 1) / per_wg), (unsigned)splits);
    hipLaunchKernelGGL((mmv_small_f32_wide_kernel<DP, FR, FOLD, FLK_KF, COLS>), grid, dim3(256), 0, st, (const float *)A.data,
                       (const float *)A.hnorm, vecp, vec_ld, (const float *)B.data, (const float *)B.hnorm, A.nblk,
                       B.nblk, a_chunk_blocks, partial, B.npad, tcols, B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_small_f32_wide_kernel");
    return FLK_OK;
}

template <int DP, bool FOLD>
static int launch_wide_dp(const PackedView &A, const PackedView &B, const float *vecp, int64_t vec_ld, int tcols,
                          int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
#define FLK_WIDE_FORM(COLSV)                                                                                     \
    case COLSV:                                                                                                  \
        return launch_wide_one<DP, wide_blocks_per_wave(DP, COLSV), FOLD, COLSV>(A, B, vecp, vec_ld, tcols,       \
                                                                                 a_chunk_blocks, splits, partial, st);
    switch (wide_form_cols(tcols)) {
        FLK_WIDE_FORM(8) FLK_WIDE_FORM(16) FLK_WIDE_FORM(24) FLK_WIDE_FORM(32) FLK_WIDE_FORM(40) FLK_WIDE_FORM(48)
        FLK_WIDE_FORM(64)
    }
#undef FLK_WIDE_FORM
    return fail(FLK_EINVAL, "mmv_small wide: column chunk %d not in 1..64", tcols);
}

int FLK_CAT(launch_mmv_small_f32_wide_kf, FLK_KF)(const PackedView &A, const PackedView &B, const float *vecp,
                                                  int64_t vec_ld, int tcols, int64_t a_chunk_blocks, int splits,
                                                  float *partial, hipStream_t st) {
    if (tcols < 1 || tcols > kWideMaxCols)
        return fail(FLK_EINVAL, "mmv_small wide: column chunk %d not in 1..64", tcols);
    const int dp = (int)(A.dpad / 2);
    const bool fold = f32_fold_applies(A.d);
#define FLK_WIDE(DPV)                                                                                        \
    case DPV:                                                                                                \
        return fold ? launch_wide_dp<DPV, true>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st) \
                    : launch_wide_dp<DPV, false>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
#define FLK_WIDE_PLAIN(DPV) \
    case DPV: return launch_wide_dp<DPV, false>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
    switch (dp) {
        FLK_WIDE(1) FLK_WIDE(2) FLK_WIDE(3) FLK_WIDE(4) FLK_WIDE(5) FLK_WIDE(6) FLK_WIDE(7) FLK_WIDE(8)
        FLK_WIDE(9) FLK_WIDE(10) FLK_WIDE(11) FLK_WIDE(12) FLK_WIDE(13) FLK_WIDE(14) FLK_WIDE(15) FLK_WIDE(16)
        FLK_WIDE_PLAIN(17) FLK_WIDE_PLAIN(18) FLK_WIDE_PLAIN(19) FLK_WIDE_PLAIN(20) FLK_WIDE_PLAIN(21)
        FLK_WIDE_PLAIN(22) FLK_WIDE_PLAIN(23) FLK_WIDE_PLAIN(24) FLK_WIDE_PLAIN(25) FLK_WIDE_PLAIN(26)
        FLK_WIDE_PLAIN(27) FLK_WIDE_PLAIN(28) FLK_WIDE_PLAIN(29) FLK_WIDE_PLAIN(30) FLK_WIDE_PLAIN(31)
        FLK_WIDE_PLAIN(32)
    }
#undef FLK_WIDE
#undef FLK_WIDE_PLAIN
    return fail(FLK_EUNSUPPORTED, "mmv_small wide: padded feature count %lld not in 2..64", (long long)A.dpad);
}

}  // namespace flk
