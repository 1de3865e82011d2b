// Register-resident kernel-vector product of the bf16x3 mode for many right-hand sides (5 to 64 per pass), fp32 data,
// up to 62 features (four k-steps), gfx950.  Compiled once per kernel function (-DFLK_KF=0..4).
//
//   partial[split][t][b] = sum_{a in chunk(split)} K(A_a, B_b) * vec[a,t]
//
// The cross term of a 32 x 32 tile is the bf16x3 chain of mmv_split.hip (6 KS v_mfma_f32_32x32x16_bf16 on the split
// operands, the half norms riding in the last two features: the accumulator starts from zero and ends as the
// exponent); the contraction against vec is that of mmv_small_f32_wide.hip (mmv_wide_common.h): the kernel values in
// the accumulator registers are the A operand of fp32 32x32x2, 16x16x1 and 4x4x1 steps whose B operand comes from a
// stage of the A block's right-hand sides that the four waves of the workgroup share.  The bf16 chains run on the
// matrix cores beside the fp32 instructions (the exponentials and the fp32 contraction steps of the other wave of the
// SIMD), so a pass costs about what its exponentials and its contraction cost.  The contraction itself stays on the
// fp32 steps at every width: done on the bf16 matrix cores as well (kernel values and right-hand sides split three
// ways) it was a third faster at 32 and 64 columns, but a column whose terms cancel came out a digit further from the
// fp64 result than with the fp32 steps (1.4e-5 against 1.6e-6 for a 200-fold cancellation), which is not the accuracy
// this mode promises.
#include "kernel_fn.h"
#include "split_common.h"
#include "mmv_wide_common.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int kSplitWideWaves = 4;

template <int KS> struct SplitWideFrag { uintx4 p[KS][3]; };

template <int KS>
__device__ __forceinline__ void load_split_wide(SplitWideFrag<KS> &f, const uintx4 *__restrict__ P, int64_t blk, int lane) {
    const uintx4 *p = P + (blk * KS * 3) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int c = 0; c < 3; c++) f.p[ks][c] = p[(ks * 3 + c) * 64];
}

// The right-hand sides of an A block: thread t fetches vec[row t % 32][t / 32 + 8 c], c = 0 .. COLS / 8 - 1 (128-byte runs
// of the planes; zero beyond the caller's columns: vecp holds tcols planes only), and stages them at the layout of
// mmv_wide_common.h (whose first 32 words, the half norms of the fp32 kernel, stay unused here)
template <int COLS> struct SplitWideRowVals { float x[COLS / 8]; };
template <int COLS>
__device__ __forceinline__ void split_wide_fetch(SplitWideRowVals<COLS> &rv, const float *__restrict__ vecp, int64_t vec_ld,
                                                 int tcols, int64_t ab, int tid) {
    const int r = tid & 31, p0 = tid >> 5;
#pragma unroll
    for (int c = 0; c < COLS / 8; c++) rv.x[c] = p0 + 8 * c < tcols ? vecp[(int64_t)(p0 + 8 * c) * vec_ld + ab * 32 + r] : 0.f;
}
template <int COLS>
__device__ __forceinline__ void split_wide_stage(const SplitWideRowVals<COLS> &rv, float *lds, int tid) {
    const int r = tid & 31, p0 = tid >> 5;
#pragma unroll
    for (int c = 0; c < COLS / 8; c++) lds[32 + r * WideGeo<COLS>::kStride + p0 + 8 * c] = rv.x[c];
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int KS, int FR, int KF, int COLS>
__global__ void __launch_bounds__(64 * kSplitWideWaves, 2)
    mmv_split_wide_kernel(const uintx4 *__restrict__ PA, const float *__restrict__ vecp, int64_t vec_ld,
                          const uintx4 *__restrict__ PB, int64_t na_blocks, int64_t nb_blocks, int64_t a_chunk_blocks,
                          float *__restrict__ partial, int64_t nb_pad, int tcols, bool y_fastest) {
    using G = WideGeo<COLS>;
    __shared__ __attribute__((aligned(16))) float stage[2][G::kStage];   // shared by the four waves
    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, h = lane >> 5;
    // (a wave whose blocks all lie past the end keeps going on the last block, for the barriers; it stores nothing)
    const int64_t bb0 = ((int64_t)bx * kSplitWideWaves + wave) * FR;
    const int64_t a0 = (int64_t)by * a_chunk_blocks;
    int64_t a1 = a0 + a_chunk_blocks;
    if (a1 > na_blocks) a1 = na_blocks;

    SplitWideFrag<KS> breg[FR];
#pragma unroll
    for (int q = 0; q < FR; q++) {
        const int64_t bb = bb0 + q < nb_blocks ? bb0 + q : nb_blocks - 1;
        load_split_wide<KS>(breg[q], PB, bb, lane);
        // the pair (1.0, h) in the last dword of the upper lane half becomes (h, 1.0): A.1 meets B.h, A.h meets B.1
        if (h) {
#pragma unroll
            for (int c = 0; c < 3; c++) {
                const unsigned w = breg[q].p[KS - 1][c][3];
                breg[q].p[KS - 1][c][3] = (w >> 16) | (w << 16);
            }
        }
    }
    WideAcc<FR, COLS> out;
    wide_zero<FR, COLS>(out);

    SplitWideFrag<KS> fa;
    SplitWideRowVals<COLS> rv;
    if (a0 < a1) {
        load_split_wide<KS>(fa, PA, a0, lane);
        split_wide_fetch<COLS>(rv, vecp, vec_ld, tcols, a0, tid);
        split_wide_stage<COLS>(rv, stage[0], tid);
    }
    wide_barrier();
    // One barrier per A block: a stage is written after the barrier that follows its last reader and read after the
    // barrier that follows its writers.  The conditions are the same for every wave of the workgroup.
    int buf = 0;
    for (int64_t ab = a0; ab < a1; ab++) {
        const float *lds = stage[buf];
        floatx16 acc[FR];
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[q][r] = 0.f;
        // partial products, lowest order first: (mid,mid) (hi,lo) (lo,hi) (hi,mid) (mid,hi) (hi,hi)
        constexpr int kPieceA[6] = {1, 0, 2, 0, 1, 0}, kPieceB[6] = {1, 2, 0, 1, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
            for (int pr = 0; pr < 6; pr++)
#pragma unroll
                for (int q = 0; q < FR; q++)
                    acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa.p[ks][kPieceA[pr]]),
                                                                     __builtin_bit_cast(bf16x8, breg[q].p[ks][kPieceB[pr]]),
                                                                     acc[q], 0, 0, 0);
        // operands and right-hand sides of the next A block: into the registers the chains have just read; the loads
        // complete behind the exponentials and the contraction
        const bool has1 = ab + 1 < a1;
        if (has1) {
            load_split_wide<KS>(fa, PA, ab + 1, lane);
            split_wide_fetch<COLS>(rv, vecp, vec_ld, tcols, ab + 1, tid);
        }
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[q][r] = kernel_value<KF>(acc[q][r]);
        __builtin_amdgcn_sched_barrier(0);
        wide_contract<FR, COLS>(acc, lds, j, h, out);
        if (has1) split_wide_stage<COLS>(rv, stage[buf ^ 1], tid);
        wide_barrier();
        buf ^= 1;
    }
    wide_store<FR, COLS>(out, partial, by, tcols, nb_pad, bb0, nb_blocks, lane);
}

template <int KS, int FR, int COLS>
static int launch_split_wide_one(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, int tcols,
                                 int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
    const int64_t per_wg = kSplitWideWaves * FR;
    dim3 grid((unsigned)((B.nblk + per_wg - 1) / per_wg), (unsigned)splits);
    hipLaunchKernelGGL((mmv_split_wide_kernel<KS, FR, FLK_KF, COLS>), grid, dim3(64 * kSplitWideWaves), 0, st,
                       (const uintx4 *)A.data, vecp, vec_ld, (const uintx4 *)B.data, A.nblk, B.nblk, a_chunk_blocks,
                       partial, B.npad, tcols, B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_split_wide_kernel");
    return FLK_OK;
}

template <int KS>
static int launch_split_wide_ks(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, int tcols,
                                int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
#define FLK_SPLIT_WIDE_FORM(COLSV)                                                                                  \
    case COLSV:                                                                                                     \
        return launch_split_wide_one<KS, kSplitWideBlocksPerWave, COLSV>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, \
                                                                         splits, partial, st);
    switch (split_wide_form_cols(tcols, KS)) {
        FLK_SPLIT_WIDE_FORM(8) FLK_SPLIT_WIDE_FORM(16) FLK_SPLIT_WIDE_FORM(32) FLK_SPLIT_WIDE_FORM(40)
        FLK_SPLIT_WIDE_FORM(48) FLK_SPLIT_WIDE_FORM(64)
    }
#undef FLK_SPLIT_WIDE_FORM
    return fail(FLK_EINVAL, "mmv_split wide: column chunk %d not in 1..%d", tcols, kSplitWideMaxCols);
}

int FLK_CAT(launch_mmv_split_wide_kf, FLK_KF)(const SplitView &A, const SplitView &B, const float *vecp,
                                              int64_t vec_ld, int tcols, int64_t a_chunk_blocks, int splits,
                                              float *partial, hipStream_t st) {
    if (A.ks != B.ks || A.d != B.d) return fail(FLK_EINVAL, "mmv_split: operands packed with different feature counts");
    if (tcols < 1 || tcols > kSplitWideMaxCols)
        return fail(FLK_EINVAL, "mmv_split wide: column chunk %d not in 1..%d", tcols, kSplitWideMaxCols);
    switch (A.ks) {
        case 1: return launch_split_wide_ks<1>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        case 2: return launch_split_wide_ks<2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        case 3: return launch_split_wide_ks<3>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        case 4: return launch_split_wide_ks<4>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
    }
    return fail(FLK_EUNSUPPORTED, "mmv_split wide: %lld features (more than %lld)", (long long)A.d,
                (long long)kSplitWideMaxD);
}

}  // namespace flk
