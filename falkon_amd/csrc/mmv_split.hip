// Register-resident kernel-vector product of the bf16x3 mode (see split_common.h), fp32 data, d <= 62, gfx950.
// Compiled once per kernel function (-DFLK_KF=0..4).
//
//   partial[split][t][b] = sum_{a in chunk(split)} K(A_a, B_b) * vec[a,t]
//
// Same structure as the fp32 register-resident kernel: a wave keeps FR blocks of 32 output rows (B side) in
// registers, streams blocks of 32 reduction rows (A side) from L2/HBM and never stores K.  The cross term of a
// 32 x 32 tile is 6 * KS v_mfma_f32_32x32x16_bf16 (KS k-steps of 16 features, six partial products each, lowest
// order first); the half norms ride in the last two features, so the accumulator starts from zero and ends as
// the exponent.  The matrix cores run beside the vector ALU: the chain of fragment q is issued interleaved with
// the epilogue (exp2, FMAs against vec) of fragment q-1, which the scheduling barriers below spell out; the loop
// body is branch free so that it stays one scheduling region.
#include "kernel_fn.h"
#include "split_common.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int kSplitWaves = 4;
constexpr int kSplitFlushEvery = 16;   // A blocks between flushes of the short accumulator

template <int KS> struct SplitFrag { uintx4 p[KS][3]; };

template <int KS>
__device__ __forceinline__ void load_split(SplitFrag<KS> &f, const uintx4 *__restrict__ P, int64_t blk, int lane) {
    const uintx4 *p = P + (blk * KS * 3) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int c = 0; c < 3; c++) f.p[ks][c] = p[(ks * 3 + c) * 64];
}

__device__ __forceinline__ bf16x8 as_bf16x8(uintx4 v) { return __builtin_bit_cast(bf16x8, v); }

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int KS, int FR, int TT, int KF>
__global__ void __launch_bounds__(64 * kSplitWaves, 2)
    mmv_split_kernel(const uintx4 *__restrict__ PA, const float *__restrict__ vecp, int64_t vec_ld,
                     const uintx4 *__restrict__ PB, int64_t na_blocks, int64_t nb_blocks, int64_t a_chunk_blocks,
                     float *__restrict__ partial, int64_t nb_pad, int tcols, bool y_fastest) {
    static_assert(TT <= 4, "two staged dwords per lane cover at most four columns of 32 rows");
    constexpr int kStageDw = (TT + 1) / 2;      // dwords a lane stages per A block: columns lane/32 + 2c, row lane%32
    __shared__ __attribute__((aligned(16))) float stage[kSplitWaves][2][64 * kStageDw];
    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 31, h = lane >> 5;
    const int64_t bb0 = ((int64_t)bx * kSplitWaves + wave) * FR;
    if (bb0 >= nb_blocks) return;               // whole wave idle; no barriers in this kernel
    const int64_t a0 = (int64_t)by * a_chunk_blocks;
    int64_t a1 = a0 + a_chunk_blocks;
    if (a1 > na_blocks) a1 = na_blocks;

    // resident B fragments (blocks past the end re-read the last block; their results are not stored)
    SplitFrag<KS> breg[FR];
#pragma unroll
    for (int q = 0; q < FR; q++) {
        const int64_t bb = bb0 + q < nb_blocks ? bb0 + q : nb_blocks - 1;
        load_split<KS>(breg[q], PB, bb, lane);
        // the pair (1.0, h) in the last dword of the upper lane half becomes (h, 1.0): A.1 meets B.h, A.h meets B.1
        if (h) {
#pragma unroll
            for (int c = 0; c < 3; c++) {
                const unsigned w = breg[q].p[KS - 1][c][3];
                breg[q].p[KS - 1][c][3] = (w >> 16) | (w << 16);
            }
        }
    }
    float o1[FR][TT], o2[FR][TT];
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int t = 0; t < TT; t++) { o1[q][t] = 0.f; o2[q][t] = 0.f; }

    // vec[a, t] of an A block reaches the lanes through a wave-private LDS buffer: one or two dwords per lane from
    // global memory (column lane/32 + 2c clamped to the caller's last one, row lane%32), read back as broadcast
    // 16-byte pieces
    const float *vsrc[kStageDw];
#pragma unroll
    for (int c = 0; c < kStageDw; c++) {
        const int col = (lane >> 5) + 2 * c;
        vsrc[c] = vecp + (int64_t)(col < tcols ? col : tcols - 1) * vec_ld + (lane & 31);
    }
    SplitFrag<KS> fa;
    int buf = 0;
    if (a0 < a1) {
        load_split<KS>(fa, PA, a0, lane);
#pragma unroll
        for (int c = 0; c < kStageDw; c++) stage[wave][0][64 * c + lane] = vsrc[c][a0 * 32];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    int since_flush = 0;
    for (int64_t ab = a0; ab < a1; ab++) {
        const float *lds = stage[wave][buf];
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        floatx4 vec[TT][4];
#pragma unroll
        for (int t = 0; t < TT; t++)
#pragma unroll
            for (int g = 0; g < 4; g++) vec[t][g] = *(const floatx4 *)(lds + 32 * t + 8 * g + 4 * h);
        floatx16 acc[FR];
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[q][r] = 0.f;
        // partial products, lowest order first: (mid,mid) (hi,lo) (lo,hi) (hi,mid) (mid,hi) (hi,hi)
        constexpr int kPieceA[6] = {1, 0, 2, 0, 1, 0}, kPieceB[6] = {1, 2, 0, 1, 0, 0};
        constexpr int kChain = 6 * KS;                                        // MFMAs per fragment
        constexpr int kValuPerMfma = (16 * (1 + TT) + kChain - 1) / kChain;   // epilogue ops issued behind each MFMA
#pragma unroll
        for (int q = 0; q <= FR; q++) {
            if (q < FR) {
#pragma unroll
                for (int ks = 0; ks < KS; ks++)
#pragma unroll
                    for (int pr = 0; pr < 6; pr++)
                        acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(fa.p[ks][kPieceA[pr]]),
                                                                         as_bf16x8(breg[q].p[ks][kPieceB[pr]]), acc[q],
                                                                         0, 0, 0);
            }
            if (q > 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float k = kernel_value<KF>(acc[q - 1][r]);
#pragma unroll
                    for (int t = 0; t < TT; t++) o1[q - 1][t] = __builtin_fmaf(k, vec[t][r >> 2][r & 3], o1[q - 1][t]);
                }
            }
            // order within the region: chain 0 alone, then every MFMA of chain q followed by its share of epilogue q-1
            if (q == 0) {
                __builtin_amdgcn_sched_group_barrier(0x008, kChain, 0);
            } else if (q < FR) {
#pragma unroll
                for (int i = 0; i < kChain; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma, 0);
                }
            }
        }
        // operands of the next A block into the registers the chains have just read (the last iteration re-reads
        // its own block: no branch in the loop body)
        const int64_t nxt = ab + 1 < a1 ? ab + 1 : ab;
        load_split<KS>(fa, PA, nxt, lane);
#pragma unroll
        for (int c = 0; c < kStageDw; c++) stage[wave][buf ^ 1][64 * c + lane] = vsrc[c][nxt * 32];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        buf ^= 1;
        if (++since_flush >= kSplitFlushEvery) {
            since_flush = 0;
#pragma unroll
            for (int q = 0; q < FR; q++)
#pragma unroll
                for (int t = 0; t < TT; t++) { o2[q][t] += o1[q][t]; o1[q][t] = 0.f; }
        }
    }
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int t = 0; t < TT; t++) {
            float s = o2[q][t] + o1[q][t];
            s += __shfl_xor(s, 32, 64);
            if (h == 0 && bb0 + q < nb_blocks && t < tcols)
                partial[((int64_t)by * tcols + t) * nb_pad + (bb0 + q) * 32 + j] = s;
        }
}

template <int KS, int FR, int TT>
static int launch_split_one(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, int tcols,
                            int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
    const int64_t per_wg = kSplitWaves * FR;
    dim3 grid((unsigned)((B.nblk + per_wg - 1) / per_wg), (unsigned)splits);
    hipLaunchKernelGGL((mmv_split_kernel<KS, FR, TT, FLK_KF>), grid, dim3(64 * kSplitWaves), 0, st,
                       (const uintx4 *)A.data, vecp, vec_ld, (const uintx4 *)B.data, A.nblk, B.nblk, a_chunk_blocks,
                       partial, B.npad, tcols, B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_split_kernel");
    return FLK_OK;
}

// three and four columns: two resident fragments per wave whatever the feature count (registers)
template <int KS, int FR>
static int launch_split_tt(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, int tcols,
                           int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
    if (tcols == 1) return launch_split_one<KS, FR, 1>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
    if (tcols == 2) return launch_split_one<KS, FR, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
    return launch_split_one<KS, 2, 4>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
}

int FLK_CAT(launch_mmv_split_kf, FLK_KF)(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld,
                                         int tcols, int64_t a_chunk_blocks, int splits, float *partial,
                                         hipStream_t st) {
    if (A.ks != B.ks || A.d != B.d) return fail(FLK_EINVAL, "mmv_split: operands packed with different feature counts");
    if (tcols < 1 || tcols > kSplitMaxCols)
        return fail(FLK_EINVAL, "mmv_split: column chunk %d not in 1..%d", tcols, kSplitMaxCols);
    if (split_b_blocks_per_wg(A.ks, tcols) != kSplitWaves * (A.ks <= 2 && tcols <= 2 ? 4 : 2))
        return fail(FLK_EINVAL, "mmv_split: launch geometry out of step with the planner");
    switch (A.ks) {
        case 1: return launch_split_tt<1, 4>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        case 2: return launch_split_tt<2, 4>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        case 3: return launch_split_tt<3, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
        case 4: return launch_split_tt<4, 2>(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st);
    }
    return fail(FLK_EUNSUPPORTED, "mmv_split: %lld features (more than %lld)", (long long)A.d, (long long)kSplitMaxD);
}

}  // namespace flk
