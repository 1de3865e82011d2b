// LDS-tiled kernel-vector product of the bf16x3 mode (see split_common.h) for feature counts beyond the
// register-resident kernel, fp32 data, gfx950.  Compiled once per kernel function (-DFLK_KF=0..4).
//
//   partial[split'][t][b] = sum_{a in chunk} K(A_a, B_b) * vec[a,t]
//
// A workgroup owns one tile of output rows (B side) and walks over the tiles of reduction rows (A side) of its
// chunk.  The packed operands are consumed one k-step of 16 features at a time: the three bfloat16 pieces of the
// k-step of both tiles are staged in LDS (two stages, one barrier per k-step; the packed layout already is the
// operand order, so a stage is a plain copy of 16-byte vectors), every wave keeps a WA_FR x WB_FR grid of MFMA
// accumulators and issues the six partial products of each pair with v_mfma_f32_32x32x16_bf16.  The half norms
// ride in the last two features (the B side swaps the pair when it reads its operands), so after the last k-step
// the accumulators hold the exponent.  Epilogue as in the fp32 LDS-tiled kernel: per-lane FMAs for up to four
// right-hand sides, a second small fp32 MFMA contraction (accumulator registers as the A operand) beyond that.
#include "kernel_fn.h"
#include "mfma_traits.h"
#include "split_common.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

static __device__ __forceinline__ bf16x8 bits_as_bf16x8(uintx4 v) { return __builtin_bit_cast(bf16x8, v); }

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int WVA, int WVB, int WA_FR, int WB_FR, int TT, int KF>
__global__ void __launch_bounds__(64 * WVA * WVB, (WVA * WVB == 4 ? 2 : 1))   // two waves per SIMD either way
    mmv_split_large_kernel(const uintx4 *__restrict__ PA, const float *__restrict__ vecp, int64_t vec_ld, int tcols,
                           const uintx4 *__restrict__ PB, int64_t na_blocks, int64_t nb_blocks, int ks_count,
                           int64_t a_tiles_per_chunk, float *__restrict__ partial, int64_t nb_pad, bool y_fastest) {
    typedef LTraits<float> TR;
    constexpr int kThreads = 64 * WVA * WVB;
    constexpr int NAB = WVA * WA_FR, NBB = WVB * WB_FR;          // blocks of 32 rows per tile
    constexpr int A_ROWS = NAB * 32;
    constexpr int kBlockVecs = 3 * 64;                            // 16-byte vectors per block and k-step
    constexpr int A_VECS = NAB * kBlockVecs, B_VECS = NBB * kBlockVecs;
    constexpr int A_VPT = (A_VECS + kThreads - 1) / kThreads, B_VPT = (B_VECS + kThreads - 1) / kThreads;
    constexpr bool kMfmaEpi = TT > 4;
    constexpr int kVecStride = 17;
    constexpr int kRowBuf = kMfmaEpi ? A_ROWS * kVecStride : TT * A_ROWS;
    __shared__ __attribute__((aligned(16))) uintx4 ldsA[2][A_VECS];
    __shared__ __attribute__((aligned(16))) uintx4 ldsB[2][B_VECS];
    __shared__ __attribute__((aligned(32))) float ldsRow[kRowBuf];   // vec of the A tile

    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wa = wave % WVA, wb = wave / WVA;
    const int j = lane & 31, lg = lane >> 5;
    const int64_t bblk0 = (int64_t)bx * NBB;
    const int64_t a_tiles = (na_blocks + NAB - 1) / NAB;
    const int64_t at0 = (int64_t)by * a_tiles_per_chunk;
    int64_t at1 = at0 + a_tiles_per_chunk;
    if (at1 > a_tiles) at1 = a_tiles;

    float out[WB_FR][kMfmaEpi ? 1 : TT];          // per-lane FMA path: out[q][t] for this lane's output row
    floatx16 out2[kMfmaEpi ? WB_FR : 1];          // MFMA path: lane = column t, registers = output rows
#pragma unroll
    for (int q = 0; q < WB_FR; q++)
#pragma unroll
        for (int t = 0; t < (kMfmaEpi ? 1 : TT); t++) out[q][t] = 0.f;
#pragma unroll
    for (int q = 0; q < (kMfmaEpi ? WB_FR : 1); q++)
#pragma unroll
        for (int r = 0; r < 16; r++) out2[q][r] = 0.f;

    // where this thread's pieces of a stage come from: vector vi of a tile is (block vi / 192, offset vi % 192);
    // blocks past the end re-read the last block (their rows get zero weight / are not stored), and the vector
    // indices past the tile (the tile is not a multiple of the thread count) repeat the last vector
    const uintx4 *srcA[A_VPT], *srcB[B_VPT];

    for (int64_t at = at0; at < at1; at++) {
        const int64_t ablk0 = at * NAB;
#pragma unroll
        for (int c = 0; c < A_VPT; c++) {
            int vi = tid + c * kThreads;
            if (vi >= A_VECS) vi = A_VECS - 1;
            int64_t b = ablk0 + vi / kBlockVecs;
            if (b >= na_blocks) b = na_blocks - 1;
            srcA[c] = PA + b * ks_count * kBlockVecs + vi % kBlockVecs;
        }
#pragma unroll
        for (int c = 0; c < B_VPT; c++) {
            int vi = tid + c * kThreads;
            if (vi >= B_VECS) vi = B_VECS - 1;
            int64_t b = bblk0 + vi / kBlockVecs;
            if (b >= nb_blocks) b = nb_blocks - 1;
            srcB[c] = PB + b * ks_count * kBlockVecs + vi % kBlockVecs;
        }
        floatx16 acc[WA_FR][WB_FR];
#pragma unroll
        for (int p = 0; p < WA_FR; p++)
#pragma unroll
            for (int q = 0; q < WB_FR; q++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[p][q][r] = 0.f;

        uintx4 ra[A_VPT], rb[B_VPT];
        auto fetch = [&](int s) {
#pragma unroll
            for (int c = 0; c < A_VPT; c++) ra[c] = srcA[c][(int64_t)s * kBlockVecs];
#pragma unroll
            for (int c = 0; c < B_VPT; c++) rb[c] = srcB[c][(int64_t)s * kBlockVecs];
        };
        auto commit = [&](int buf) {
#pragma unroll
            for (int c = 0; c < A_VPT; c++) {
                const int vi = tid + c * kThreads;
                if (vi < A_VECS) ldsA[buf][vi] = ra[c];
            }
#pragma unroll
            for (int c = 0; c < B_VPT; c++) {
                const int vi = tid + c * kThreads;
                if (vi < B_VECS) ldsB[buf][vi] = rb[c];
            }
        };

        // Prologue of an A tile: first k-step and the tile's right-hand side values are loaded before anything
        // waits; the barrier that protects ldsRow and the stages from the previous tile's epilogue comes after.
        fetch(0);
        constexpr int kRowVals = (kMfmaEpi ? 16 : TT) * A_ROWS;
        constexpr int kRowValsPerThread = (kRowVals + kThreads - 1) / kThreads;
        float rowv[kRowValsPerThread];
#pragma unroll
        for (int c = 0; c < kRowValsPerThread; c++) {
            const int e = tid + c * kThreads;
            const int which = e / A_ROWS, r = e % A_ROWS;
            const int64_t row = ablk0 * 32 + r;
            float val = 0.f;                      // rows past n_a carry zero weight
            if (e < kRowVals && row < na_blocks * 32 && which < tcols) val = vecp[(int64_t)which * vec_ld + row];
            rowv[c] = val;
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < kRowValsPerThread; c++) {
            const int e = tid + c * kThreads;
            const int which = e / A_ROWS, r = e % A_ROWS;
            if (e < kRowVals) {
                if (!kMfmaEpi) ldsRow[e] = rowv[c];
                else ldsRow[r * kVecStride + which] = rowv[c];
            }
        }
        commit(0);
        __syncthreads();

        for (int s = 0; s < ks_count; s++) {
            const int buf = s & 1;
            const bool more = s + 1 < ks_count;
            if (more) fetch(s + 1);
            uintx4 a[WA_FR][3], b[WB_FR][3];
#pragma unroll
            for (int c = 0; c < 3; c++) {
#pragma unroll
                for (int p = 0; p < WA_FR; p++) a[p][c] = ldsA[buf][((wa * WA_FR + p) * 3 + c) * 64 + lane];
#pragma unroll
                for (int q = 0; q < WB_FR; q++) b[q][c] = ldsB[buf][((wb * WB_FR + q) * 3 + c) * 64 + lane];
            }
            // B role, last k-step: the pair (1.0, h) in the last dword of the upper lane half becomes (h, 1.0)
            if (!more && lg) {
#pragma unroll
                for (int q = 0; q < WB_FR; q++)
#pragma unroll
                    for (int c = 0; c < 3; c++) b[q][c][3] = (b[q][c][3] >> 16) | (b[q][c][3] << 16);
            }
            // partial products, lowest order first: (mid,mid) (hi,lo) (lo,hi) (hi,mid) (mid,hi) (hi,hi)
            constexpr int kPieceA[6] = {1, 0, 2, 0, 1, 0}, kPieceB[6] = {1, 2, 0, 1, 0, 0};
#pragma unroll
            for (int pr = 0; pr < 6; pr++)
#pragma unroll
                for (int p = 0; p < WA_FR; p++)
#pragma unroll
                    for (int q = 0; q < WB_FR; q++)
                        acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bits_as_bf16x8(a[p][kPieceA[pr]]),
                                                                            bits_as_bf16x8(b[q][kPieceB[pr]]),
                                                                            acc[p][q], 0, 0, 0);
            // the other stage was last read one k-step ago, and every wave has passed the barrier since
            if (more) commit(buf ^ 1);
            __syncthreads();
        }

        // epilogue: K = kernel_value(acc) ; out[q][t] += K * vec[i][t]
        if constexpr (!kMfmaEpi) {
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
                const int rbase = (wa * WA_FR + p) * 32;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int ro = rbase + TR::group_off(g, lg);
                    float kv[WB_FR][4];
#pragma unroll
                    for (int q = 0; q < WB_FR; q++)
#pragma unroll
                        for (int e = 0; e < 4; e++) kv[q][e] = kernel_value<KF>(acc[p][q][4 * g + e]);
#pragma unroll
                    for (int t = 0; t < TT; t++) {
                        const floatx4 vv = *(const floatx4 *)(&ldsRow[t * A_ROWS + ro]);
#pragma unroll
                        for (int q = 0; q < WB_FR; q++)
#pragma unroll
                            for (int e = 0; e < 4; e++) out[q][t] = __builtin_fmaf(kv[q][e], vv[e], out[q][t]);
                    }
                }
            }
        } else {
#pragma unroll
            for (int p = 0; p < WA_FR; p++)
#pragma unroll
                for (int q = 0; q < WB_FR; q++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[p][q][r] = kernel_value<KF>(acc[p][q][r]);
            // out2[q][j-rows][t] += sum_i K[i][j] vec[i][t]: accumulator register s2 of a lane is exactly the fp32
            // MFMA A operand of step s2 (row i = acc_row(s2, lg), column j = lane % 32); the B operand is
            // vec[acc_row(s2, lg)][t] with t = lane % 16 (columns past 16 are never stored)
            const float *vb = &ldsRow[j & 15];
            // one read ahead, fenced (otherwise all reads are hoisted to the front and spilled)
            float bval = vb[((wa * WA_FR) * 32 + TR::acc_row(0, lg)) * kVecStride], bnext = 0.f;
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
                const int rbase = (wa * WA_FR + p) * 32;
#pragma unroll
                for (int s2 = 0; s2 < 16; s2++) {
                    if (s2 + 1 < 16) bnext = vb[(rbase + TR::acc_row(s2 + 1, lg)) * kVecStride];
                    else if (p + 1 < WA_FR) bnext = vb[(rbase + 32 + TR::acc_row(0, lg)) * kVecStride];
#pragma unroll
                    for (int q = 0; q < WB_FR; q++) out2[q] = TR::mfma(acc[p][q][s2], bval, out2[q]);
                    asm volatile("" : "+v"(bval) : "v"(vb) : "memory");
                    bval = bnext;
                }
            }
        }
    }

    if constexpr (kMfmaEpi) {
        const int tl = j & 15;
        if (j < 16 && tl < tcols) {
#pragma unroll
            for (int q = 0; q < WB_FR; q++) {
                const int64_t bb = bblk0 + wb * WB_FR + q;
                if (bb < nb_blocks) {
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        partial[(((int64_t)by * WVA + wa) * tcols + tl) * nb_pad + bb * 32 + TR::acc_row(r, lg)] =
                            out2[q][r];
                }
            }
        }
    } else {
#pragma unroll
        for (int q = 0; q < WB_FR; q++) {
            const int64_t bb = bblk0 + wb * WB_FR + q;
#pragma unroll
            for (int t = 0; t < TT; t++) {
                float s = out[q][t];
                s += __shfl_xor(s, 32, 64);
                if (lg == 0 && bb < nb_blocks && t < tcols)
                    partial[(((int64_t)by * WVA + wa) * tcols + t) * nb_pad + bb * 32 + j] = s;
            }
        }
    }
}

// 4 waves (2 x 2), two workgroups per CU so that one workgroup's barrier and LDS latencies are covered by the
// other; tile 128 (A) x 128 (B) rows
constexpr int kSLWavesA = 2, kSLWavesB = 2, kSLFragsA = 2, kSLFragsB = 2;

#if FLK_KF == FLK_GAUSSIAN   // the tile geometry is the same for every kernel function: defined once
int split_large_a_tile_blocks() { return kSLWavesA * kSLFragsA; }
int split_large_b_tile_blocks() { return kSLWavesB * kSLFragsB; }
int split_large_partials_per_split() { return kSLWavesA; }
int split_large_max_cols() { return 16; }
#endif

template <int TT>
static int launch_split_large_tt(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, int tcols,
                                 int64_t a_tiles_per_chunk, int splits, float *partial, hipStream_t st) {
    const int64_t nbb = kSLWavesB * kSLFragsB;
    dim3 grid((unsigned)((B.nblk + nbb - 1) / nbb), (unsigned)splits);
    hipLaunchKernelGGL((mmv_split_large_kernel<kSLWavesA, kSLWavesB, kSLFragsA, kSLFragsB, TT, FLK_KF>), grid,
                       dim3(64 * kSLWavesA * kSLWavesB), 0, st, (const uintx4 *)A.data, vecp, vec_ld, tcols,
                       (const uintx4 *)B.data, A.nblk, B.nblk, (int)A.ks, a_tiles_per_chunk, partial, B.npad,
                       B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_split_large_kernel");
    return FLK_OK;
}

int FLK_CAT(launch_mmv_split_large_kf, FLK_KF)(const SplitView &A, const SplitView &B, const float *vecp,
                                               int64_t vec_ld, int tcols, int64_t a_tiles_per_chunk, int splits,
                                               float *partial, hipStream_t st) {
    if (A.ks != B.ks || A.d != B.d)
        return fail(FLK_EINVAL, "mmv_split_large: operands packed with different feature counts");
    if (tcols < 1 || tcols > 16) return fail(FLK_EINVAL, "mmv_split_large: column chunk %d not in 1..16", tcols);
    if (tcols == 1) return launch_split_large_tt<1>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    if (tcols == 2) return launch_split_large_tt<2>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    if (tcols <= 4) return launch_split_large_tt<4>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    return launch_split_large_tt<16>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
}

}  // namespace flk
