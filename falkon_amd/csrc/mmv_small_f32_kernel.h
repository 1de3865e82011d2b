// Register-resident kernel-vector product for the radial kernels of kernel_fn.h, fp32, gfx950.
// (Written for the Gaussian, K = exp2(e); the other kernel functions replace the exp2 of the epilogue.)
//
//   partial[split][t][b] = sum_{a in chunk(split)} exp2(A~_a . B~_b + hA_a + hB_b) * vec[a,t]
//
// The kernel matrix is never stored.  A wave owns FR blocks of 32 output rows
// (the "B side") whose packed features stay in registers for the whole kernel,
// and streams blocks of 32 reduction rows (the "A side") straight from L2/HBM
// into registers (the packed layout makes every load a contiguous 128-byte run
// per half wave).  For every (A block, B block) pair the 32x32 cross term is
// v_mfma_f32_32x32x2_f32 accumulated over the features, started from the two
// half norms, so the accumulator holds the base-2 exponent directly; then
// clamp-at-zero, v_exp_f32 and T FMAs per entry contract it against vec.
// Accumulator layout of the 32x32x2 MFMA: lane l, register r holds
//   column j = l % 32 (B row), row i = 8*(r/4) + 4*(l/32) + r%4 (A row),
// so a lane sums over A rows privately and needs no cross-lane traffic until
// the very end (one xor-32 shuffle to join the two lane halves).
#pragma once
#include "flk_common.h"
#include "kernel_fn.h"

namespace flk {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kWavesPerWg = 4;
constexpr int kFlushEvery = 16;  // A blocks between flushes of the short accumulator

// Per-row quantities of an A block (half norms and right-hand side entries) reach the lanes through
// a small wave-private LDS buffer: each lane fetches ONE dword from global memory, the wave writes the
// 32*(1+TT) values to LDS and every lane reads back the 16 rows it accumulates over with broadcast
// ds_read_b128.  Loading those 16 values per lane straight from global memory costs the texture
// addresser a full 64-lane x 16-byte pass per instruction although only 128 distinct bytes are
// touched, which measurably throttles the kernel.  No workgroup barrier is involved: a wave only
// ever reads what it wrote itself.
template <int TT> struct RowVals {
    static constexpr int N = 32 * (1 + TT);       // floats staged per A block
    static constexpr int C = (N + 63) / 64;       // dwords fetched per lane
    float x[C];
};

template <int TT>
__device__ __forceinline__ void fetch_rowvals(RowVals<TT> &rv, const float *const (&src)[RowVals<TT>::C], int64_t ab) {
#pragma unroll
    for (int c = 0; c < RowVals<TT>::C; c++) rv.x[c] = src[c][ab * 32];
}

template <int TT>
__device__ __forceinline__ void stage_rowvals(const RowVals<TT> &rv, float *lds, int lane) {
#pragma unroll
    for (int c = 0; c < RowVals<TT>::C; c++) {
        int e = lane + 64 * c;
        if (e < RowVals<TT>::N) lds[e] = rv.x[c];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

template <int DP>
__device__ __forceinline__ void load_a(float (&a)[DP], const float *__restrict__ PA, int64_t ab, int j, int h) {
    const float *p = PA + (ab * (2 * DP) + (int64_t)h * DP) * 32 + j;
#pragma unroll
    for (int s = 0; s < DP; s++) a[s] = p[s * 32];
}

template <int DP, int FR, int TT, bool FOLD, int KF>
__device__ __forceinline__ void tile_step(const float (&a)[DP], const float *lds, int h, const float (&breg)[FR][DP],
                                          const float (&hb)[FR], float (&o1)[FR][TT]) {
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    floatx4 hn[4];
#pragma unroll
    for (int g = 0; g < 4; g++) hn[g] = *(const floatx4 *)(lds + 8 * g + 4 * h);
    floatx16 acc[FR];
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[q][r] = FOLD ? hn[r >> 2][r & 3] : hn[r >> 2][r & 3] + hb[q];
    if constexpr (TT <= 4) {
        // few right-hand sides: their entries are read before the MFMA chain and wait in registers
        floatx4 vec[TT][4];
#pragma unroll
        for (int t = 0; t < TT; t++)
#pragma unroll
            for (int g = 0; g < 4; g++) vec[t][g] = *(const floatx4 *)(lds + 32 + 32 * t + 8 * g + 4 * h);
#pragma unroll
        for (int s = 0; s < DP; s++)
#pragma unroll
            for (int q = 0; q < FR; q++)
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], breg[q][s], acc[q], 0, 0, 0);
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float k = kernel_value<KF>(acc[q][r]);
#pragma unroll
                for (int t = 0; t < TT; t++) o1[q][t] = __builtin_fmaf(k, vec[t][r >> 2][r & 3], o1[q][t]);
            }
    } else {
        // many right-hand sides: kernel values replace the exponents in the accumulator registers,
        // then each group of four rows is contracted against one broadcast LDS read per column
#pragma unroll
        for (int s = 0; s < DP; s++)
#pragma unroll
            for (int q = 0; q < FR; q++)
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], breg[q][s], acc[q], 0, 0, 0);
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[q][r] = kernel_value<KF>(acc[q][r]);
        // Groups of up to four columns of one row group, software pipelined by hand: the reads of the
        // next group are issued, then a compiler memory fence pins them there, then the FMAs of the
        // current group run.  Without the fences the compiler moves all 4*TT LDS reads to the front
        // (to hide their latency) and spills.
        constexpr int NGRP = 4 * ((TT + 3) / 4);
        floatx4 cur[4], nxt[4];
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (u < TT) cur[u] = *(const floatx4 *)(lds + 32 + 32 * u + 4 * h);
#pragma unroll
        for (int grp = 0; grp < NGRP; grp++) {
            const int g = grp / ((TT + 3) / 4), t0 = 4 * (grp % ((TT + 3) / 4));
            if (grp + 1 < NGRP) {
                const int g1 = (grp + 1) / ((TT + 3) / 4), t1 = 4 * ((grp + 1) % ((TT + 3) / 4));
#pragma unroll
                for (int u = 0; u < 4; u++)
                    if (t1 + u < TT) nxt[u] = *(const floatx4 *)(lds + 32 + 32 * (t1 + u) + 8 * g1 + 4 * h);
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (t0 + u < TT) {
#pragma unroll
                    for (int q = 0; q < FR; q++)
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            o1[q][t0 + u] = __builtin_fmaf(acc[q][4 * g + e], cur[u][e], o1[q][t0 + u]);
                }
            // fence: the updated accumulators pass through it, so this group's FMAs stay above it and the
            // next group's reads (ordered by the memory clobber) stay below the previous one
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (t0 + u < TT) {
                    if constexpr (FR == 4)
                        asm volatile("" : "+v"(o1[0][t0 + u]), "+v"(o1[1][t0 + u]), "+v"(o1[2][t0 + u]), "+v"(o1[3][t0 + u])
                                     : "v"(lds) : "memory");
                    else
                        asm volatile("" : "+v"(o1[0][t0 + u]), "+v"(o1[1][t0 + u]) : "v"(lds) : "memory");
                }
#pragma unroll
            for (int u = 0; u < 4; u++) cur[u] = nxt[u];
        }
    }
}

// FOLD (odd feature counts only): the one padding feature of the packed rows carries 1.0, and the
// resident B fragment puts hB_j into that slot, so the MFMA chain adds hB_j by itself and the
// accumulators start from the A block's half norms without any VALU add.
template <int DP, int FR, int TT, bool FOLD, int KF>
__global__ void __launch_bounds__(256, 2)   // two waves per SIMD: at most 256 registers per lane
    mmv_small_f32_kernel(const float *__restrict__ PA, const float *__restrict__ hA, const float *__restrict__ vecp,
                         int64_t vec_ld, const float *__restrict__ PB, const float *__restrict__ hB, int64_t na_blocks,
                         int64_t nb_blocks, int64_t a_chunk_blocks, float *__restrict__ partial, int64_t nb_pad,
                         int tcols, bool y_fastest) {
    // TT columns are computed, the first tcols of them stored; vecp must hold TT planes (zeros beyond the
    // caller's columns).
    using RV = RowVals<TT>;
    constexpr bool kTwoLevel = TT <= 4;   // long accumulator only where registers allow; wider TT uses short chunks
    __shared__ __attribute__((aligned(16))) float stage[kWavesPerWg][2][RV::N];
    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j = lane & 31, h = lane >> 5;
    const int64_t bb0 = ((int64_t)bx * kWavesPerWg + wave) * FR;
    if (bb0 >= nb_blocks) return;  // whole wave idle; no barriers in this kernel
    const int64_t a0 = (int64_t)by * a_chunk_blocks;
    int64_t a1 = a0 + a_chunk_blocks;
    if (a1 > na_blocks) a1 = na_blocks;

    // resident B fragments (blocks past the end re-read the last block; their results are not stored)
    float breg[FR][DP];
    float hb[FR];
#pragma unroll
    for (int q = 0; q < FR; q++) {
        int64_t bb = bb0 + q < nb_blocks ? bb0 + q : nb_blocks - 1;
        load_a<DP>(breg[q], PB, bb, j, h);
        hb[q] = hB[bb * 32 + j];
        if (FOLD) breg[q][DP - 1] = h ? hb[q] : breg[q][DP - 1];   // feature 2*DP-1 lives in lane half 1, step DP-1
    }
    // where this lane's staged dwords come from: element e = lane + 64c of [hn(32) | vec_0(32) | vec_1(32) ...]
    const float *src[RV::C];
#pragma unroll
    for (int c = 0; c < RV::C; c++) {
        int e = lane + 64 * c;
        src[c] = (e < 32 || e >= RV::N) ? hA + (e & 31) : vecp + (int64_t)((e - 32) >> 5) * vec_ld + (e & 31);
    }

    float o1[FR][TT], o2[FR][kTwoLevel ? TT : 1];
#pragma unroll
    for (int q = 0; q < FR; q++)
#pragma unroll
        for (int t = 0; t < TT; t++) { o1[q][t] = 0.f; if (kTwoLevel) o2[q][t] = 0.f; }

    float fa0[DP], fa1[DP];
    RV rv;
    float *lds0 = stage[wave][0], *lds1 = stage[wave][1];
    if (a0 < a1) {
        load_a<DP>(fa0, PA, a0, j, h);
        fetch_rowvals<TT>(rv, src, a0);
        stage_rowvals<TT>(rv, lds0, lane);
    }
    int since_flush = 0;
    for (int64_t ab = a0; ab < a1; ab += 2) {
        const bool has1 = ab + 1 < a1;
        if (has1) { load_a<DP>(fa1, PA, ab + 1, j, h); fetch_rowvals<TT>(rv, src, ab + 1); }
        tile_step<DP, FR, TT, FOLD, KF>(fa0, lds0, h, breg, hb, o1);
        if (has1) {
            stage_rowvals<TT>(rv, lds1, lane);
            const bool has2 = ab + 2 < a1;
            if (has2) { load_a<DP>(fa0, PA, ab + 2, j, h); fetch_rowvals<TT>(rv, src, ab + 2); }
            tile_step<DP, FR, TT, FOLD, KF>(fa1, lds1, h, breg, hb, o1);
            if (has2) stage_rowvals<TT>(rv, lds0, lane);
        }
        since_flush += 2;
        if (kTwoLevel && since_flush >= kFlushEvery) {
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
            float s = kTwoLevel ? o2[q][t] + o1[q][t] : o1[q][t];
            s += __shfl_xor(s, 32, 64);
            if (h == 0 && bb0 + q < nb_blocks && t < tcols)
                partial[((int64_t)by * tcols + t) * nb_pad + (bb0 + q) * 32 + j] = s;
        }
}


}  // namespace flk
