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

// Forms of the kernel that contracts on the matrix cores (mmv_small_f32_wide.hip): columns per pass that serve tcols
// right-hand sides, and resident blocks per wave of a form: four up to 16 padded features where a block has 16 output
// accumulators or fewer (8, 16 and 32 columns), two otherwise (registers)
constexpr int wide_form_cols(int tcols) {
    return tcols <= 8 ? 8 : tcols <= 16 ? 16 : tcols <= 24 ? 24 : tcols <= 32 ? 32 : tcols <= 40 ? 40 : tcols <= 48 ? 48 : 64;
}
constexpr int wide_blocks_per_wave(int dp, int cols) {
    return dp <= 8 && (cols == 8 || cols == 16 || cols == 32) ? 4 : 2;
}
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

// keep = false clears the right-hand side entries of the block (its kernel values then contribute nothing to the
// sums): for the block that is processed a second time when a chunk holds an odd number of blocks.  A bit mask, not a
// product with zero: an infinite entry of the right-hand side must not turn into NaN there.  Applied here and not
// where the values are fetched, so that nothing touches the loaded registers before the tile step in between is done.
template <int TT>
__device__ __forceinline__ void stage_rowvals(const RowVals<TT> &rv, float *lds, int lane, bool keep = true) {
    const unsigned mask = keep ? 0xffffffffu : 0u;
#pragma unroll
    for (int c = 0; c < RowVals<TT>::C; c++) {
        int e = lane + 64 * c;
        if (e < RowVals<TT>::N) lds[e] = e >= 32 ? __uint_as_float(__float_as_uint(rv.x[c]) & mask) : rv.x[c];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// (the block's base address is wave-uniform, i.e. scalar arithmetic where the block index is a scalar, and the lane's
// part a 32-bit offset: computed per lane in 64 bits the addresses of a two-block trip cost a dozen multi-cycle vector
// instructions, which do not overlap with the MFMAs)
// Floats of a packed block of 32 rows whose features are consumed in DP steps: 2 DP features up to 64, and the
// feature count padded for the LDS-tiled kernel (whole chunks of kLargeKChunk steps, zeros past the data) beyond.
constexpr int block_floats(int dp) { return (dp <= 32 ? 2 * dp : (2 * dp + 2 * (int)kLargeKChunk - 1) / (2 * (int)kLargeKChunk) * (2 * (int)kLargeKChunk)) * 32; }

template <int DP>
__device__ __forceinline__ void load_a(float (&a)[DP], const float *__restrict__ PA, int64_t ab, int j, int h) {
    const auto blk = scalar_base(PA + ab * block_floats(DP));      // one block index per wave
    const int off = h * (DP * 32) + j;
#pragma unroll
    for (int s = 0; s < DP; s++) a[s] = blk[off + s * 32];
}

// FOLD: the accumulators start from the A block's half norms alone (the output side's half norm arrives through the
// MFMA chain, or, with RAW, is applied to the finished sums).  RAW (Gaussian only): the accumulator holds the exponent
// without the output side's half norm; it can be positive, so the kernel value is the bare exp2, not clamped at 1.
template <int KF, bool RAW> __device__ __forceinline__ float tile_value(float e) {
    if constexpr (RAW) return __builtin_amdgcn_exp2f(e);
    else return kernel_value<KF>(e);
}

template <int DP, int FR, int TT, bool FOLD, int KF, bool RAW = false, bool PIN = false>
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
        // PIN (where there are registers to spare): keep these reads in front of the MFMA chain; the compiler
        // would sink them to the epilogue, where each read then stalls the wave for the LDS latency
        if constexpr (PIN) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < DP; s++)
#pragma unroll
            for (int q = 0; q < FR; q++)
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], breg[q][s], acc[q], 0, 0, 0);
#pragma unroll
        for (int q = 0; q < FR; q++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float k = tile_value<KF, RAW>(acc[q][r]);
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
            for (int r = 0; r < 16; r++) acc[q][r] = tile_value<KF, RAW>(acc[q][r]);
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

// The reduction loop of one wave over the A blocks a0 .. a1: streams the blocks (double buffered in registers, row
// values through the wave's LDS stage) and accumulates into o1 / o2.  NOADD: the accumulators start from the A block's
// half norms alone (see the kernel).
template <int DP, int FR, int TT, bool NOADD, int KF, bool TWO_LEVEL, bool RAW>
__device__ __forceinline__ void reduce_blocks(const float *__restrict__ PA, const float *const (&src)[RowVals<TT>::C],
                                              int64_t a0, int64_t a1, int lane, int j, int h, float *lds0, float *lds1,
                                              const float (&breg)[FR][DP], const float (&hb)[FR], float (&o1)[FR][TT],
                                              float (&o2)[FR][TWO_LEVEL ? TT : 1]) {
    using RV = RowVals<TT>;
    float fa0[DP], fa1[DP];
    RV rv;
    a0 = as_scalar(a0);      // the chunk's bounds are the same for the whole wave: block indices stay scalar
    a1 = as_scalar(a1);
    if (a0 >= a1) return;
    int since_flush = 0;
    // One right-hand side and four resident blocks (the kernels of the single-column products at up to 32 features):
    // a branch-free loop body with its phases pinned.  Measured on N = 1e6, M = 2e4, dfmmv: d = 28 19.95 -> 19.32 ms,
    // d = 16 12.62 -> 12.29.  The other shapes keep the loop below (with two or four columns the pinned reads do
    // not fit the registers; with two resident blocks it measured slower: d = 64 46.8 -> 51.3 ms).
    if constexpr (TT == 1 && FR >= 3) {
        // Both tile steps of the body always run and every block's loads are issued unconditionally, one block ahead.
        // (With loads or a tile step under a condition the compiler sinks the loads to their use, and at each wait
        // has to assume that they may not have been issued, so it waits for the newest loads instead of the ones it
        // needs.)  Past the end of the chunk the last block is loaded again: with an odd number of blocks it is
        // processed twice, the second time against a right-hand side of zeros; the launch plans make the chunks
        // even, so this happens in the last chunk at most.
        // The scheduling barriers keep the phases of a step apart in the generated code: the loads of the next block
        // are issued before the tile's arithmetic, and the staging of its row values, which has to wait for their
        // load, stays behind the tile (hoisted to the front it waits out a full memory latency with nothing in flight).
        // Block indices count from the chunk's first block, in 32 bits: the loop's comparisons and the blocks' base
        // addresses are then scalar instructions (a 64-bit less-than exists on the vector ALU only).
        const float *const PAc = PA + a0 * block_floats(DP);
        const float *srcc[RV::C];
#pragma unroll
        for (int c = 0; c < RV::C; c++) srcc[c] = src[c] + a0 * 32;
        const int nblk = (int)(a1 - a0), last = nblk - 1;
        fetch_rowvals<TT>(rv, srcc, 0);
        load_a<DP>(fa0, PAc, 0, j, h);
        stage_rowvals<TT>(rv, lds0, lane);
        for (int ab = 0; ab < nblk; ab += 2) {
            const bool second = ab + 1 < nblk;
            const int n1 = second ? ab + 1 : last;
            fetch_rowvals<TT>(rv, srcc, n1);    // first: staged right after this tile step
            load_a<DP>(fa1, PAc, n1, j, h);
            __builtin_amdgcn_sched_barrier(0);
            tile_step<DP, FR, TT, NOADD, KF, RAW, true>(fa0, lds0, h, breg, hb, o1);
            __builtin_amdgcn_sched_barrier(0);
            stage_rowvals<TT>(rv, lds1, lane, second);
            const int n2 = ab + 2 < last ? ab + 2 : last;
            fetch_rowvals<TT>(rv, srcc, n2);
            load_a<DP>(fa0, PAc, n2, j, h);
            __builtin_amdgcn_sched_barrier(0);
            tile_step<DP, FR, TT, NOADD, KF, RAW, true>(fa1, lds1, h, breg, hb, o1);
            __builtin_amdgcn_sched_barrier(0);
            stage_rowvals<TT>(rv, lds0, lane);
            since_flush += 2;
            if (TWO_LEVEL && since_flush >= kFlushEvery) {
                // (the empty asm keeps this a branch taken every eighth trip: turned into selects it costs a dozen
                // vector instructions in every trip)
                asm volatile("" ::: "memory");
                since_flush = 0;
#pragma unroll
                for (int q = 0; q < FR; q++)
#pragma unroll
                    for (int t = 0; t < TT; t++) { o2[q][t] += o1[q][t]; o1[q][t] = 0.f; }
            }
        }
    } else {
        load_a<DP>(fa0, PA, a0, j, h);
        fetch_rowvals<TT>(rv, src, a0);
        stage_rowvals<TT>(rv, lds0, lane);
        for (int64_t ab = a0; ab < a1; ab += 2) {
            const bool has1 = ab + 1 < a1;
            if (has1) { load_a<DP>(fa1, PA, ab + 1, j, h); fetch_rowvals<TT>(rv, src, ab + 1); }
            tile_step<DP, FR, TT, NOADD, KF, RAW>(fa0, lds0, h, breg, hb, o1);
            if (has1) {
                stage_rowvals<TT>(rv, lds1, lane);
                const bool has2 = ab + 2 < a1;
                if (has2) { load_a<DP>(fa0, PA, ab + 2, j, h); fetch_rowvals<TT>(rv, src, ab + 2); }
                tile_step<DP, FR, TT, NOADD, KF, RAW>(fa1, lds1, h, breg, hb, o1);
                if (has2) stage_rowvals<TT>(rv, lds0, lane);
            }
            since_flush += 2;
            if (TWO_LEVEL && since_flush >= kFlushEvery) {
                since_flush = 0;
#pragma unroll
                for (int q = 0; q < FR; q++)
#pragma unroll
                    for (int t = 0; t < TT; t++) { o2[q][t] += o1[q][t]; o1[q][t] = 0.f; }
            }
        }
    }
}

// Largest -hB (= half the squared norm of a scaled output row, in bits of the exponent) for which the Gaussian's
// output-side half norm is taken out of the exponent: 2^(x.c + hA) <= 2^(-hB) then stays far below the fp32 range
// (2^64 times the sum over the reduction rows of |vec| would have to overflow).
constexpr float kFactorOutMaxBits = 64.0f;

// FOLD (odd feature counts only): the one padding feature of the packed rows carries 1.0, and the
// resident B fragment puts hB_j into that slot, so the MFMA chain adds hB_j by itself and the
// accumulators start from the A block's half norms without any VALU add.
// Even feature counts have no spare slot.  For the Gaussian the same adds (one per kernel value) are saved by
// factoring the output row's half norm out of the sum: out_j = 2^hB_j * sum_i 2^(x_i.c_j + hA_i) vec_i, valid as long
// as 2^(-hB_j) is nowhere near the fp32 range, which every wave checks on its own resident rows (kFactorOutMaxBits;
// rows with a non-finite half norm fail the check) before it picks between the two loops.  The partial exponent
// x.c + hA can be positive, so on that path a kernel value is not clamped entry by entry: where two points
// coincide K is 1 to rounding (1 + 1e-6 at worst) instead of exactly 1.
template <int DP, int FR, int TT, bool FOLD, int KF>
// Two waves per SIMD (at most 256 registers per lane), except the single-column kernels with four (up to 96 features) or
// three (up to 128) resident blocks beyond 32 features: their resident fragments alone take up to 192 registers, and they
// run one wave per SIMD on up to 512.
__global__ void __launch_bounds__(256, (DP > 32 || (DP > 16 && FR >= 3)) ? 1 : 2)
    mmv_small_f32_kernel(const float *__restrict__ PA, const float *__restrict__ hA, const float *__restrict__ vecp,
                         int64_t vec_ld, const float *__restrict__ PB, const float *__restrict__ hB, int64_t na_blocks,
                         int64_t nb_blocks, int64_t a_chunk_blocks, float *__restrict__ partial, int64_t nb_pad,
                         int tcols, bool y_fastest) {
    // TT columns are computed, the first tcols of them stored; vecp must hold TT planes (zeros beyond the
    // caller's columns).
    using RV = RowVals<TT>;
    constexpr bool kTwoLevel = TT <= 4;   // long accumulator only where registers allow; wider TT uses short chunks
    // (wider column chunks are out of registers with two loops; with two resident blocks per wave, beyond 32 features,
    // the kernel with both loops measured slower than the plain one: d = 64, one column, 46.8 ms per dfmmv at N = 1e6,
    // M = 2e4 against 42.9, d = 40 32.9 against 27.8)
    constexpr bool kCanFactorOut = !FOLD && KF == FLK_GAUSSIAN && TT <= 2 && FR >= 3;
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
    [[maybe_unused]] bool small_norms = true;
#pragma unroll
    for (int q = 0; q < FR; q++) {
        int64_t bb = bb0 + q < nb_blocks ? bb0 + q : nb_blocks - 1;
        load_a<DP>(breg[q], PB, bb, j, h);
        hb[q] = hB[bb * 32 + j];
        if (FOLD) breg[q][DP - 1] = h ? hb[q] : breg[q][DP - 1];   // feature 2*DP-1 lives in lane half 1, step DP-1
        if constexpr (kCanFactorOut) small_norms = small_norms && hb[q] >= -kFactorOutMaxBits;   // false for NaN
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

    float *lds0 = stage[wave][0], *lds1 = stage[wave][1];
    [[maybe_unused]] bool factored = false;
    if constexpr (kCanFactorOut) {
        factored = __all(small_norms);      // wave-uniform
        if (factored)
            reduce_blocks<DP, FR, TT, true, KF, kTwoLevel, true>(PA, src, a0, a1, lane, j, h, lds0, lds1, breg, hb, o1, o2);
        else
            reduce_blocks<DP, FR, TT, FOLD, KF, kTwoLevel, false>(PA, src, a0, a1, lane, j, h, lds0, lds1, breg, hb, o1, o2);
    } else {
        reduce_blocks<DP, FR, TT, FOLD, KF, kTwoLevel, false>(PA, src, a0, a1, lane, j, h, lds0, lds1, breg, hb, o1, o2);
    }
#pragma unroll
    for (int q = 0; q < FR; q++) {
        [[maybe_unused]] float out_scale = 1.0f;
        if constexpr (kCanFactorOut) out_scale = factored ? __builtin_amdgcn_exp2f(hb[q]) : 1.0f;
#pragma unroll
        for (int t = 0; t < TT; t++) {
            float s = kTwoLevel ? o2[q][t] + o1[q][t] : o1[q][t];
            s += __shfl_xor(s, 32, 64);
            if constexpr (kCanFactorOut) s *= out_scale;
            if (h == 0 && bb0 + q < nb_blocks && t < tcols)
                partial[((int64_t)by * tcols + t) * nb_pad + (bb0 + q) * 32 + j] = s;
        }
    }
}


}  // namespace flk
