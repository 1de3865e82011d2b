// LDS-tiled kernel-vector product of the bf16x3 mode (see split_common.h), fp32 data, gfx950: feature counts beyond
// the register-resident kernels (its epilogue contracts up to 64 columns per pass on the matrix cores).
// Compiled once per kernel function (-DFLK_KF=0..4).
//
//   partial[split'][t][b] = sum_{a in chunk} K(A_a, B_b) * vec[a,t]
//
// A workgroup owns one tile of output rows (B side) and walks over the tiles of reduction rows (A side) of its
// chunk.  The packed operands are consumed one k-step of 16 features at a time: the three bfloat16 pieces of the
// k-step of both tiles are staged in LDS (three stages filled two k-steps ahead by direct global-to-LDS loads, one
// barrier per k-step; the packed layout already is the operand order), every wave keeps a WA_FR x WB_FR grid of MFMA
// accumulators and issues the six partial products of each pair with v_mfma_f32_32x32x16_bf16.  The half norms
// ride in the last two features (the B side swaps the pair when it reads its operands), so after the last k-step
// the accumulators hold the exponent.  Epilogue as in the fp32 LDS-tiled kernel: per-lane FMAs for up to four
// right-hand sides, a second small fp32 MFMA contraction (accumulator registers as the A operand) beyond that: 16
// columns per pass with the 16x16x1 step, 32 or 64 with one or two groups of 32x32x2 steps.  The right-hand sides of
// the tile then take the room of the third operand stage (two stages, filled one k-step ahead).
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

// Bare workgroup barrier: the wave's own LDS traffic is drained first, and the compiler may not move memory
// operations across it.  (__syncthreads would also wait for every vector memory operation, i.e. for the direct
// global-to-LDS loads that are meant to stay in flight across the barrier.)
static __device__ __forceinline__ void wg_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
// STORE: the kernel matrix instead of the product: entry (a, b) goes to kout[a * kout_ld + b] (then TT = 1, tcols = 0,
// vecp is not read and partial not written); hnA / hnB are the operands' fp32 half norms, read only to give the rows
// that hold a NaN or an infinity their NaN back (the clamps of the kernel functions would hide it).
template <int WVA, int WVB, int WA_FR, int WB_FR, int TT, int KF, bool STORE = false>
__global__ void __launch_bounds__(64 * WVA * WVB, (WVA * WVB == 4 ? 2 : 1))   // two waves per SIMD either way
    mmv_split_large_kernel(const uintx4 *__restrict__ PA, const float *__restrict__ vecp, int64_t vec_ld, int tcols,
                           const uintx4 *__restrict__ PB, int64_t na_blocks, int64_t nb_blocks, int ks_count,
                           int64_t a_tiles_per_chunk, float *__restrict__ partial, int64_t nb_pad, bool y_fastest,
                           float *__restrict__ kout = nullptr, int64_t kout_ld = 0, int64_t n_a = 0, int64_t n_b = 0,
                           const float *__restrict__ hnA = nullptr, const float *__restrict__ hnB = nullptr) {
    typedef LTraits<float> TR;
    constexpr int kWaves = WVA * WVB, kThreads = 64 * kWaves;
    constexpr int NAB = WVA * WA_FR, NBB = WVB * WB_FR;          // blocks of 32 rows per tile
    constexpr int A_ROWS = NAB * 32;
    constexpr int kBlockVecs = 3 * 64;                            // 16-byte vectors per block and k-step
    constexpr int A_VECS = NAB * kBlockVecs, B_VECS = NBB * kBlockVecs;
    // a stage is copied in units of one piece of one block (64 lanes x 16 bytes = one direct-to-LDS load of a wave)
    constexpr int kUnits = (NAB + NBB) * 3, kUnitsPerWave = kUnits / kWaves;
    static_assert(kUnits % kWaves == 0, "the units of a stage must split evenly over the waves");
    // k-steps in LDS: one in use, the others in flight.  Passes of 32 and 64 columns give the third stage's room to
    // the right-hand sides of the tile (64 columns: 2 x 48 KB of operands + 64 KB, all of the CU's LDS).
    constexpr bool kMfmaEpi = TT > 4;
    constexpr int kGroups32 = TT / 32;                            // groups of 32 columns (32x32x2 steps)
    constexpr int kStages = kGroups32 ? 2 : 3;
    constexpr int kVecStride = kGroups32 ? TT : 16;
    constexpr int kRowBuf = kMfmaEpi ? A_ROWS * kVecStride : TT * A_ROWS;
    __shared__ __attribute__((aligned(16))) uintx4 ldsA[kStages][A_VECS];
    __shared__ __attribute__((aligned(16))) uintx4 ldsB[kStages][B_VECS];
    __shared__ __attribute__((aligned(32))) float ldsRow[kRowBuf];   // vec of the A tile

    unsigned bx, by;
    // Where the reduction side is the big operand the contracting mode is banded too (8 output tiles x 8 reduction
    // chunks per XCD instead of 64 output tiles on one chunk): the 256-row output tiles then stay in the XCD's L2.
    // Measured on N = 5e5, M = 1e4, d = 784: bytes fetched per launch 68 -> 38 GB (mean of both passes); the launch
    // time does not move (29.8 ms): the re-reads came out of the Infinity Cache.
    if constexpr (STORE) xcd_remap_banded(bx, by);
    else if (y_fastest) xcd_remap(bx, by, true);
    else xcd_remap_banded(bx, by);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform by construction: let the compiler know
    const int wa = wave % WVA, wb = wave / WVA;
    const int j = lane & 31, lg = lane >> 5;
    const int64_t bblk0 = (int64_t)bx * NBB;
    const int64_t a_tiles = (na_blocks + NAB - 1) / NAB;
    const int64_t at0 = (int64_t)by * a_tiles_per_chunk;
    int64_t at1 = at0 + a_tiles_per_chunk;
    if (at1 > a_tiles) at1 = a_tiles;

    float out[WB_FR][kMfmaEpi ? 1 : TT];          // per-lane FMA path: out[q][t] for this lane's output row
    constexpr int kOut2 = kMfmaEpi ? WB_FR * (kGroups32 ? kGroups32 : 1) : 1;
    floatx16 out2[kOut2];                         // MFMA path: lane = column t, registers = output rows; [q][group]
#pragma unroll
    for (int q = 0; q < WB_FR; q++)
#pragma unroll
        for (int t = 0; t < (kMfmaEpi ? 1 : TT); t++) out[q][t] = 0.f;
#pragma unroll
    for (int q = 0; q < kOut2; q++)
#pragma unroll
        for (int r = 0; r < 16; r++) out2[q][r] = 0.f;
    // Slot of (row r of the tile, column c) in ldsRow.  With 32 or 64 columns the column index is swizzled with the row
    // so that neither the writers (consecutive rows of one column) nor the readers (32 consecutive columns of one
    // row) meet in one bank.
    auto vec_slot = [](int r, int c) { return r * kVecStride + (kGroups32 ? (c ^ (r & (kVecStride - 1))) : c); };

    // The stages are filled by direct global-to-LDS loads (global_load_lds_dwordx4: lane l of the issuing wave
    // writes its 16 bytes at the wave-uniform LDS address + 16 l, which is the packed order), three k-steps deep,
    // without passing through registers.  The compiler does not order these loads against the LDS reads: the
    // vmcnt waits below do (the loop issues no other vector memory instruction).  Unit u of a stage is piece u % 3
    // of block u / 3 of the A tile, then of the B tile; blocks past the end re-read the last block (their rows get
    // zero weight / are not stored).
    // where this wave's units of a stage come from (wave-uniform; the lane and the k-step are added at issue)
    const uintx4 *unit_src[kUnitsPerWave];
    auto set_tile = [&](int64_t ablk0) {
#pragma unroll
        for (int i = 0; i < kUnitsPerWave; i++) {
            const int u = wave * kUnitsPerWave + i;
            const bool is_a = u < NAB * 3;
            const int blk = is_a ? u / 3 : (u - NAB * 3) / 3;
            int64_t b = (is_a ? ablk0 : bblk0) + blk;
            const int64_t last = (is_a ? na_blocks : nb_blocks) - 1;
            if (b > last) b = last;
            unit_src[i] = (is_a ? PA : PB) + b * ks_count * kBlockVecs + (u % 3) * 64;
        }
    };
    auto issue_stage = [&](int s, int stage) {
#pragma unroll
        for (int i = 0; i < kUnitsPerWave; i++) {
            const int u = wave * kUnitsPerWave + i;
            const bool is_a = u < NAB * 3;
            const int blk = is_a ? u / 3 : (u - NAB * 3) / 3;
            const uintx4 *src = unit_src[i] + s * kBlockVecs + lane;
            uintx4 *dst = is_a ? &ldsA[stage][(blk * 3 + u % 3) * 64] : &ldsB[stage][(blk * 3 + u % 3) * 64];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                             (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
        }
    };

    if (at0 < at1) {
        set_tile(at0 * NAB);
#pragma unroll
        for (int g = 0; g < kStages - 1; g++)
            if (g < ks_count) issue_stage(g, g);
    }
    for (int64_t at = at0; at < at1; at++) {
        const int64_t ablk0 = at * NAB;
        floatx16 acc[WA_FR][WB_FR];
#pragma unroll
        for (int p = 0; p < WA_FR; p++)
#pragma unroll
            for (int q = 0; q < WB_FR; q++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[p][q][r] = 0.f;

        // the tile's right-hand side values: loaded, then written to ldsRow once every wave has left the previous
        // tile's epilogue (the loads complete behind the two stages already in flight, so nothing is outstanding
        // when the k-steps start)
        constexpr int kRowVals = (kMfmaEpi ? kVecStride : TT) * A_ROWS;
        constexpr int kRowValsPerThread = (kRowVals + kThreads - 1) / kThreads;
        // value c of a thread: column tid / A_ROWS + c * kColStep of row tid % A_ROWS; the column step is the same for
        // every thread, so that the addresses differ by multiples of a wave-uniform stride (worked out per thread
        // they are 2 x kRowValsPerThread registers that the compiler keeps across the tile loop)
        static_assert(kThreads % A_ROWS == 0, "a thread's values must lie in one row of the tile");
        constexpr int kColStep = kThreads / A_ROWS;
        float rowv[kRowValsPerThread];
        {
            const int col0 = tid / A_ROWS;
            const int64_t row = ablk0 * 32 + tid % A_ROWS;
            const bool row_ok = row < na_blocks * 32;     // rows past n_a carry zero weight
            const float *src = vecp + (int64_t)col0 * vec_ld + row;
#pragma unroll
            for (int c = 0; c < kRowValsPerThread; c++) {
                const int which = col0 + c * kColStep;
                float val = 0.f;
                if (tid + c * kThreads < kRowVals && row_ok && which < tcols) val = src[(int64_t)(c * kColStep) * vec_ld];
                rowv[c] = val;
            }
        }
        wg_barrier();
        {
            // (opaque, so that the swizzled slots are worked out here and not kept in registers across the tile loop)
            int r = tid % A_ROWS, col0 = tid / A_ROWS;
            asm volatile("" : "+v"(r), "+v"(col0));
#pragma unroll
            for (int c = 0; c < kRowValsPerThread; c++) {
                if (tid + c * kThreads < kRowVals) {
                    if (!kMfmaEpi) ldsRow[tid + c * kThreads] = rowv[c];
                    else ldsRow[vec_slot(r, col0 + c * kColStep)] = rowv[c];
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

        for (int s = 0; s < ks_count; s++) {
            const int stage = s % kStages;
            // this wave's loads of k-step s have landed (those of k-step s + 1 may still be in flight); after the
            // barrier so have everybody's, and every wave has finished reading the stage that k-step s + 2 goes to
            if (kStages == 3 && s + 1 < ks_count) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kUnitsPerWave) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            wg_barrier();
            // operands: the B fragments' three pieces stay in registers for the k-step, the A fragments come one piece
            // at a time (lo, mid, hi: partial products roughly from the lowest order up), each LDS vector read once
            // (read order: what the first partial product needs comes first, lo of A and hi of B)
            uintx4 b[WB_FR][3], a_first[WA_FR];
#pragma unroll
            for (int q = 0; q < WB_FR; q++) b[q][0] = ldsB[stage][((wb * WB_FR + q) * 3 + 0) * 64 + lane];
#pragma unroll
            for (int p = 0; p < WA_FR; p++) a_first[p] = ldsA[stage][((wa * WA_FR + p) * 3 + 2) * 64 + lane];
#pragma unroll
            for (int c = 1; c < 3; c++)
#pragma unroll
                for (int q = 0; q < WB_FR; q++) b[q][c] = ldsB[stage][((wb * WB_FR + q) * 3 + c) * 64 + lane];
            // B role, last k-step: the pair (1.0, h) in the last dword of the upper lane half becomes (h, 1.0)
            if (s + 1 == ks_count && lg) {
#pragma unroll
                for (int q = 0; q < WB_FR; q++)
#pragma unroll
                    for (int c = 0; c < 3; c++) b[q][c][3] = (b[q][c][3] >> 16) | (b[q][c][3] << 16);
            }
            // A piece -> the B pieces it meets: lo x hi | mid x (mid, hi) | hi x (lo, mid, hi)
            constexpr int kPieceOrder[3] = {2, 1, 0};
            constexpr int kPartners[3][3] = {{2, 1, 0}, {1, 0, -1}, {0, -1, -1}};   // indexed by A piece
#pragma unroll
            for (int o = 0; o < 3; o++) {
                const int ca = kPieceOrder[o];
                uintx4 a[WA_FR];
#pragma unroll
                for (int p = 0; p < WA_FR; p++)
                    a[p] = o == 0 ? a_first[p] : ldsA[stage][((wa * WA_FR + p) * 3 + ca) * 64 + lane];
#pragma unroll
                for (int w = 0; w < 3; w++) {
                    const int cb = kPartners[ca][w];
                    if (cb < 0) continue;
#pragma unroll
                    for (int p = 0; p < WA_FR; p++)
#pragma unroll
                        for (int q = 0; q < WB_FR; q++)
                            acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bits_as_bf16x8(a[p]), bits_as_bf16x8(b[q][cb]),
                                                                                acc[p][q], 0, 0, 0);
                }
                // the loads of a later k-step go out behind the first group of MFMAs, not in front of it: right
                // after the barrier every wave of the CU would otherwise be issuing loads while the matrix cores idle
                if (o == 0 && s + kStages - 1 < ks_count) issue_stage(s + kStages - 1, (s + kStages - 1) % kStages);
            }
        }
        // every wave has read its last operands once it passes this barrier: the first two k-steps of the next
        // tile go out before the epilogue and land while it runs
        wg_barrier();
        if (at + 1 < at1) {
            set_tile((at + 1) * NAB);
#pragma unroll
            for (int g = 0; g < kStages - 1; g++)
                if (g < ks_count) issue_stage(g, g);
        }

        // epilogue: K = kernel_value(acc) ; out[q][t] += K * vec[i][t]
        if constexpr (STORE) {
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
                const int64_t ablk = ablk0 + wa * WA_FR + p;
                if (ablk < na_blocks) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int64_t row0 = ablk * 32 + TR::group_off(g, lg);       // four consecutive rows
                        const floatx4 ha = *(const floatx4 *)(hnA + row0);
#pragma unroll
                        for (int q = 0; q < WB_FR; q++) {
                            const int64_t bb = bblk0 + wb * WB_FR + q;
                            if (bb < nb_blocks) {
                                const int64_t col = bb * 32 + j;
                                const float hb = hnB[col];
#pragma unroll
                                for (int e = 0; e < 4; e++) {
                                    const float h = ha[e] + hb;                       // h - h: 0, or NaN for a bad row
                                    const float k = kernel_value<KF>(acc[p][q][4 * g + e]) + (h - h);
                                    if (row0 + e < n_a && col < n_b)
                                        __builtin_nontemporal_store(k, &kout[(row0 + e) * kout_ld + col]);
                                }
                            }
                        }
                    }
                }
            }
        } else if constexpr (!kMfmaEpi) {
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
        } else if constexpr (kGroups32 > 0) {
            // 32 columns per group with the 32x32x2 step: accumulator register s2 of lane l is K[i][j] with i =
            // acc_row(s2, lg), j = l % 32, i.e. its A operand for the pair of rows (lg = 0, 1); the B operand is
            // vec[acc_row(s2, lg)][32 g + l % 32]; a lane ends up with column 32 g + l % 32 of output rows acc_row(r, lg).
            // The lane's part of the slot (vec_slot with r = 32 (wa WA_FR + p) + acc_row(s2, lg) and c = 32 g + j) is
            // kept opaque: computed in the open, the compiler works out all 64 or 128 read addresses in front of the
            // tile loop and spills them.
            int lane_off = (wa * WA_FR * 32 + 4 * lg) * kVecStride, lane_col = j ^ (4 * lg);
            asm volatile("" : "+v"(lane_off), "+v"(lane_col));
            auto read_vec = [&](int p, int s2, int g) {
                const int rc = p * 32 + 8 * (s2 >> 2) + (s2 & 3);      // the row without the lane's part (a constant)
                return ldsRow[lane_off + rc * kVecStride + ((32 * g + lane_col) ^ (rc & (kVecStride - 1)))];
            };
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
#pragma unroll
                for (int q = 0; q < WB_FR; q++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[p][q][r] = kernel_value<KF>(acc[p][q][r]);
                float bval[kGroups32], bnext[kGroups32];
#pragma unroll
                for (int g = 0; g < kGroups32; g++) bval[g] = read_vec(p, 0, g);
#pragma unroll
                for (int s2 = 0; s2 < 16; s2++) {
                    if (s2 + 1 < 16) {
#pragma unroll
                        for (int g = 0; g < kGroups32; g++) bnext[g] = read_vec(p, s2 + 1, g);
                    }
#pragma unroll
                    for (int g = 0; g < kGroups32; g++)
#pragma unroll
                        for (int q = 0; q < WB_FR; q++)
                            out2[q * kGroups32 + g] = __builtin_amdgcn_mfma_f32_32x32x2f32(acc[p][q][s2], bval[g],
                                                                                           out2[q * kGroups32 + g], 0, 0, 0);
                    // one read ahead, fenced (otherwise all reads are hoisted to the front and spilled)
#pragma unroll
                    for (int g = 0; g < kGroups32; g++) {
                        asm volatile("" : "+v"(bval[g]) : : "memory");
                        bval[g] = bnext[g];
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
            // out2[q][j-rows][t] += sum_i K[i][j] vec[i][t] with the four-block fp32 16x16x1 step (half the cycles of a
            // 32x32x2 step, which would leave 16 of its 32 columns unused): as its A operand, accumulator register s2
            // of lane l is K[i][j] with i = acc_row(s2, lg), j = l % 32, so block b = l / 16 holds the output rows
            // 16 (b & 1) .. + 15 against the row of lane half b >> 1; its B operand is vec[acc_row(s2, lg)][t = l % 16],
            // which is what the lanes of that quarter read.  Block b accumulates in registers 4 b .. 4 b + 3 (output
            // row 16 (b & 1) + 4 (lane / 16) + r, column lane % 16): blocks b and b + 2 are partial sums of the same
            // outputs, added at the store.
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
                    for (int q = 0; q < WB_FR; q++)
                        out2[q] = __builtin_amdgcn_mfma_f32_16x16x1f32(acc[p][q][s2], bval, out2[q], 0, 0, 0);
                    asm volatile("" : "+v"(bval) : "v"(vb) : "memory");
                    bval = bnext;
                }
            }
        }
    }

    if constexpr (STORE) {
        // nothing left to write
    } else if constexpr (kGroups32 > 0) {
#pragma unroll
        for (int g = 0; g < kGroups32; g++) {
            const int t = 32 * g + j;
            if (t < tcols) {
#pragma unroll
                for (int q = 0; q < WB_FR; q++) {
                    const int64_t bb = bblk0 + wb * WB_FR + q;
                    if (bb < nb_blocks) {
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            partial[(((int64_t)by * WVA + wa) * tcols + t) * nb_pad + bb * 32 + TR::acc_row(r, lg)] =
                                out2[q * kGroups32 + g][r];
                    }
                }
            }
        }
    } else if constexpr (kMfmaEpi) {
        const int tl = lane & 15, mq = lane >> 4;
        if (tl < tcols) {
#pragma unroll
            for (int q = 0; q < WB_FR; q++) {
                const int64_t bb = bblk0 + wb * WB_FR + q;
                if (bb < nb_blocks) {
#pragma unroll
                    for (int b = 0; b < 2; b++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            partial[(((int64_t)by * WVA + wa) * tcols + tl) * nb_pad + bb * 32 + 16 * b + 4 * mq + r] =
                                out2[q][4 * b + r] + out2[q][4 * (b + 2) + r];
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

// 8 waves (2 x 4) with 4 x 2 accumulators each, one workgroup per CU (two waves per SIMD); tile 256 (A) x 256 (B)
// rows: every operand read from LDS feeds two or four MFMAs, and a k-step (48 MFMAs per wave) outlasts the latency
// of the next k-step's loads
constexpr int kSLWavesA = 2, kSLWavesB = 4, kSLFragsA = 4, kSLFragsB = 2;

#if FLK_KF == FLK_GAUSSIAN   // the tile geometry is the same for every kernel function: defined once
int split_large_a_tile_blocks() { return kSLWavesA * kSLFragsA; }
int split_large_b_tile_blocks() { return kSLWavesB * kSLFragsB; }
int split_large_partials_per_split() { return kSLWavesA; }
int split_large_max_cols() { return 64; }
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

// The kernel matrix out[a][b] = K(A_a, B_b) in the bf16x3 mode: one workgroup per (A tile, B tile), or a few A tiles
// per workgroup where the grid would not hold them all.
int FLK_CAT(launch_fmm_split_large_kf, FLK_KF)(const SplitView &A, const SplitView &B, float *out, int64_t ld,
                                               hipStream_t st) {
    if (A.ks != B.ks || A.d != B.d)
        return fail(FLK_EINVAL, "fmm (bf16x3): operands packed with different feature counts");
    if (A.n == 0 || B.n == 0) return FLK_OK;
    if (A.hnorm == nullptr || B.hnorm == nullptr) return fail(FLK_EINVAL, "fmm (bf16x3): operands without half norms");
    const int64_t nab = kSLWavesA * kSLFragsA, nbb = kSLWavesB * kSLFragsB;
    const int64_t a_tiles = (A.nblk + nab - 1) / nab;
    const int64_t per_wg = (a_tiles + 65534) / 65535;
    dim3 grid((unsigned)((B.nblk + nbb - 1) / nbb), (unsigned)((a_tiles + per_wg - 1) / per_wg));
    hipLaunchKernelGGL((mmv_split_large_kernel<kSLWavesA, kSLWavesB, kSLFragsA, kSLFragsB, 1, FLK_KF, true>), grid,
                       dim3(64 * kSLWavesA * kSLWavesB), 0, st, (const uintx4 *)A.data, (const float *)nullptr,
                       (int64_t)0, 0, (const uintx4 *)B.data, A.nblk, B.nblk, (int)A.ks, per_wg, (float *)nullptr,
                       B.npad, B.n > A.n, out, ld, A.n, B.n, A.hnorm, B.hnorm);
    FLK_LAUNCH_CHECK("mmv_split_large_kernel (kernel matrix)");
    return FLK_OK;
}

int FLK_CAT(launch_mmv_split_large_kf, FLK_KF)(const SplitView &A, const SplitView &B, const float *vecp,
                                               int64_t vec_ld, int tcols, int64_t a_tiles_per_chunk, int splits,
                                               float *partial, hipStream_t st) {
    if (A.ks != B.ks || A.d != B.d)
        return fail(FLK_EINVAL, "mmv_split_large: operands packed with different feature counts");
    if (tcols < 1 || tcols > 64) return fail(FLK_EINVAL, "mmv_split_large: column chunk %d not in 1..64", tcols);
    if (tcols == 1) return launch_split_large_tt<1>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    if (tcols == 2) return launch_split_large_tt<2>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    if (tcols <= 4) return launch_split_large_tt<4>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    if (tcols <= 16) return launch_split_large_tt<16>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    if (tcols <= 32) return launch_split_large_tt<32>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
    return launch_split_large_tt<64>(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st);
}

}  // namespace flk
