// LDS-tiled Gaussian kernel-vector product for large feature counts (d > 64), fp32 and fp64, gfx950.
//
//   partial[split'][t][b] = sum_{a in chunk} exp2(A~_a . B~_b + hA_a + hB_b) * vec[a,t]
//
// A workgroup owns one tile of output rows (B side) and walks over the tiles of
// reduction rows (A side) of its chunk.  For every (A tile, B tile) the cross term is a GEMM over
// the features: feature chunks of both tiles are staged in LDS (double buffered, one barrier per
// chunk, 16-byte global loads straight from the packed layout, which is already in operand order),
// every wave keeps a WA_FR x WB_FR grid of MFMA accumulators in registers.  After the last feature
// chunk the accumulators hold x~.c~; the epilogue adds the half norms, applies exp2 with the clamp,
// and contracts the tile against vec into per-lane output accumulators that live in registers for
// the whole kernel.  K is never written anywhere.
//
// Waves are arranged WVA (A) x WVB (B); waves with the same wb produce partial sums for the same
// output rows and simply write separate partials (they count as extra splits for the reduction).
//
// Right-hand sides per pass: up to 4 (fp32) / 8 (fp64) are contracted with per-lane FMAs; beyond, a second MFMA takes
// the kernel values in the accumulator registers as its A operand and a 16-column (fp32 also 32-column) slice of vec
// as its B operand, and up to 64 columns ride on one evaluation of K as two groups of 32 (fp32) or four of 16 (fp64).
// Measured, dfmmv at N = 5e5, M = 1e4, d = 784: fp32 T = 16 123.4 ms, 32 132.2, 64 149.0 (four passes of 16: 494);
// fp64 T = 16 258.9, 32 262.7, 64 287.1 (1036).  N = 5e5, M = 2e4, d = 100: fp32 47.0 / 50.6 / 84.4, fp64 89.2 / 97.9 / 131.8.
#include <type_traits>

#include "flk_common.h"
#include "kernel_fn.h"
#include "mfma_traits.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

// Right-hand sides up to which the epilogue contracts with per-lane FMAs (measured: the MFMA contraction is the
// faster one from five columns on in fp32, from nine on in fp64, where it costs four 64-cycle MFMAs per 16 x 16 tile).
template <typename T> constexpr int kLargeFmaCols = sizeof(T) == 8 ? 8 : 4;

template <typename T, int WVA, int WVB, int WA_FR, int WB_FR, int KC> struct LGeo {
    typedef LTraits<T> TR;
    static constexpr int kLWavesA = WVA, kLWavesB = WVB, kLThreads = 64 * WVA * WVB;
    static_assert(kLargeKChunk % KC == 0, "packed features are padded to kLargeKChunk steps");
    static constexpr int NAB = kLWavesA * WA_FR;             // A blocks per tile
    static constexpr int NBB = kLWavesB * WB_FR;             // B blocks per tile
    static constexpr int A_ROWS = NAB * TR::BLK, B_ROWS = NBB * TR::BLK;
    static constexpr int A_ELEMS = NAB * KC * 64, B_ELEMS = NBB * KC * 64;   // per stage
    static constexpr int A_VECS = A_ELEMS / TR::VPL, B_VECS = B_ELEMS / TR::VPL;
    static constexpr int A_VPT = A_VECS / kLThreads;      // 16-byte vectors per thread
    static constexpr int B_VPT = B_VECS / kLThreads;
    static_assert(A_VECS % kLThreads == 0 && B_VECS % kLThreads == 0, "stage must split evenly over the threads");
};

// One 16-byte piece of a stage: vector index vi enumerates [block][step][lane group][row/VPL], which is
// also the order in LDS, so the LDS side of the copy is linear.  MFMA step s contracts the features
// KG s .. KG s + KG - 1 (lane group lg takes feature KG s + lg), so a step's operands are adjacent rows of the
// packed block and the zero padding past d sits in the last steps of the last chunk, which the kernel skips.
// The packed feature count is a whole number of chunks (padded_features), so there is no feature tail to mask.
template <typename T, int KC, bool SCALAR_BLK = false>
__device__ __forceinline__ const T *stage_src(const T *__restrict__ P, int64_t blk0, int64_t nblk, int64_t dpad,
                                              int64_t s0, int vi) {
    typedef LTraits<T> TR;
    constexpr int VPB = TR::BLK / TR::VPL;
    const int jv = vi % VPB;
    const int lg = (vi / VPB) % TR::KG;
    const int s = (vi / (VPB * TR::KG)) % KC;
    // A block's vectors of a chunk are a whole number of waves: the block is the same for the 64 lanes.  SCALAR_BLK
    // says so to the compiler, which then keeps the blocks' base addresses in scalar registers.  That pays where the
    // vector registers are short (the fp32 passes of 48 and 64 columns otherwise reload spilled addresses in every
    // chunk: N = 5e5, M = 1e4, d = 784, 64 columns 138.3 -> 135.9 ms, d = 300 at N = 2.5e5, M = 2e4 62.8 -> 61.2) and costs
    // elsewhere (16 columns at d = 784: 120.0 -> 126.8 ms, fp64 248.6 -> 269.1).
    static_assert((VPB * TR::KG * KC) % 64 == 0, "a wave's vectors must belong to one block");
    const int blk = SCALAR_BLK ? __builtin_amdgcn_readfirstlane(vi / (VPB * TR::KG * KC)) : vi / (VPB * TR::KG * KC);
    int64_t b = blk0 + blk;
    if (b >= nblk) b = nblk - 1;                 // past the end: any valid block (its rows get zero weight / are not stored)
    return P + (b * dpad + (s0 + s) * TR::KG + lg) * TR::BLK + jv * TR::VPL;
}

// The same address as a scalar base (block and chunk: the same for the 64 lanes of a wave) plus the lane's 32-bit offset
// inside the chunk, which does not change from chunk to chunk or tile to tile.
template <typename T, int KC>
__device__ __forceinline__ int stage_lane_offset(int vi) {
    typedef LTraits<T> TR;
    constexpr int VPB = TR::BLK / TR::VPL;
    const int jv = vi % VPB, lg = (vi / VPB) % TR::KG, s = (vi / (VPB * TR::KG)) % KC;
    return (s * TR::KG + lg) * TR::BLK + jv * TR::VPL;
}
template <typename T, int KC>
__device__ __forceinline__ auto stage_base(const T *__restrict__ P, int64_t blk0, int64_t nblk, int64_t dpad, int vi) {
    typedef LTraits<T> TR;
    constexpr int VPB = TR::BLK / TR::VPL;
    int64_t b = blk0 + __builtin_amdgcn_readfirstlane(vi / (VPB * TR::KG * KC));
    if (b >= nblk) b = nblk - 1;                 // past the end: any valid block (its rows get zero weight / are not stored)
    return scalar_base(P + b * dpad * TR::BLK);
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
// O = void: the product (partial sums of K against vec).  O = an element type: the kernel matrix itself, entry
// (a, b) stored as O at kout[a * kout_ld + b] (then TT = 1, vecp is not read and partial not written).
template <typename T, int WVA, int WVB, int WA_FR, int WB_FR, int KC, int TT, int KF, typename O = void>
__global__ void __launch_bounds__(64 * WVA * WVB, (WVA * WVB == 4 ? 2 : 1))   // two waves per SIMD either way
    mmv_large_kernel(const T *__restrict__ PA, const T *__restrict__ hA, const T *__restrict__ vecp, int64_t vec_ld,
                     int tcols, const T *__restrict__ PB, const T *__restrict__ hB, int64_t na_blocks,
                     int64_t nb_blocks, int64_t dpad, int n_chunks_used, int last_steps, int64_t a_tiles_per_chunk,
                     T *__restrict__ partial, int64_t nb_pad, bool y_fastest, void *__restrict__ kout = nullptr,
                     int64_t kout_ld = 0, int64_t n_a = 0, int64_t n_b = 0) {
    constexpr bool kStore = !std::is_void<O>::value;
    typedef LTraits<T> TR;
    typedef LGeo<T, WVA, WVB, WA_FR, WB_FR, KC> G;
    constexpr int kLWavesA = WVA, kLWavesB = WVB, kLThreads = 64 * WVA * WVB;
    typedef typename TR::acc_t acc_t;
    typedef typename TR::vec4_t vec4_t;
    typedef typename TR::v16_t V16;

    __shared__ __attribute__((aligned(16))) T ldsA[2][G::A_ELEMS];
    __shared__ __attribute__((aligned(16))) T ldsB[2][G::B_ELEMS];
    // More than four (fp32) / eight (fp64) columns: the contraction against vec runs on the MFMA as well (a second,
    // small GEMM whose A operand are the kernel values sitting in the accumulator registers, see the epilogue), with vec staged
    // as [row][16 or 32 columns] at an odd stride.  Fewer columns: per-lane FMAs, vec staged planar.
    // fp32: the 32x32x2 step has room for 32 columns (lane % 32), fp64's 16x16x4 for 16.
    constexpr bool kMfmaEpi = TT > kLargeFmaCols<T>;
    // fp64 with one column: the accumulators of a lane all belong to one output row j and start from hB_j, one
    // addition per kernel value less in the epilogue (measured, dfmmv at N = 5e5, M = 2e4: d = 65 51.4 -> 50.1 ms,
    // 128 86.0 -> 84.2, 784 472.1 -> 463.7; with four columns, with the MFMA epilogue and in fp32 it is a loss of up to 1 %)
    constexpr bool kSeeded = !kStore && sizeof(T) == 8 && TT == 1;
    // More columns than one step holds: NC groups of columns ride on the same kernel values (one more contraction
    // per group, NC times the output accumulators).
    constexpr int kGroupCols = (sizeof(T) == 4 && TT > 16) ? 32 : 16;
    // fp32 with 48 columns: a group of 32 and, as the second group, 16 columns on the four-block 16x16x1 step
    constexpr bool kTail16 = kMfmaEpi && sizeof(T) == 4 && TT == 48;
    constexpr int NC = kTail16 ? 2 : (kMfmaEpi && TT > kGroupCols) ? TT / kGroupCols : 1;
    constexpr int kEpiCols = kTail16 ? 48 : kGroupCols * NC;
    // fp32 with up to 16 columns: the four-block 16x16x1 step contracts them in half the cycles of a 32x32x2 step that
    // would leave half of its columns unused (see the epilogue)
    constexpr bool kHalf16 = kMfmaEpi && sizeof(T) == 4 && kGroupCols == 16;
    static_assert(TT <= kEpiCols || !kMfmaEpi, "columns per pass must be a whole number of column groups");
    constexpr int kVecStride = kEpiCols + 1;
    constexpr int kRowBuf = kMfmaEpi ? G::A_ROWS * (1 + kVecStride) : (1 + TT) * G::A_ROWS;
    __shared__ __attribute__((aligned(32))) T ldsRow[kRowBuf];   // [hA | vec ...] of the A tile
    // fp64 products: 2^x from the table in LDS (kernel_fn.h; 16 KB beside the stages and the row values).  The epilogue is
    // a fixed cost per kernel value, so this pays where a tile has few feature chunks: N = 5e5, M = 2e4, dfmmv, one column,
    // d = 65 54.4 -> 51.7 ms, 100 73.0 -> 70.5, 128 89.0 -> 86.1, 300 189.0 -> 188.0, 784 unchanged; 10 columns 1 to 3 %.
    constexpr bool kExpTab = sizeof(T) == 8 && !kStore;
    __shared__ double exp_tab[kExpTab ? kExpTableSize : 1];
    if constexpr (kExpTab) {
        exp2_table_fill(exp_tab, threadIdx.x, kLThreads);
        __syncthreads();
    }
    auto kval = [&](T e) -> T {
        if constexpr (kExpTab) return (T)kernel_value<FLK_KF, true>((double)e, exp_tab);
        else return kernel_value<FLK_KF>(e);
    };

    unsigned bx, by;
    // (Banding the contracting mode as well was measured on N = 5e5, M = 1e4, d = 784: bytes fetched per launch
    // 62 -> 93 GB, launch time unchanged at 60.8 ms: the re-reads come out of the Infinity Cache and do not bound
    // the kernel, whose matrix pipe is 88 % busy.)
    if constexpr (kStore) xcd_remap_banded(bx, by);
    else xcd_remap(bx, by, y_fastest);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wa = wave % kLWavesA, wb = wave / kLWavesA;
    const int j = lane % TR::BLK, lg = lane / TR::BLK;
    const int64_t DPsteps = dpad / TR::KG;
    const int64_t bblk0 = (int64_t)bx * G::NBB;
    const int64_t a_tiles = (na_blocks + G::NAB - 1) / G::NAB;
    const int64_t at0 = (int64_t)by * a_tiles_per_chunk;
    int64_t at1 = at0 + a_tiles_per_chunk;
    if (at1 > a_tiles) at1 = a_tiles;
    // chunks of KC steps that hold features of the data; the last of them stops after last_steps steps (dpad is padded
    // to whole chunks of kLargeKChunk steps: what lies past the data is zero and is never read)
    const int64_t n_chunks = n_chunks_used;

    // half norms of this lane's output rows
    T hb[WB_FR];
#pragma unroll
    for (int q = 0; q < WB_FR; q++) {
        int64_t bb = bblk0 + wb * WB_FR + q;
        if (bb >= nb_blocks) bb = nb_blocks - 1;
        hb[q] = hB[bb * TR::BLK + TR::out_row(j)];
    }
    T out[WB_FR][kMfmaEpi ? 1 : TT];          // per-lane FMA path: out[q][t] for this lane's output row
    acc_t out2[kMfmaEpi ? WB_FR : 1][NC];     // MFMA path: lane = column t (of every group), registers = output rows
#pragma unroll
    for (int q = 0; q < WB_FR; q++)
#pragma unroll
        for (int t = 0; t < (kMfmaEpi ? 1 : TT); t++) out[q][t] = T(0);
#pragma unroll
    for (int q = 0; q < (kMfmaEpi ? WB_FR : 1); q++)
#pragma unroll
        for (int g = 0; g < NC; g++)
#pragma unroll
            for (int r = 0; r < TR::ACCN; r++) out2[q][g][r] = T(0);

    // where a thread's staged vectors come from: offsets inside a chunk (fixed), bases of the output tile's blocks (fixed)
    int aoff[G::A_VPT], boff[G::B_VPT];
    decltype(scalar_base(PB)) bbase[G::B_VPT];
#pragma unroll
    for (int c = 0; c < G::A_VPT; c++) aoff[c] = stage_lane_offset<T, KC>(tid + c * kLThreads);
#pragma unroll
    for (int c = 0; c < G::B_VPT; c++) {
        boff[c] = stage_lane_offset<T, KC>(tid + c * kLThreads);
        bbase[c] = stage_base<T, KC>(PB, bblk0, nb_blocks, dpad, tid + c * kLThreads);
    }

    for (int64_t at = at0; at < at1; at++) {
        const int64_t ablk0 = at * G::NAB;
        acc_t acc[WA_FR][WB_FR];
#pragma unroll
        for (int p = 0; p < WA_FR; p++)
#pragma unroll
            for (int q = 0; q < WB_FR; q++)
#pragma unroll
                for (int r = 0; r < TR::ACCN; r++) acc[p][q][r] = kSeeded ? hb[q] : T(0);

        V16 ra[G::A_VPT], rb[G::B_VPT];
        constexpr bool kScalarBlk = sizeof(T) == 4 && TT >= 48;
        // global addresses: a scalar base per staged block (the tile's blocks; the chunk adds a scalar offset) plus the
        // lane's 32-bit offset inside a chunk
        typedef const V16 __attribute__((address_space(1))) *global_v16;
        decltype(scalar_base(PA)) abase[G::A_VPT];
#pragma unroll
        for (int c = 0; c < G::A_VPT; c++) abase[c] = stage_base<T, KC>(PA, ablk0, na_blocks, dpad, tid + c * kLThreads);
        typedef const T __attribute__((address_space(1))) *global_t;
        auto fetch = [&](int64_t chunk) {
            const int64_t s0 = chunk * (KC * TR::KG * TR::BLK * (int64_t)sizeof(T));      // bytes
#pragma unroll
            for (int c = 0; c < G::A_VPT; c++) ra[c] = *(global_v16)((global_t)as_scalar((int64_t)abase[c] + s0) + aoff[c]);
#pragma unroll
            for (int c = 0; c < G::B_VPT; c++) rb[c] = *(global_v16)((global_t)as_scalar((int64_t)bbase[c] + s0) + boff[c]);
        };
        auto commit = [&](int buf) {
#pragma unroll
            for (int c = 0; c < G::A_VPT; c++) *(V16 *)(&ldsA[buf][(tid + c * kLThreads) * TR::VPL]) = ra[c];
#pragma unroll
            for (int c = 0; c < G::B_VPT; c++) *(V16 *)(&ldsB[buf][(tid + c * kLThreads) * TR::VPL]) = rb[c];
        };

        // Prologue of an A tile.  All global loads (first feature chunk, then the per-row values hA and vec)
        // are issued before anything waits, and the barrier that protects ldsRow and the stages from the
        // previous tile's epilogue comes after them, so one memory round trip covers the whole prologue.
        // (Loading the next tile's first chunk and row values during this tile's last chunk and epilogue, into the
        // then idle prefetch registers, was measured over d = 65 .. 1000 and 1 .. 64 columns: 1 to 2 % faster up to four
        // columns, 4 to 15 % slower with the MFMA epilogue below 200 features, whose 17 to 33 row values per thread then
        // spill; not kept.)
        fetch(0);
        constexpr int kRowVals = (1 + (kMfmaEpi ? kEpiCols : TT)) * G::A_ROWS;
        constexpr int kRowValsPerThread = (kRowVals + kLThreads - 1) / kLThreads;
        T rowv[kRowValsPerThread];
        // A wave's 64 values belong to one vector (hA or one column of vec): its number is made a scalar, so that the
        // column's offset and the test against tcols are scalar work.  (The leading dimension goes through an empty asm
        // in every tile: otherwise the compiler forms one pointer per row value ahead of the tile loop, up to 33 of
        // them, and keeps them in scratch memory.)
        static_assert(G::A_ROWS % 64 == 0 && kLThreads % 64 == 0, "a wave's row values must belong to one vector");
        // (not for fp64 with 32 columns, measured: C4's shape 260.7 ms per dfmmv against 265.4 with, where 16 columns take
        // 251.5 against 260.1 and 64 columns 279.1 against 283.6)
        constexpr bool kScalarWhich = sizeof(T) == 4 || TT != 32;
        int64_t vld = vec_ld;
        if constexpr (kScalarWhich) asm volatile("" : "+s"(vld));
#pragma unroll
        for (int c = 0; c < kRowValsPerThread; c++) {
            const int e = tid + c * kLThreads;
            const int which = kScalarWhich ? __builtin_amdgcn_readfirstlane(e / G::A_ROWS) : e / G::A_ROWS, r = e % G::A_ROWS;
            const int64_t row = ablk0 * TR::BLK + r;
            T val = T(0);                      // rows past n_a carry zero weight
            if (e < kRowVals && row < na_blocks * TR::BLK) {
                if (which == 0) val = hA[row];
                else if (which - 1 < tcols) val = vecp[(int64_t)(which - 1) * vld + row];
            }
            rowv[c] = val;
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < kRowValsPerThread; c++) {
            const int e = tid + c * kLThreads;
            const int which = kScalarWhich ? __builtin_amdgcn_readfirstlane(e / G::A_ROWS) : e / G::A_ROWS, r = e % G::A_ROWS;
            if (e < kRowVals) {
                if (!kMfmaEpi || which == 0) ldsRow[e] = rowv[c];
                else ldsRow[G::A_ROWS + r * kVecStride + (which - 1)] = rowv[c];
            }
        }
        commit(0);
        __syncthreads();

        // Operands are read from LDS one step ahead of the MFMAs that use them.  The empty asm between a
        // step's reads (for the next step) and its MFMAs is a compiler fence: it redefines the accumulators
        // (so the MFMAs of this step stay below it and those of the previous step above it) and clobbers
        // memory through the LDS pointers (so reads stay on their side of it).  Left alone the compiler
        // either hoists all KC steps' reads to the top of the chunk, which costs ~40 registers and pushes
        // the global prefetch registers around, or issues each step's reads right before their use.
        //
        // Chunk schedule: the next chunk's global loads are issued at the top, written to the other LDS
        // stage in the middle of the chunk (that stage has not been read since the previous barrier), and
        // the one barrier of the chunk sits BEFORE the last step's MFMAs: by then every wave holds its last
        // operands in registers, so right after the barrier a wave issues the reads of the next chunk's
        // first step and covers their latency with the MFMAs it still has to issue.
        static_assert((WA_FR == 4 || WA_FR == 8) && WB_FR == 2, "the step fence lists its operands explicitly");
        constexpr int kCommitStep = KC / 2;
        static_assert(KC % 2 == 0, "the two operand sets alternate by step and must line up across chunks");
        T av[2][WA_FR], bv[2][WB_FR];          // operand sets: step s uses set s%2 while set (s+1)%2 is being read
        {
            const T *la = &ldsA[0][(wa * WA_FR) * KC * 64 + lane];
            const T *lb = &ldsB[0][(wb * WB_FR) * KC * 64 + lane];
#pragma unroll
            for (int p = 0; p < WA_FR; p++) av[0][p] = la[(p * KC) * 64];
#pragma unroll
            for (int q = 0; q < WB_FR; q++) bv[0][q] = lb[(q * KC) * 64];
        }
        // The last chunk is a variant of its own (kLast): nothing to prefetch, no barrier (the next tile's prologue
        // has one before it writes LDS), and it stops after last_steps steps: the features past d in it are padding.
        auto run_chunk = [&](auto last_tag, const int buf) {
            constexpr bool kLast = decltype(last_tag)::value;
            const T *la = &ldsA[buf][(wa * WA_FR) * KC * 64 + lane];
            const T *lb = &ldsB[buf][(wb * WB_FR) * KC * 64 + lane];
            const T *la2 = &ldsA[buf ^ 1][(wa * WA_FR) * KC * 64 + lane];
            const T *lb2 = &ldsB[buf ^ 1][(wb * WB_FR) * KC * 64 + lane];
#pragma unroll
            for (int s = 0; s < KC; s++) {
                if (kLast && s >= last_steps) break;
                const int cur = s & 1, nxt = cur ^ 1;
                if (s + 1 < KC) {
#pragma unroll
                    for (int p = 0; p < WA_FR; p++) av[nxt][p] = la[(p * KC + s + 1) * 64];
#pragma unroll
                    for (int q = 0; q < WB_FR; q++) bv[nxt][q] = lb[(q * KC + s + 1) * 64];
                } else if (!kLast) {
                    __syncthreads();          // all waves: this chunk's LDS reads done, next stage written
#pragma unroll
                    for (int p = 0; p < WA_FR; p++) av[nxt][p] = la2[(p * KC) * 64];
#pragma unroll
                    for (int q = 0; q < WB_FR; q++) bv[nxt][q] = lb2[(q * KC) * 64];
                }
                asm volatile("" : "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[1][0]), "+v"(acc[1][1]),
                                  "+v"(acc[2][0]), "+v"(acc[2][1]), "+v"(acc[3][0]), "+v"(acc[3][1])
                             : "v"(la), "v"(lb) : "memory");
                if constexpr (WA_FR == 8)
                    asm volatile("" : "+v"(acc[4][0]), "+v"(acc[4][1]), "+v"(acc[5][0]), "+v"(acc[5][1]),
                                      "+v"(acc[6][0]), "+v"(acc[6][1]), "+v"(acc[7][0]), "+v"(acc[7][1])
                                 : "v"(la), "v"(lb) : "memory");
#pragma unroll
                for (int p = 0; p < WA_FR; p++)
#pragma unroll
                    for (int q = 0; q < WB_FR; q++) acc[p][q] = TR::mfma(av[cur][p], bv[cur][q], acc[p][q]);
                if (!kLast && s == kCommitStep) commit(buf ^ 1);
            }
        };
        for (int64_t ch = 0; ch + 1 < n_chunks; ch++) {
            fetch(ch + 1);
            run_chunk(std::false_type{}, (int)(ch & 1));
        }
        run_chunk(std::true_type{}, (int)((n_chunks - 1) & 1));

        // epilogue: exponent = acc + hA_i + hB_j ; K = exp2 clamped ; out[q][t] += K * vec[i][t]
        // Columns are contracted in groups of four whose LDS reads are issued one group ahead; the fence
        // after each group (the updated accumulators pass through an empty asm that also clobbers memory
        // through the LDS pointer) keeps the compiler from moving every read to the front and spilling.
        static_assert(WB_FR == 2, "the epilogue fence lists its operands explicitly");
        if constexpr (kStore) {
            typedef typename std::conditional<kStore, O, T>::type OT;
            OT *dst = (OT *)kout;
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
#pragma unroll
                for (int g = 0; g < TR::NG; g++) {
                    const int ro = (wa * WA_FR + p) * TR::BLK + TR::group_off(g, lg);     // four consecutive rows
                    const vec4_t hn = *(const vec4_t *)(&ldsRow[ro]);
#pragma unroll
                    for (int q = 0; q < WB_FR; q++) {
                        const int64_t col = (bblk0 + wb * WB_FR + q) * TR::BLK + TR::out_row(j);
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            // h - h is 0, or NaN where a row holds a NaN or an infinity (the clamps would hide it)
                            const T h = hn[e] + hb[q];
                            const T k = kernel_value<FLK_KF>(acc[p][q][4 * g + e] + h) + (h - h);
                            const int64_t row = ablk0 * TR::BLK + ro + e;
                            if (row < n_a && col < n_b) __builtin_nontemporal_store((OT)k, &dst[row * kout_ld + col]);
                        }
                    }
                }
            }
        } else if constexpr (!kMfmaEpi) {
        constexpr int NTG = (TT + 3) / 4;
#pragma unroll
        for (int p = 0; p < WA_FR; p++) {
            const int rbase = (wa * WA_FR + p) * TR::BLK;
#pragma unroll
            for (int g = 0; g < TR::NG; g++) {
                const int ro = rbase + TR::group_off(g, lg);
                const vec4_t hn = *(const vec4_t *)(&ldsRow[ro]);
                vec4_t cur[4], nxt[4];
#pragma unroll
                for (int u = 0; u < 4; u++)
                    if (u < TT) cur[u] = *(const vec4_t *)(&ldsRow[(1 + u) * G::A_ROWS + ro]);
                T kv[WB_FR][4];
#pragma unroll
                for (int q = 0; q < WB_FR; q++)
#pragma unroll
                    for (int e = 0; e < 4; e++) kv[q][e] = kval(acc[p][q][4 * g + e] + (kSeeded ? hn[e] : hn[e] + hb[q]));
#pragma unroll
                for (int tg = 0; tg < NTG; tg++) {
                    const int t0 = 4 * tg;
                    if (tg + 1 < NTG) {
#pragma unroll
                        for (int u = 0; u < 4; u++)
                            if (t0 + 4 + u < TT) nxt[u] = *(const vec4_t *)(&ldsRow[(1 + t0 + 4 + u) * G::A_ROWS + ro]);
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        if (t0 + u < TT) {
#pragma unroll
                            for (int q = 0; q < WB_FR; q++)
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    out[q][t0 + u] = __builtin_fma(kv[q][e], cur[u][e], out[q][t0 + u]);
                        }
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        if (t0 + u < TT)
                            asm volatile("" : "+v"(out[0][t0 + u]), "+v"(out[1][t0 + u]) : "v"(&ldsRow[0]) : "memory");
#pragma unroll
                    for (int u = 0; u < 4; u++) cur[u] = nxt[u];
                }
            }
        }
        } else {
            // kernel values in place of the exponents
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
                const int rbase = (wa * WA_FR + p) * TR::BLK;
#pragma unroll
                for (int g = 0; g < TR::NG; g++) {
                    const vec4_t hn = *(const vec4_t *)(&ldsRow[rbase + TR::group_off(g, lg)]);
#pragma unroll
                    for (int q = 0; q < WB_FR; q++)
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            acc[p][q][4 * g + e] = kval(acc[p][q][4 * g + e] + (hn[e] + hb[q]));
                }
            }
            // out2[q][j-rows][t] += sum_i K[i][j] vec[i][t]: accumulator register s of a lane is exactly the MFMA
            // A operand of step s (row i = acc_row(s, lg), column j = lane), so K needs no data movement; the
            // B operand is vec[acc_row(s, lg)][t] with t = lane % kGroupCols (+ kGroupCols per further group).
            // The 16-column fp32 form uses the four-block 16x16x1 step instead: with the same A operand, block
            // b = lane / 16 holds the output rows 16 (b & 1) .. + 15 against the row of lane half b >> 1, its B operand is
            // vec[acc_row(s, lg)][t = lane % 16], which is what the lanes of that quarter read, and it accumulates in
            // registers 4 b .. 4 b + 3 (output row 16 (b & 1) + 4 (lane / 16) + r, column lane % 16); blocks b and
            // b + 2 are partial sums of the same outputs, added at the store.
            const int tl = j & (kGroupCols - 1);
            // index of this lane's first B value (step 0 of its wave row's first block); every other read lies a
            // compile-time constant further on
            const int lane_idx = G::A_ROWS + tl + ((wa * WA_FR) * TR::BLK + TR::acc_row(0, lg)) * kVecStride;
            // one read ahead, fenced like the feature loop (otherwise all reads are hoisted and spilled)
            // (the 16-column group behind a group of 32: its lanes 16 .. 31 read the columns of lanes 0 .. 15)
            const int tail_adj = kTail16 ? (j & 16) : 0;
            T bval[NC], bnext[NC];
#pragma unroll
            for (int g = 0; g < NC; g++) {
                bval[g] = ldsRow[lane_idx + g * kGroupCols - (kTail16 && g == 1 ? tail_adj : 0)];
                bnext[g] = T(0);
            }
#pragma unroll
            for (int p = 0; p < WA_FR; p++) {
#pragma unroll
                for (int s2 = 0; s2 < TR::ACCN; s2++) {
                    // the lane's offset goes through an empty asm before every read: the rows lie further apart than the
                    // offset field of a paired LDS read reaches, and from an offset it can see through the compiler
                    // forms one address register per read, keeps all of them live across the tile loop (60 with 64
                    // columns) and reloads them from scratch memory between the MFMAs; this way each address is one
                    // addition next to its read
                    int off = lane_idx * (int)sizeof(T);       // in bytes: no shift left between the asm and the read
                    // (the 16-column fp32 form has room for its 16 addresses: left alone it is 1 % faster, C4 123.4 ->
                    // 122.2 ms per dfmmv)
                    if constexpr (!(sizeof(T) == 4 && TT == 16)) asm volatile("" : "+v"(off));
                    const T *lane_row = (const T *)((const char *)ldsRow + off);
                    const bool more = s2 + 1 < TR::ACCN || p + 1 < WA_FR;
                    const int step = s2 + 1 < TR::ACCN ? p * TR::BLK + TR::acc_row(s2 + 1, 0) - TR::acc_row(0, 0)
                                                       : (p + 1) * TR::BLK;
#pragma unroll
                    for (int g = 0; g < NC; g++)
                        if (more) bnext[g] = lane_row[step * kVecStride + g * kGroupCols - (kTail16 && g == 1 ? tail_adj : 0)];
#pragma unroll
                    for (int g = 0; g < NC; g++)
#pragma unroll
                        for (int q = 0; q < WB_FR; q++) {
                            if constexpr (kHalf16 || kTail16) {
                                if (kHalf16 || g == 1)
                                    out2[q][g] = __builtin_amdgcn_mfma_f32_16x16x1f32(acc[p][q][s2], bval[g], out2[q][g], 0, 0, 0);
                                else out2[q][g] = TR::mfma(acc[p][q][s2], bval[g], out2[q][g]);
                            } else {
                                out2[q][g] = TR::mfma(acc[p][q][s2], bval[g], out2[q][g]);
                            }
                        }
#pragma unroll
                    for (int g = 0; g < NC; g++) {
                        asm volatile("" : "+v"(bval[g]) : "v"(&ldsRow[0]) : "memory");
                        bval[g] = bnext[g];
                    }
                }
            }
        }
    }

    if constexpr (kStore) {
        // nothing left to write
    } else if constexpr (kMfmaEpi) {
        if constexpr (kHalf16 || kTail16) {
            // the group on the 16x16x1 step: registers 4 b + r and 4 (b + 2) + r together are output row
            // 16 b + 4 (lane / 16) + r of column lane % 16 (behind the 32 columns of the first group, if there is one)
            constexpr int g16 = kTail16 ? 1 : 0;
            const int col = (kTail16 ? kGroupCols : 0) + (lane & 15), mq = lane >> 4;
            if (col < tcols) {
#pragma unroll
                for (int q = 0; q < WB_FR; q++) {
                    const int64_t bb = bblk0 + wb * WB_FR + q;
                    if (bb < nb_blocks) {
#pragma unroll
                        for (int b = 0; b < 2; b++)
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                partial[(((int64_t)by * kLWavesA + wa) * tcols + col) * nb_pad + bb * TR::BLK + 16 * b + 4 * mq + r] =
                                    out2[q][g16][4 * b + r] + out2[q][g16][4 * (b + 2) + r];
                    }
                }
            }
        }
        // lane = column t (both lane groups hold different output rows): no cross-lane step
        const int tl = j & (kGroupCols - 1);
#pragma unroll
        for (int g = 0; g < (kHalf16 ? 0 : kTail16 ? 1 : NC); g++) {
            const int col = tl + g * kGroupCols;
            if (j < kGroupCols && col < tcols) {
#pragma unroll
                for (int q = 0; q < WB_FR; q++) {
                    const int64_t bb = bblk0 + wb * WB_FR + q;
                    if (bb < nb_blocks) {
#pragma unroll
                        for (int r = 0; r < TR::ACCN; r++)
                            partial[(((int64_t)by * kLWavesA + wa) * tcols + col) * nb_pad + bb * TR::BLK +
                                    TR::acc_row(r, lg)] = out2[q][g][r];
                    }
                }
            }
        }
    } else {
        // join the lane groups that hold the same output row, then one partial per (split, wa)
#pragma unroll
        for (int q = 0; q < WB_FR; q++) {
            const int64_t bb = bblk0 + wb * WB_FR + q;
#pragma unroll
            for (int t = 0; t < TT; t++) {
                T s = out[q][t];
                if (TR::KG == 4) s += __shfl_xor(s, 16, 64);
                s += __shfl_xor(s, 32, 64);
                if (lg == 0 && bb < nb_blocks && t < tcols)
                    partial[(((int64_t)by * kLWavesA + wa) * tcols + t) * nb_pad + bb * TR::BLK + TR::out_row(j)] = s;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// dispatch
// ---------------------------------------------------------------------------
template <typename T> struct LCfg;
// fp32: 4 waves (2 x 2), two workgroups per CU so that one workgroup's barrier and LDS latencies are covered
// by the other; tile 256 (A) x 128 (B) rows.
template <> struct LCfg<float>  { static constexpr int WVA = 2, WVB = 2, WA_FR = 4, WB_FR = 2, KC = 8; };
// fp64: 8 waves (2 x 4), one workgroup per CU; tile 256 (A) x 128 (B) rows in feature stages of four steps: every wave
// holds 8 x 2 accumulator blocks (128 registers), so that a byte staged through LDS feeds a third more MFMAs than on a
// 128 x 128 tile in stages of eight steps, which the kernel used before (measured, dfmmv at N = 5e5, M = 1e4, d = 784, 10
// columns: 245.5 -> 239.4 ms; one column 241.8 -> 238.3, 16 columns 247.0 -> 242.6; N = 5e5, M = 2e4, d = 100: 76.1 -> 73.2,
// 10 columns 88.0 -> 83.4; N = 2.5e5, M = 2e4, d = 300: 97.5 -> 95.4).  (On the 128 x 128 tile, stages of four steps
// instead of eight were 3 to 7 % faster below 128 features and 2 to 3 % slower from 256 on.)
template <> struct LCfg<double> { static constexpr int WVA = 2, WVB = 4, WA_FR = 8, WB_FR = 2, KC = 4; };

// fp32 with 17 .. 32 columns: the row values of an A tile take 34 KB of LDS, two workgroups with the 48 KB of feature
// stages each no longer fit a CU; 8 waves (2 x 4) on a 256 x 256 tile, one workgroup per CU.
struct LCfgWide32 { static constexpr int WVA = 2, WVB = 4, WA_FR = 4, WB_FR = 2, KC = 8; };
// fp64 with 17 .. 32 columns (two groups of 16): the row values take 35 KB; feature stages of four steps instead of eight
// (64 KB instead of 128) make room for them.
struct LCfgWide64 { static constexpr int WVA = 2, WVB = 4, WA_FR = 4, WB_FR = 2, KC = 4; };

constexpr int kLargeMaxCols = 16;
#if FLK_KF == FLK_GAUSSIAN   // the tile geometry is the same for every kernel function: defined once
// Reduction blocks per tile: every pass of a call walks the same tiles, so the count follows the call's columns in all
// (fp64 beyond 16 columns: the 128-row tile of the many-column configuration, also for a last pass of few columns).
template <typename T> int mmv_large_a_tile_blocks(int64_t t) {
    if (sizeof(T) == 8 && t > kLargeMaxCols) return LCfgWide64::WVA * LCfgWide64::WA_FR;
    return LCfg<T>::WVA * LCfg<T>::WA_FR;
}
template <typename T> int mmv_large_b_tile_blocks(int64_t t) {
    if (sizeof(T) == 4 && t > kLargeMaxCols) return LCfgWide32::WVB * LCfgWide32::WB_FR;
    return LCfg<T>::WVB * LCfg<T>::WB_FR;
}
template <typename T> int mmv_large_partials_per_split() { return LCfg<T>::WVA; }
template <typename T> int mmv_large_max_cols(int64_t t) {
    return t > 2 * kLargeMaxCols ? 4 * kLargeMaxCols : t > kLargeMaxCols ? 2 * kLargeMaxCols : kLargeMaxCols;
}
template int mmv_large_max_cols<float>(int64_t);
template int mmv_large_max_cols<double>(int64_t);
template int mmv_large_a_tile_blocks<float>(int64_t);
template int mmv_large_a_tile_blocks<double>(int64_t);
template int mmv_large_b_tile_blocks<float>(int64_t);
template int mmv_large_b_tile_blocks<double>(int64_t);
template int mmv_large_partials_per_split<float>();
template int mmv_large_partials_per_split<double>();
#endif

template <typename T, int TT, typename C = LCfg<T>>
static int launch_large_tt(const PackedView &A, const PackedView &B, const T *vecp, int64_t vec_ld, int tcols,
                           int a_tile_blocks, int64_t a_tiles_per_chunk, int splits, T *partial, hipStream_t st) {
    if (a_tile_blocks != C::WVA * C::WA_FR)
        return fail(FLK_EINVAL, "mmv_large: the launch plan counts tiles of %d blocks, the kernel's hold %d", a_tile_blocks,
                    C::WVA * C::WA_FR);
    const int64_t nbb = C::WVB * C::WB_FR;
    dim3 grid((unsigned)((B.nblk + nbb - 1) / nbb), (unsigned)splits);
    // feature chunks that hold features of the data, and the MFMA steps of the last of them that do
    const int64_t chunk_features = (int64_t)C::KC * LTraits<T>::KG;
    const int64_t n_chunks = (A.d + chunk_features - 1) / chunk_features;
    const int64_t tail = A.d - (n_chunks - 1) * chunk_features;
    const int last_steps = (int)((tail + LTraits<T>::KG - 1) / LTraits<T>::KG);
    if (n_chunks < 1 || n_chunks * chunk_features > A.dpad || last_steps < 1 || last_steps > C::KC)
        return fail(FLK_EINVAL, "mmv_large: operand padding does not match d");
    hipLaunchKernelGGL((mmv_large_kernel<T, C::WVA, C::WVB, C::WA_FR, C::WB_FR, C::KC, TT, FLK_KF>), grid,
                       dim3(64 * C::WVA * C::WVB), 0, st,
                       (const T *)A.data, (const T *)A.hnorm, vecp, vec_ld, tcols, (const T *)B.data,
                       (const T *)B.hnorm, A.nblk, B.nblk, A.dpad, (int)n_chunks, last_steps, a_tiles_per_chunk, partial, B.npad,
                       B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_large_kernel");
    return FLK_OK;
}

// The kernel matrix out[a][b] = K(A_a, B_b) through the same tiles (operands packed for d > 64): one workgroup per
// (A tile, B tile), or a few A tiles per workgroup where the grid would not hold them all.
template <typename T, typename O>
int FLK_CAT(launch_fmm_large_kf, FLK_KF)(const PackedView &A, const PackedView &B, O *out, int64_t ld, hipStream_t st) {
    typedef LCfg<T> C;
    if (A.dpad != B.dpad || A.d != B.d) return fail(FLK_EINVAL, "fmm: operands packed with different feature counts");
    if (A.n == 0 || B.n == 0) return FLK_OK;
    const int64_t nab = C::WVA * C::WA_FR, nbb = C::WVB * C::WB_FR;
    const int64_t a_tiles = (A.nblk + nab - 1) / nab;
    const int64_t per_wg = (a_tiles + 65534) / 65535;
    dim3 grid((unsigned)((B.nblk + nbb - 1) / nbb), (unsigned)((a_tiles + per_wg - 1) / per_wg));
    const int64_t chunk_features = (int64_t)C::KC * LTraits<T>::KG;
    const int64_t n_chunks = (A.d + chunk_features - 1) / chunk_features;
    const int64_t tail = A.d - (n_chunks - 1) * chunk_features;
    const int last_steps = (int)((tail + LTraits<T>::KG - 1) / LTraits<T>::KG);
    if (A.dpad % chunk_features != 0 || n_chunks * chunk_features > A.dpad || last_steps < 1 || last_steps > C::KC)
        return fail(FLK_EINVAL, "fmm: operand padding does not match the LDS-tiled kernel");
    hipLaunchKernelGGL((mmv_large_kernel<T, C::WVA, C::WVB, C::WA_FR, C::WB_FR, C::KC, 1, FLK_KF, O>), grid,
                       dim3(64 * C::WVA * C::WVB), 0, st, (const T *)A.data, (const T *)A.hnorm, (const T *)nullptr,
                       (int64_t)0, 0, (const T *)B.data, (const T *)B.hnorm, A.nblk, B.nblk, A.dpad,
                       (int)n_chunks, last_steps, per_wg,
                       (T *)nullptr, B.npad, B.n > A.n, (void *)out, ld, A.n, B.n);
    FLK_LAUNCH_CHECK("mmv_large_kernel (kernel matrix)");
    return FLK_OK;
}
template int FLK_CAT(launch_fmm_large_kf, FLK_KF)<float, float>(const PackedView &, const PackedView &, float *, int64_t,
                                                                hipStream_t);
template int FLK_CAT(launch_fmm_large_kf, FLK_KF)<double, double>(const PackedView &, const PackedView &, double *,
                                                                  int64_t, hipStream_t);
template int FLK_CAT(launch_fmm_large_kf, FLK_KF)<double, float>(const PackedView &, const PackedView &, float *, int64_t,
                                                                 hipStream_t);

template <typename T>
int FLK_CAT(launch_mmv_large_kf, FLK_KF)(const PackedView &A, const PackedView &B, const T *vecp, int64_t vec_ld,
                                         int tcols, int a_tile_blocks, int64_t a_tiles_per_chunk, int splits,
                                         T *partial, hipStream_t st) {
    if (A.dpad != B.dpad) return fail(FLK_EINVAL, "mmv_large: operands packed with different feature counts");
    const int most = 4 * kLargeMaxCols;
    if (tcols < 1 || tcols > most) return fail(FLK_EINVAL, "mmv_large: column chunk %d not in 1..%d", tcols, most);
    if (tcols > kLargeMaxCols) {
        if constexpr (sizeof(T) == 4) {
            if (tcols > 3 * kLargeMaxCols)
                return launch_large_tt<T, 64, LCfgWide32>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
            if (tcols > 2 * kLargeMaxCols)       // 33 to 48 columns: a group of 32 and a group of 16
                return launch_large_tt<T, 48, LCfgWide32>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
            return launch_large_tt<T, 32, LCfgWide32>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
        } else {
            if (tcols > 3 * kLargeMaxCols)
                return launch_large_tt<T, 64, LCfgWide64>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
            if (tcols > 2 * kLargeMaxCols)       // 33 to 48 columns: three groups of 16
                return launch_large_tt<T, 48, LCfgWide64>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
            return launch_large_tt<T, 32, LCfgWide64>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
        }
    }
    if constexpr (sizeof(T) == 8)       // a last pass of few columns behind passes of many: on their tiles
        if (a_tile_blocks == LCfgWide64::WVA * LCfgWide64::WA_FR && a_tile_blocks != LCfg<T>::WVA * LCfg<T>::WA_FR)
            return launch_large_tt<T, 32, LCfgWide64>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
    if (tcols == 1) return launch_large_tt<T, 1>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
    if (tcols == 2) return launch_large_tt<T, 2>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
    if (tcols <= 4) return launch_large_tt<T, 4>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
    if constexpr (kLargeFmaCols<T> == 8)
        if (tcols <= 8) return launch_large_tt<T, 8>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);
    return launch_large_tt<T, 16>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st);   // MFMA epilogue
}
template int FLK_CAT(launch_mmv_large_kf, FLK_KF)<float>(const PackedView &, const PackedView &, const float *, int64_t,
                                                         int, int, int64_t, int, float *, hipStream_t);
template int FLK_CAT(launch_mmv_large_kf, FLK_KF)<double>(const PackedView &, const PackedView &, const double *,
                                                          int64_t, int, int, int64_t, int, double *, hipStream_t);

}  // namespace flk
