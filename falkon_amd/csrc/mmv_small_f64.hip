// Register-resident kernel-vector product for the radial kernels of kernel_fn.h, fp64, gfx950.
// Compiled once per kernel function (-DFLK_KF=0..4).
//
// Same structure as the fp32 kernel with the 16x16x4 fp64 MFMA: a wave keeps FR
// blocks of 16 output rows (B side) in registers and streams blocks of 16
// reduction rows (A side).  Lane l supplies features q*DP + s (q = l / 16) of
// block position l % 16.  Accumulator register r of lane l holds
//   column j = l % 16 (B position), row 4*r + q (A position);
// positions map to matrix rows through the packing order pos(row) =
// 4*(row%4) + row/4, so a lane's four accumulator rows are the consecutive
// matrix rows 4*q .. 4*q+3 of the A block.
#include "flk_common.h"
#include "kernel_fn.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

typedef double doublex4 __attribute__((ext_vector_type(4)));

// The Gaussian's half norms and exponents are carried times 2048 (kernel_fn.h, kGaussExpBits).  Where the output rows'
// half norms are factored out of the sums (RAW), the exponent x.c + hA is bounded by -hB of the output row and can be
// positive, which the exponential does not take: every wave shifts it down by the largest -hB of its resident rows,
// rounded up to the next whole bit, so that it is negative, and multiplies the shift back into the finished sums.  The
// rows' -hB may be up to kRawMaxBits bits: a term that matters for a row (within 2^-60 of its largest) is then no
// smaller than 2^-(kRawMaxBits + 60), far inside the normal range.  (A constant shift would be simpler, but the
// exponent would then always carry the rounding error of a number that size, 3e-14 of the kernel value at 450 bits.)
constexpr double kRawMaxBits = 449.0;

constexpr int kWavesPerWg64 = 4;
constexpr int kFlushEvery64 = 16;

template <int DP, int TT>
struct AFrag64 {
    double a[DP];
    doublex4 hn;
    doublex4 vec[TT];
};

template <int DP, int TT>
__device__ __forceinline__ void load_afrag64(AFrag64<DP, TT> &f, const double *__restrict__ PA,
                                             const double *__restrict__ hA, const double *__restrict__ vecp,
                                             int64_t vec_ld, int64_t ab, int j, int q) {
    // scalar block bases, 32-bit lane offsets (flk_common.h: scalar_base)
    const auto blk = scalar_base(PA + ab * (4 * DP * 16));
    const int off = q * (DP * 16) + j;
#pragma unroll
    for (int s = 0; s < DP; s++) f.a[s] = blk[off + s * 16];
    typedef const doublex4 __attribute__((address_space(1))) *rows4;
    f.hn = *(rows4)(scalar_base(hA + ab * 16) + 4 * q);
#pragma unroll
    for (int t = 0; t < TT; t++) f.vec[t] = *(rows4)(scalar_base(vecp + t * vec_ld + ab * 16) + 4 * q);
}

// RAW (Gaussian only): the output rows' half norms stay out of the exponent (they multiply the finished sums), so the
// accumulators start from the A block's half norms alone and the kernel value is the bare 2^e, not clamped at 1.
template <int DP, int FR, int TT, bool RAW>
__device__ __forceinline__ void tile_step64(const AFrag64<DP, TT> &f, const double (&breg)[FR][DP],
                                            const double (&hb)[FR], double (&o1)[FR][TT], const double *exp_tab,
                                            double raw_shift) {
    doublex4 acc[FR];
    // RAW: the exponent is shifted down by the wave's raw_shift (four subtractions per A block)
    doublex4 hn_raw;
#pragma unroll
    for (int r = 0; r < 4; r++) hn_raw[r] = f.hn[r] - raw_shift;
#pragma unroll
    for (int c = 0; c < FR; c++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[c][r] = RAW ? hn_raw[r] : f.hn[r] + hb[c];
#pragma unroll
    for (int s = 0; s < DP; s++)
#pragma unroll
        for (int c = 0; c < FR; c++) acc[c] = __builtin_amdgcn_mfma_f64_16x16x4f64(f.a[s], breg[c][s], acc[c], 0, 0, 0);
#pragma unroll
    for (int c = 0; c < FR; c++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            // (three and four columns leave room for one wave per SIMD only, and a lone wave cannot hide the table's
            // LDS latency: those variants evaluate the polynomial; measured d = 28, T = 4: 16.2 ms against 18.8)
            double k;
            if constexpr (TT <= 2)
                k = RAW ? exp2_table_scaled<(DP > 4)>(acc[c][r], exp_tab) : kernel_value<FLK_KF, (DP > 4)>(acc[c][r], exp_tab);
            else k = RAW ? Exp2Poly{}.scaled(acc[c][r]) : kernel_value<FLK_KF>(acc[c][r]);
#pragma unroll
            for (int t = 0; t < TT; t++) o1[c][t] = __builtin_fma(k, f.vec[t][r], o1[c][t]);
        }
}

// One wave's walk over the A blocks a0 .. a1 (double buffered in registers), accumulating into o1 / o2.
template <int DP, int FR, int TT, bool RAW>
__device__ __forceinline__ void reduce_blocks64(const double *__restrict__ PA, const double *__restrict__ hA,
                                                const double *__restrict__ vecp, int64_t vec_ld, int64_t a0, int64_t a1,
                                                int j, int q, const double (&breg)[FR][DP], const double (&hb)[FR],
                                                double (&o1)[FR][TT], double (&o2)[FR][TT], const double *exp_tab,
                                                double raw_shift) {
    AFrag64<DP, TT> f0, f1;
    // the chunk's bounds are the same for the whole wave; block indices count from its first block, in 32 bits, so
    // that the loop's comparisons and the blocks' base addresses are scalar instructions
    a0 = as_scalar(a0);
    a1 = as_scalar(a1);
    if (a0 >= a1) return;
    PA += a0 * (4 * DP * 16);
    hA += a0 * 16;
    vecp += a0 * 16;
    const int nblk = (int)(a1 - a0);
    load_afrag64<DP, TT>(f0, PA, hA, vecp, vec_ld, 0, j, q);
    int since_flush = 0;
    for (int ab = 0; ab < nblk; ab += 2) {
        const bool has1 = ab + 1 < nblk;
        if (has1) load_afrag64<DP, TT>(f1, PA, hA, vecp, vec_ld, ab + 1, j, q);
        tile_step64<DP, FR, TT, RAW>(f0, breg, hb, o1, exp_tab, raw_shift);
        if (has1) {
            if (ab + 2 < nblk) load_afrag64<DP, TT>(f0, PA, hA, vecp, vec_ld, ab + 2, j, q);
            tile_step64<DP, FR, TT, RAW>(f1, breg, hb, o1, exp_tab, raw_shift);
        }
        since_flush += 2;
        if (since_flush >= kFlushEvery64) {
            since_flush = 0;
#pragma unroll
            for (int c = 0; c < FR; c++)
#pragma unroll
                for (int t = 0; t < TT; t++) { o2[c][t] += o1[c][t]; o1[c][t] = 0.0; }
        }
    }
}

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <int DP, int FR, int TT, int KF>
__global__ void __launch_bounds__(256, 2)
    mmv_small_f64_kernel(const double *__restrict__ PA, const double *__restrict__ hA, const double *__restrict__ vecp,
                         int64_t vec_ld, const double *__restrict__ PB, const double *__restrict__ hB,
                         int64_t na_blocks, int64_t nb_blocks, int64_t a_chunk_blocks, double *__restrict__ partial,
                         int64_t nb_pad, bool y_fastest) {
    // gfx950 has no fp64 exponential: 2^(k/2048) from a table in LDS, filled here (kernel_fn.h)
    __shared__ double exp_tab[TT <= 2 ? kExpTableSize : 1];
    if constexpr (TT <= 2) {
        exp2_table_fill(exp_tab, threadIdx.x, 256);
        __syncthreads();
    }
    unsigned bx, by;
    xcd_remap(bx, by, y_fastest);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j = lane & 15, q = lane >> 4;
    const int jrow = 4 * (j & 3) + (j >> 2);  // matrix row (within its block) held at position j
    const int64_t bb0 = ((int64_t)bx * kWavesPerWg64 + wave) * FR;
    if (bb0 >= nb_blocks) return;
    const int64_t a0 = (int64_t)by * a_chunk_blocks;
    int64_t a1 = a0 + a_chunk_blocks;
    if (a1 > na_blocks) a1 = na_blocks;

    double breg[FR][DP];
    double hb[FR];
#pragma unroll
    for (int c = 0; c < FR; c++) {
        int64_t bb = bb0 + c < nb_blocks ? bb0 + c : nb_blocks - 1;
        const double *p = PB + (bb * (4 * DP) + (int64_t)q * DP) * 16 + j;
#pragma unroll
        for (int s = 0; s < DP; s++) breg[c][s] = p[s * 16];
        hb[c] = hB[bb * 16 + jrow];
    }

    double o1[FR][TT], o2[FR][TT];
#pragma unroll
    for (int c = 0; c < FR; c++)
#pragma unroll
        for (int t = 0; t < TT; t++) { o1[c][t] = 0.0; o2[c][t] = 0.0; }

    // Gaussian: 2^hB_j is taken out of the sums, out_j = 2^hB_j sum_i 2^(x_i.c_j + hA_i) vec_i, which saves an add and
    // the clamp per kernel value, as long as 2^(-hB_j) is nowhere near the fp64 range (kRawMaxBits); every wave checks its own
    // resident rows (rows with a non-finite half norm fail the check).  On that path a kernel value is not clamped
    // entry by entry: where two points coincide K is 1 to rounding instead of exactly 1.
    constexpr bool kCanFactorOut = KF == FLK_GAUSSIAN;
    bool factored = false;
    double raw_shift = 0.0;
    if constexpr (kCanFactorOut) {
        bool small_norms = true;
        double most = 0.0;             // largest -hB among the wave's resident rows, in units of 1/2048 bit
#pragma unroll
        for (int c = 0; c < FR; c++) {
            small_norms = small_norms && hb[c] >= -kRawMaxBits * kGaussExpScale;
            most = fmax(most, -hb[c]);
        }
        factored = __all(small_norms);
        for (int off = 32; off > 0; off >>= 1) most = fmax(most, __shfl_xor(most, off, 64));
        // a whole number of bits above it: both factors 2^(-shift/2048) and 2^(shift/2048) are then exact powers of two
        raw_shift = (floor(most * (1.0 / kGaussExpScale)) + 1.0) * kGaussExpScale;
    }
    if (kCanFactorOut && factored)
        reduce_blocks64<DP, FR, TT, true>(PA, hA, vecp, vec_ld, a0, a1, j, q, breg, hb, o1, o2, exp_tab, raw_shift);
    else
        reduce_blocks64<DP, FR, TT, false>(PA, hA, vecp, vec_ld, a0, a1, j, q, breg, hb, o1, o2, exp_tab, 0.0);
#pragma unroll
    for (int c = 0; c < FR; c++) {
        const double out_scale = (kCanFactorOut && factored) ? exp2_nonpositive((hb[c] + raw_shift) * (1.0 / kGaussExpScale)) : 1.0;
#pragma unroll
        for (int t = 0; t < TT; t++) {
            double s = o2[c][t] + o1[c][t];
            s += __shfl_xor(s, 16, 64);
            s += __shfl_xor(s, 32, 64);
            if (kCanFactorOut) s *= out_scale;
            if (q == 0 && bb0 + c < nb_blocks)
                partial[((int64_t)by * TT + t) * nb_pad + (bb0 + c) * 16 + jrow] = s;
        }
    }
}

// right-hand sides per pass of the FMA kernel above: four, except from 52 padded features on, where its
// four-column variant is out of registers and runs one wave per SIMD (dfmmv at N = 5e5, M = 2e4, four columns against
// the 16-column kernel: d = 52 56.3 ms against 49.9, d = 56 54.1 against 52.2, d = 64 56.6 against 49.0 for three)
inline int fma_cols64(int64_t dpad) { return dpad >= 52 ? 3 : 4; }
constexpr int kWideCols64 = 16;  // of the kernel that contracts on the matrix cores
constexpr int kMaxDp64Fr4 = 8;   // dpad <= 32
constexpr int kMaxDp64Fr2 = 16;  // dpad <= 64

// resident blocks per wave of the FMA kernel with tt columns (fr: the single-column kernel's count)
constexpr int fr64_for(int dp, int fr, int tt) {
    if (fr != 4) return fr;
    // Matern 3/2 and 5/2 with one column at 25 .. 28 features: the four-block variant does not fit 256 registers
    // (two blocks, dfmmv at N = 5e5, M = 2e4, d = 28: 44.5 -> 40.0 ms)
    if ((FLK_KF == FLK_MATERN32 || FLK_KF == FLK_MATERN52) && tt == 1 && dp == 7) return 2;
    return ((tt == 2 && dp >= 2) || (tt == 3 && dp >= 6) || (tt >= 4 && dp >= 5)) ? 2 : fr;
}

#if FLK_KF == FLK_GAUSSIAN   // the geometry does not depend on the kernel function: defined once
template <> int64_t mmv_small_max_d<double>() { return 4 * kMaxDp64Fr2; }
template <> bool mmv_small_serves<double>(int64_t d, int64_t) { return d <= 4 * kMaxDp64Fr2; }
// more than four right-hand sides: the 16-column kernel of mmv_small_f64_wide.hip, which reads 16 planes
// (beyond 16 columns two groups of 16 share one evaluation of K: 17 columns that way take less time than a
// 16-column pass and a one-column pass, at every feature count)
// (beyond 32 columns three or four groups share one evaluation of K, with half the resident blocks.  A 32-column pass
// followed by a pass of the FMA kernel for one to four more columns is never the faster pair: dfmmv at N = 5e5, M = 2e4,
// d = 9, T = 33: 49.5 ms against 43.6 for the three-group form, d = 28: 69.2 against 54.1)
static inline bool four_groups64(int64_t dpad, int64_t t) { (void)dpad; return t > 2 * kWideCols64; }
template <> int mmv_small_max_cols<double>(int64_t dpad, int64_t t) {
    if (four_groups64(dpad, t)) return 4 * kWideCols64;
    if (t > kWideCols64) return 2 * kWideCols64;
    return t > fma_cols64(dpad) ? kWideCols64 : fma_cols64(dpad);
}
template <> int mmv_small_width<double>(int64_t dpad, int tc) {
    if (tc > 3 * kWideCols64) return 4 * kWideCols64;
    if (tc > 2 * kWideCols64) return 3 * kWideCols64;     // 33 to 48 columns: three groups
    if (tc > kWideCols64) return 2 * kWideCols64;
    return tc > fma_cols64(dpad) ? kWideCols64 : tc;
}
template <> int mmv_small_wgs_per_cu<double>(int64_t, int64_t) { return 2; }
template <> int mmv_small_b_blocks_per_wg<double>(int64_t dpad, int64_t t) {
    const int fr = (dpad / 4) <= kMaxDp64Fr4 ? 4 : 2;
    if (t >= 2 && t <= fma_cols64(dpad)) return kWavesPerWg64 * fr64_for((int)(dpad / 4), fr, (int)t);
    return kWavesPerWg64 * (four_groups64(dpad, t) ? fr / 2 : fr);   // four column groups: half the resident blocks
}
#endif

template <int DP, int FR, int TT>
static int launch_one64(const PackedView &A, const PackedView &B, const double *vecp, int64_t vec_ld,
                        int64_t a_chunk_blocks, int splits, double *partial, hipStream_t st) {
    const int64_t per_wg = kWavesPerWg64 * FR;
    dim3 grid((unsigned)((B.nblk + per_wg - 1) / per_wg), (unsigned)splits);
    hipLaunchKernelGGL((mmv_small_f64_kernel<DP, FR, TT, FLK_KF>), grid, dim3(256), 0, st, (const double *)A.data,
                       (const double *)A.hnorm, vecp, vec_ld, (const double *)B.data, (const double *)B.hnorm, A.nblk,
                       B.nblk, a_chunk_blocks, partial, B.npad, B.n > A.n);
    FLK_LAUNCH_CHECK("mmv_small_f64_kernel");
    return FLK_OK;
}

template <int DP, int FR>
static int launch_tt64(int tt, const PackedView &A, const PackedView &B, const double *vecp, int64_t vec_ld,
                       int64_t a_chunk_blocks, int splits, double *partial, hipStream_t st) {
    // With more than one column the four-block variants need more than 256 registers and run one wave per SIMD, which
    // leaves the latency of the exponential's table reads and of the MFMA results exposed: two resident blocks (two or
    // three waves per SIMD) are faster from 8 features on with two columns, from 24 on with three and from 20 on with four.  Measured,
    // dfmmv at N = 5e5, M = 2e4, four blocks -> two: T = 2: d = 16 20.5 -> 18.1 ms, d = 28 29.6 -> 24.8, d = 32 35.6 ->
    // 29.4 (d = 4: 11.4 -> 11.6, kept at four); T = 4: d = 28 30.4 -> 28.9 (d = 16: 21.3 -> 22.5, kept at four).
    constexpr int kFr1 = fr64_for(DP, FR, 1), kFr2 = fr64_for(DP, FR, 2), kFr3 = fr64_for(DP, FR, 3), kFr4 = fr64_for(DP, FR, 4);
    switch (tt) {
        case 1: return launch_one64<DP, kFr1, 1>(A, B, vecp, vec_ld, a_chunk_blocks, splits, partial, st);
        case 2: return launch_one64<DP, kFr2, 2>(A, B, vecp, vec_ld, a_chunk_blocks, splits, partial, st);
        case 3: return launch_one64<DP, kFr3, 3>(A, B, vecp, vec_ld, a_chunk_blocks, splits, partial, st);
        case 4: return launch_one64<DP, kFr4, 4>(A, B, vecp, vec_ld, a_chunk_blocks, splits, partial, st);
    }
    return fail(FLK_EINVAL, "mmv_small: column chunk %d not in 1..4", tt);
}

template <>
int FLK_CAT(launch_mmv_small_kf, FLK_KF)<double>(const PackedView &A, const PackedView &B, const double *vecp,
                                                 int64_t vec_ld, int tt, int64_t a_chunk_blocks, int splits,
                                                 double *partial, hipStream_t st) {
    if (A.dpad != B.dpad) return fail(FLK_EINVAL, "mmv_small: operands packed with different feature counts");
    if (tt > fma_cols64(A.dpad))
        return FLK_CAT(launch_mmv_small_f64_wide_kf, FLK_KF)(A, B, vecp, vec_ld, tt, a_chunk_blocks, splits, partial, st);
    const int dp = (int)(A.dpad / 4);
#define FLK_CASE4(DPV) \
    case DPV: return launch_tt64<DPV, 4>(tt, A, B, vecp, vec_ld, a_chunk_blocks, splits, partial, st);
#define FLK_CASE2(DPV) \
    case DPV: return launch_tt64<DPV, 2>(tt, A, B, vecp, vec_ld, a_chunk_blocks, splits, partial, st);
    switch (dp) {
        FLK_CASE4(1) FLK_CASE4(2) FLK_CASE4(3) FLK_CASE4(4) FLK_CASE4(5) FLK_CASE4(6) FLK_CASE4(7) FLK_CASE4(8)
        FLK_CASE2(9) FLK_CASE2(10) FLK_CASE2(11) FLK_CASE2(12) FLK_CASE2(13) FLK_CASE2(14) FLK_CASE2(15) FLK_CASE2(16)
    }
#undef FLK_CASE4
#undef FLK_CASE2
    return fail(FLK_EUNSUPPORTED, "mmv_small<f64>: padded feature count %lld not in 4..64", (long long)A.dpad);
}

}  // namespace flk
