// Register-resident fp32 product kernel: instantiations for even feature counts, and the entry point
// that picks between them and the folded variant.  Compiled once per kernel function (-DFLK_KF=0..4).
#ifndef FLK_KF
#define FLK_KF 0
#endif
#define FLK_FOLD false
#define FLK_PASTE2(a, b) a##b
#define FLK_PASTE(a, b) FLK_PASTE2(a, b)
#define FLK_LAUNCH_NAME FLK_PASTE(launch_mmv_small_f32_plain_kf, FLK_KF)
#include "mmv_small_f32_dispatch.inc"

namespace flk {

int FLK_CAT(launch_mmv_small_f32_fold_kf, FLK_KF)(const PackedView &A, const PackedView &B, const float *vecp,
                                                  int64_t vec_ld, int tt, int64_t a_chunk_blocks, int splits,
                                                  float *partial, hipStream_t st);

// Columns per pass of the per-lane FMA kernels (must match the instantiations in launch_tt); calls with more
// right-hand sides than that go to the kernel whose contraction runs on the matrix cores (mmv_small_f32_wide.hip:
// 16, 32 or 64 columns per pass; four resident blocks per wave up to 16 padded features, two beyond).  Measured
// against its 16-column form, dfmmv at N = 5e5, M = 2e4, 9 to 12 columns: d = 9 9.3 ms on the FMA kernel against 8.9,
// d = 16 11.3 against 11.0, d = 24 14.1 against 13.4 (and 13 to 16 columns at d = 9: 10.9 against 9.0); eight columns:
// d = 9 7.8 against 8.9, d = 28 13.3 against 14.7.
static inline int fma_cols(int64_t dpad) { return dpad / 2 <= 16 ? 8 : 4; }
constexpr int kWideColumns = 32;       // one group of columns of the wide kernel
constexpr int kWideMaxDpFr4 = 8;
// The wide kernel takes two groups (64 columns) on one evaluation of K unless the few columns beyond 32 are cheaper as a
// pass of the FMA kernel behind a 32-column pass.  Measured, dfmmv at N = 1e6, M = 2e4: 64-column kernel (any 33 to
// 64 columns) d = 9 / 16 / 28 / 40 / 64: 47.2 / 51.5 / 59.1 / 67.3 / 84.3 ms; 32-column pass 27.1 / 31.3 / 39.4 / 46.3 /
// 60.8; one-column pass 8.7 / 12.3 / 19.2 / 29.9 / 46.8, 16 columns at d = 9 21.7.
static inline int cheap_extra_cols(int64_t dpad) {
    const int64_t dp = dpad / 2;
    return dp <= 5 ? 12 : dp <= 8 ? 8 : dp <= 12 ? 3 : 0;
}
static inline bool two_groups(int64_t dpad, int64_t t) { return t > kWideColumns + cheap_extra_cols(dpad); }

#if FLK_KF == FLK_GAUSSIAN   // the geometry does not depend on the kernel function: defined once
template <> int64_t mmv_small_max_d<float>() { return 2 * kMaxDpFr2; }
template <> int mmv_small_b_blocks_per_wg<float>(int64_t dpad, int64_t t) {
    if (two_groups(dpad, t)) return kWavesPerWg * 2;
    if (t > fma_cols(dpad)) return kWavesPerWg * ((dpad / 2) <= kWideMaxDpFr4 ? 4 : 2);
    return kWavesPerWg * ((dpad / 2) <= kMaxDpFr4 ? 4 : 2);
}
template <> int mmv_small_max_cols<float>(int64_t dpad, int64_t t) {
    if (two_groups(dpad, t)) return 2 * kWideColumns;
    return t > fma_cols(dpad) ? kWideColumns : fma_cols(dpad);
}
template <> int mmv_small_width<float>(int64_t dpad, int tc) {
    if (tc > kWideColumns) return 2 * kWideColumns;
    if (tc > fma_cols(dpad)) return tc > kWideColumns / 2 ? kWideColumns : kWideColumns / 2;   // the wide kernel's 16-column form
    static const int widths[] = {1, 2, 3, 4, 6, 8};
    for (int w : widths) if (tc <= w) return w;
    return tc;
}
#endif

template <>
int FLK_CAT(launch_mmv_small_kf, FLK_KF)<float>(const PackedView &A, const PackedView &B, const float *vecp,
                                                int64_t vec_ld, int tt, int64_t a_chunk_blocks, int splits,
                                                float *partial, hipStream_t st) {
    if (A.dpad != B.dpad || A.d != B.d)
        return fail(FLK_EINVAL, "mmv_small: operands packed with different feature counts");
    if (tt > fma_cols(A.dpad))
        return FLK_CAT(launch_mmv_small_f32_wide_kf, FLK_KF)(A, B, vecp, vec_ld, tt, a_chunk_blocks, splits, partial, st);
    // odd d up to kFoldMaxD: the padding feature holds 1.0 (see pack_kernel) and carries hB through the MFMA chain
    if (f32_fold_applies(A.d))
        return FLK_CAT(launch_mmv_small_f32_fold_kf, FLK_KF)(A, B, vecp, vec_ld, tt, a_chunk_blocks, splits, partial, st);
    return FLK_LAUNCH_NAME(A, B, vecp, vec_ld, tt, a_chunk_blocks, splits, partial, st);
}

}  // namespace flk
