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
// 8 to 64 columns per pass in steps of 8; wide_form_cols, wide_blocks_per_wave in mmv_small_f32_kernel.h).  Measured,
// dfmmv at N = 5e5, M = 2e4, FMA kernel against the 8-column form (which costs the same for 3 to 8 columns):
// d = 9: 4 columns 6.2 ms against 6.6, 5 columns 7.0 against 6.7, 8 columns 8.1 against 6.8; d = 16: 8.2 / 8.9 / 9.9 against
// 8.7 / 8.8 / 8.9; d = 28: 5 and 6 columns 12.4 against 12.8, 8 columns 13.4 against 12.8; d = 40 (two resident blocks):
// 4 columns 15.5 against 17.0, 5 to 8 columns on the 16-column form 18.4 against 16.9.
static inline int fma_cols(int64_t dpad) { return dpad / 2 > 8 && dpad / 2 <= 16 ? 6 : 4; }
constexpr int kWideMaxColumns = 64;    // per pass of the wide kernel

#if FLK_KF == FLK_GAUSSIAN   // the geometry does not depend on the kernel function: defined once
template <> int64_t mmv_small_max_d<float>() { return 2 * kMaxDpFr2; }
template <> bool mmv_small_serves<float>(int64_t d, int64_t t) { return d <= 2 * kMaxDpFr2 || (t >= 1 && t <= 4 && d <= 2 * kMaxDpOneColumn); }
template <> int mmv_small_b_blocks_per_wg<float>(int64_t dpad, int64_t t) {
    if (t > fma_cols(dpad))
        return kWavesPerWg * wide_blocks_per_wave((int)(dpad / 2), wide_form_cols((int)(t < kWideMaxColumns ? t : kWideMaxColumns)));
    if (t == 1 && dpad / 2 > kMaxDpFr4OneColumn) return kWavesPerWg * 3;
    return kWavesPerWg * (((dpad / 2) <= kMaxDpFr4 || t == 1) ? 4 : 2);     // (one column: four blocks at every width)
}
// The single-column kernel with four resident blocks needs more than 256 registers per lane from 48 padded features on
// and then runs one wave per SIMD; every other form runs two.
template <> int mmv_small_wgs_per_cu<float>(int64_t dpad, int64_t t) {
    return ((t == 1 && dpad / 2 >= kMinDpOneWave) || dpad / 2 > kMaxDpFr2) ? 1 : 2;
}
template <> int mmv_small_max_cols<float>(int64_t dpad, int64_t t) {
    return t > fma_cols(dpad) ? kWideMaxColumns : fma_cols(dpad);
}
template <> int mmv_small_width<float>(int64_t dpad, int tc) {
    if (tc > fma_cols(dpad)) return wide_form_cols(tc);
    static const int widths[] = {1, 2, 3, 4, 6};
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
