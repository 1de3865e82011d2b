// "bf16x3" mode of the fp32 products, gfx950: the cross term x~.c~ runs on the bf16 matrix cores.
//
// Every scaled fp32 value is written as the sum of three bfloat16 numbers, x~ = hi + mid + lo (each the
// round-to-nearest of what the previous ones leave: 3 x 8 = 24 significant bits, i.e. the fp32 value itself), and
// the product of two such sums is accumulated from the six partial products whose weight is at least 2^-16 of
// the leading one (hi.hi, hi.mid, mid.hi, hi.lo, lo.hi, mid.mid; the dropped ones are below 2^-24).  Products of
// bfloat16 numbers are exact in fp32 and v_mfma_f32_32x32x16_bf16 accumulates in fp32, so the exponent has the
// accuracy of an fp32 dot product, at 16 features per MFMA instead of 2.  bfloat16 has the exponent range of
// fp32: no input range is lost.
//
// Packed operand: [block of 32 rows][k-step of 16 features][piece hi/mid/lo][lane 0..63][8 bfloat16], lane l
// holding features 8*(l/32) .. +7 of row l%32: one global_load_dwordx4 per lane is one MFMA operand.  The last
// two features of the padded row hold 1.0 and the row's half norm h = -1/2 |x~|^2 (split like everything else).
// The kernel swaps that pair in the resident (B side) fragments, so that the MFMA chain adds 1*hB + hA*1 by
// itself and the accumulator leaves the chain as the complete exponent.
#pragma once
#include "flk_common.h"

namespace flk {

constexpr int64_t kSplitMaxD = 62;          // register-resident kernel: four k-steps, two of the 64 features taken by (1, h)
constexpr int kSplitMaxCols = 4;            // its right-hand sides per pass

inline int64_t split_ksteps(int64_t d) { return (d + 2 + 15) / 16; }

// The register-resident kernel for many right-hand sides (mmv_split_wide.hip): passes of 8 to 64 columns (the forms of
// mmv_wide_common.h), two resident blocks per wave.  Passes of 32 and 64 columns contract on the bf16 matrix cores up to
// three k-steps (with four the 64-column pass is out of registers that way: d = 56, N = 5e5, M = 2e4, 36.4 ms against
// 30.2 on the fp32 steps), which makes them cheaper than the 24- and, up to two k-steps, the 48-column pass on the fp32
// steps: d = 28, 24 / 32 columns 14.0 / 13.8 ms, 48 / 64 columns 20.8 / 19.6; d = 40 (three k-steps) 48 / 64: 23.1 / 23.7.
constexpr int64_t kSplitWideMaxD = kSplitMaxD;
constexpr int kSplitWideMaxCols = 64;
constexpr int kSplitWideBlocksPerWave = 2;
constexpr int split_wide_form_cols(int tcols, int ks) {
    return tcols <= 8 ? 8 : tcols <= 16 ? 16 : tcols <= 32 ? 32 : tcols <= 40 ? 40 : tcols <= 48 && ks >= 3 ? 48 : 64;
}

struct SplitView {
    const void *data;    // [nblk][ks][3][64] x 16 bytes
    const float *hnorm;  // [npad] half norms in fp32 (the kernels use the split copy inside data; this one tells
                         // the prologue and epilogue kernels which rows hold non-finite data)
    int64_t n, d, ks, nblk, npad;
};
inline size_t split_data_bytes(int64_t n, int64_t d) {
    const int64_t nblk = (n + 31) / 32;
    return align256((size_t)nblk * split_ksteps(d) * 3 * 64 * 16);
}
inline size_t split_packed_bytes(int64_t n, int64_t d) {
    return split_data_bytes(n, d) + align256((size_t)((n + 31) / 32 * 32) * sizeof(float));
}
inline SplitView split_view(const void *buf, int64_t n, int64_t d) {
    SplitView v;
    v.data = buf; v.n = n; v.d = d;
    v.hnorm = buf ? (const float *)((const char *)buf + split_data_bytes(n, d)) : nullptr;
    v.ks = split_ksteps(d);
    v.nblk = (n + 31) / 32;
    v.npad = v.nblk * 32;
    return v;
}
// B blocks (of 32 output rows) per workgroup of the product kernel serving t right-hand sides per pass
inline int split_b_blocks_per_wg(int64_t ks, int64_t t) { return 4 * (ks <= 2 && t <= 2 ? 4 : 2); }

int launch_pack_split(const float *X, int64_t n, int64_t d, int64_t rs, int64_t cs, const float *sigma, int64_t n_sigma,
                      double scale, void *packed, hipStream_t st);

// LDS-tiled kernel for larger feature counts: tile geometry and right-hand sides per pass
int split_large_a_tile_blocks();
int split_large_b_tile_blocks();
int split_large_partials_per_split();
int split_large_max_cols();

#define FLK_DECLARE_SPLIT_KF(KF)                                                                              \
    int launch_mmv_split_kf##KF(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld,    \
                                int tcols, int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st); \
    int launch_mmv_split_wide_kf##KF(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, \
                                     int tcols, int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st); \
    int launch_mmv_split_large_kf##KF(const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, \
                                      int tcols, int64_t a_tiles_per_chunk, int splits, float *partial,        \
                                      hipStream_t st);                                                         \
    int launch_fmm_split_large_kf##KF(const SplitView &A, const SplitView &B, float *out, int64_t ld, hipStream_t st);
FLK_DECLARE_SPLIT_KF(0)
FLK_DECLARE_SPLIT_KF(1)
FLK_DECLARE_SPLIT_KF(2)
FLK_DECLARE_SPLIT_KF(3)
FLK_DECLARE_SPLIT_KF(4)
#undef FLK_DECLARE_SPLIT_KF

inline int launch_mmv_split(int kf, const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld, int tcols,
                            int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
#define FLK_CALL(KF) launch_mmv_split_kf##KF(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st)
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}

inline int launch_mmv_split_wide(int kf, const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld,
                                 int tcols, int64_t a_chunk_blocks, int splits, float *partial, hipStream_t st) {
#define FLK_CALL(KF) launch_mmv_split_wide_kf##KF(A, B, vecp, vec_ld, tcols, a_chunk_blocks, splits, partial, st)
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}

inline int launch_mmv_split_large(int kf, const SplitView &A, const SplitView &B, const float *vecp, int64_t vec_ld,
                                  int tcols, int64_t a_tiles_per_chunk, int splits, float *partial, hipStream_t st) {
#define FLK_CALL(KF) launch_mmv_split_large_kf##KF(A, B, vecp, vec_ld, tcols, a_tiles_per_chunk, splits, partial, st)
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}

// explicit kernel matrix out[a][b] = K(A_a, B_b) (rows ld elements apart, columns contiguous) in the bf16x3 mode
inline int launch_fmm_split_large(int kf, const SplitView &A, const SplitView &B, float *out, int64_t ld,
                                  hipStream_t st) {
#define FLK_CALL(KF) launch_fmm_split_large_kf##KF(A, B, out, ld, st)
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}

}  // namespace flk
