// Shared declarations of the falkon_amd native library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/falkon_amd.h"
#include "kernel_fn.h"

namespace flk {

// Packed-operand geometry.  f32: blocks of 32 rows, features split over the two
// lane halves of a wave (MFMA 32x32x2).  f64: blocks of 16 rows, features split
// over the four lane quarters (MFMA 16x16x4).
template <typename T> struct Geo;
template <> struct Geo<float>  { static constexpr int BLK = 32; static constexpr int KG = 2; };
template <> struct Geo<double> { static constexpr int BLK = 16; static constexpr int KG = 4; };

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// Feature counts up to kSmallMaxD run the register-resident kernels and are padded to the MFMA's
// K granularity only; larger ones run the LDS-tiled kernel, which consumes features in chunks of
// kLargeKChunk MFMA steps, and are zero padded to whole chunks so that the kernel has no feature tail.
constexpr int64_t kSmallMaxD = 64;
constexpr int64_t kLargeKChunk = 8;
template <typename T> inline int64_t padded_features(int64_t d) {
    return d <= kSmallMaxD ? round_up(d, Geo<T>::KG) : round_up(d, Geo<T>::KG * kLargeKChunk);
}
// Odd feature counts up to kFoldMaxD (fp32 only): the one padding feature of a packed row holds 1.0 and the
// product kernel's resident fragment puts its half norm into that slot ("fold"), so the MFMA chain adds the
// half norm itself.  Measured: a gain for the four-blocks-per-wave kernels (d <= 32), a loss for the
// two-blocks-per-wave ones (d = 35: 16.9 ms folded against 13.0 ms for d = 36 unfolded), which therefore
// treat odd d like d + 1.
constexpr int64_t kFoldMaxD = 32;
inline bool f32_fold_applies(int64_t d) { return (d & 1) && d <= kFoldMaxD; }
inline size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

struct PackedView {
    const void *data;   // [nblk][dpad][BLK]
    const void *hnorm;  // [npad]  -1/2 * |x~|^2, zero on padding rows
    int64_t n, d, dpad, nblk, npad;
};

template <typename T>
inline PackedView packed_view(const void *buf, int64_t n, int64_t d) {
    PackedView v;
    v.n = n; v.d = d;
    v.dpad = padded_features<T>(d);
    v.nblk = (n + Geo<T>::BLK - 1) / Geo<T>::BLK;
    v.npad = v.nblk * Geo<T>::BLK;
    v.data = buf;
    v.hnorm = (const char *)buf + align256((size_t)v.nblk * v.dpad * Geo<T>::BLK * sizeof(T));
    return v;
}
template <typename T>
inline size_t packed_bytes(int64_t n, int64_t d) {
    int64_t dpad = padded_features<T>(d);
    int64_t nblk = (n + Geo<T>::BLK - 1) / Geo<T>::BLK;
    return align256((size_t)nblk * dpad * Geo<T>::BLK * sizeof(T)) + align256((size_t)nblk * Geo<T>::BLK * sizeof(T));
}

// Workgroups are handed to the 8 XCDs round-robin by linear workgroup id, and each XCD has its own L2.
// This remaps the id so that every XCD works on one contiguous range of logical ids: workgroups that
// share a chunk of the reduction side (same logical y, neighbouring x) then share an L2 instead of
// making all eight XCDs fetch that chunk from HBM.
#if defined(__HIPCC__)
// y_fastest picks which neighbours share an XCD: false -> same reduction chunk, neighbouring output tiles
// (right when the reduction side is the big operand), true -> same output tile, all reduction chunks
// (right when the output side is the big operand, whose tile is then fetched once instead of once per chunk).
__device__ __forceinline__ void xcd_remap(unsigned &bx, unsigned &by, bool y_fastest) {
    const unsigned gx = gridDim.x, gy = gridDim.y, total = gx * gy;
    const unsigned id = blockIdx.y * gx + blockIdx.x;
    const unsigned q = total / 8, r = total % 8, xcd = id % 8, local = id / 8;
    const unsigned logical = xcd * q + (xcd < r ? xcd : r) + local;
    if (y_fastest) {
        by = logical % gy;
        bx = logical / gy;
    } else {
        bx = logical % gx;
        by = logical / gx;
    }
}
// The same XCD-contiguous numbering for kernels whose workgroups each own one (x, y) tile and share nothing through
// a loop (the kernel-matrix store mode): consecutive workgroups of an XCD walk bands of kBandY tiles in y, y fastest,
// so the 32 workgroups resident on an XCD cover 8 x 4 tiles and fetch 12 operand tiles through its L2 instead of 33.
constexpr unsigned kBandY = 8;
__device__ __forceinline__ void xcd_remap_banded(unsigned &bx, unsigned &by) {
    const unsigned gx = gridDim.x, gy = gridDim.y, total = gx * gy;
    const unsigned id = blockIdx.y * gx + blockIdx.x;
    const unsigned q = total / 8, r = total % 8, xcd = id % 8, local = id / 8;
    const unsigned logical = xcd * q + (xcd < r ? xcd : r) + local;
    const unsigned band = logical / (kBandY * gx), first = band * kBandY;
    const unsigned height = gy - first < kBandY ? gy - first : kBandY;
    const unsigned within = logical - band * kBandY * gx;
    by = first + within % height;
    bx = within / height;
}
#endif

#if defined(__HIPCC__)
// A wave-uniform 64-bit value as a pair of scalars, and a wave-uniform global address as a scalar base: loads through
// it take the form "scalar base + 32-bit lane offset", and the arithmetic that leads to the base is scalar too.  (Per-lane
// 64-bit address arithmetic runs on the vector ALU, where it does not overlap with the MFMAs.)  The pointer keeps its
// global address space through the round trip; a generic pointer would turn the loads into flat loads.
__device__ __forceinline__ int64_t as_scalar(int64_t v) {
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
template <typename T>
__device__ __forceinline__ const T __attribute__((address_space(1))) *scalar_base(const T *p) {
    return (const T __attribute__((address_space(1))) *)as_scalar((int64_t)p);
}
#endif

// error plumbing -------------------------------------------------------------
int fail(int code, const char *fmt, ...);
#define FLK_HIP(expr)                                                                      \
    do {                                                                                   \
        hipError_t e__ = (expr);                                                           \
        if (e__ != hipSuccess)                                                             \
            return ::flk::fail(FLK_EHIP, "%s failed: %s", #expr, hipGetErrorString(e__));  \
    } while (0)
#define FLK_LAUNCH_CHECK(name)                                                              \
    do {                                                                                   \
        hipError_t e__ = hipGetLastError();                                                \
        if (e__ != hipSuccess)                                                             \
            return ::flk::fail(FLK_EHIP, "launch of %s failed: %s", name, hipGetErrorString(e__)); \
    } while (0)

// Blocked triangular solve with a resident factor and the inverses of its diagonal blocks (trsv.hip)
// Cholesky factor of one diagonal tile and the inverse of that factor (potrf.hip)
int potrf_tile_rows(int dtype);
template <typename T>
int launch_potrf_tile(T *A, int64_t n, int64_t lda, T *inv, int64_t ldinv, int *info, int info_base, hipStream_t st);
int64_t tri_solve_work_elems(int64_t m, int64_t t, int64_t block);
template <typename T>
int launch_tri_solve(const T *L, int64_t m, int64_t ld, int row_major, const T *dinv, const T *dinv_t, int64_t block,
                     int transposed, const T *b, int64_t ldb, T *x, int64_t ldx, int64_t t, T *work, hipStream_t st);

// launchers implemented in the .hip files -------------------------------------
template <typename TI, typename T>   // TI: caller's element type, T: type of the packed operand
int launch_pack(const TI *X, int64_t n, int64_t d, int64_t rs, int64_t cs, const TI *sigma, int64_t n_sigma,
                double scale, T *pdata, T *hnorm, int64_t dpad, int64_t nblk, bool one_pad, hipStream_t st);

// One launch for the prologue of a one-shot product: packs the output-side operand (1) and the reduction-side operand
// (2) and writes the planar copy vp[tcols + zero_planes][nblk2 * BLK] of the right-hand side v that multiplies the rows
// of operand 2 (NaN in the rows whose half norm is not finite, as launch_vec_planar does); tcols = 0: no vector.
template <typename T>
int launch_pack_pair(const T *X1, int64_t n1, int64_t rs1, int64_t cs1, T *pdata1, T *hnorm1, int64_t nblk1, const T *X2,
                     int64_t n2, int64_t rs2, int64_t cs2, T *pdata2, T *hnorm2, int64_t nblk2, int64_t d, const T *sigma,
                     int64_t n_sigma, double scale, int64_t dpad, bool one_pad, const T *v, int64_t v_rs, int64_t v_cs,
                     T *vp, int64_t tcols, int64_t zero_planes, hipStream_t st);

// Non-finite data: a row holding a NaN or an infinity has a non-finite half norm.  The product kernels clamp the
// kernel value (K <= 1, D^2 >= 1e-20), which turns such a row's NaN exponents into numbers; so that the result still
// says NaN where the reference's does, the planar copy of a right-hand side takes NaN in the rows whose reduction-side
// half norm (row_half_norm, may be null) is not finite, and the finalize kernel writes NaN into the output rows whose
// half norm is not finite.
template <typename T>
int launch_vec_planar(const T *v, int64_t n, int64_t t, int64_t rs, int64_t cs, T *vp, int64_t npad,
                      int64_t zero_planes, const T *row_half_norm,
                      hipStream_t st);   // also clears zero_planes planes after the t-th
template <typename T> int launch_zero_fill(T *p, int64_t count, hipStream_t st);

template <typename T>
int launch_finalize(const T *partial, int splits, int64_t t, int64_t nb, int64_t nb_pad, const T *addend,
                    int64_t add_rs, int64_t add_cs, T *out, int64_t out_rs, int64_t out_cs, bool zero_pad,
                    const T *row_half_norm, hipStream_t st);

// One conjugate-gradient iteration's vector updates for t right-hand sides (cg.hip).
template <typename T>
int launch_cg_update(int mode, T *X, T *R, T *P, const T *Q, const T *B, int64_t m, int64_t t, int64_t rs, int64_t cs,
                     T *rsold, int *state, int parity, double eps, double tol2, int differential, hipStream_t st);

// Register-resident ("small d") product kernel; the queries do not depend on the kernel function.
template <typename T> int64_t mmv_small_max_d();
// Whether the register-resident kernels serve a product of d features with t right-hand sides in all (beyond
// mmv_small_max_d: some single-column products, on operands padded for the LDS-tiled kernel).
template <typename T> bool mmv_small_serves(int64_t d, int64_t t);
// (t: right-hand sides of the call; the fp32 kernels switch to their 32-column variant beyond a few columns)
template <typename T> int mmv_small_b_blocks_per_wg(int64_t dpad, int64_t t);
template <typename T> int mmv_small_wgs_per_cu(int64_t dpad, int64_t t);      // workgroups of that kernel a CU holds at once
template <typename T> int mmv_small_max_cols(int64_t dpad, int64_t t);   // right-hand sides per pass
template <typename T> int mmv_small_width(int64_t dpad, int tc);         // planes the kernel serving tc columns reads

// Planes a planar right-hand side buffer must hold for t columns: kernels compute whole column
// chunks and read zero planes beyond the caller's columns.
constexpr int64_t kColPad = 31;

// LDS-tiled ("large d") product kernel: any padded feature count, up to mmv_large_max_cols columns per pass.
// Writes splits * mmv_large_partials_per_split partial results.
template <typename T> int mmv_large_a_tile_blocks(int64_t t);   // reduction blocks per tile with t columns in all
template <typename T> int mmv_large_b_tile_blocks(int64_t t);   // output blocks per workgroup with t columns in all
template <typename T> int mmv_large_partials_per_split();
template <typename T> int mmv_large_max_cols(int64_t t);   // columns per pass when there are t in all

// The kernels that evaluate K are compiled once per kernel function (the same source with -DFLK_KF=0..4,
// FLK_GAUSSIAN .. FLK_LAPLACIAN_DU): launchers carry the function in their name, and the helpers below pick one.
//   launch_mmv_small_kf*: register-resident product kernel, FLK_EUNSUPPORTED if dpad is out of its range;
//   launch_mmv_large_kf*: LDS-tiled product kernel, writes splits * mmv_large_partials_per_split partials;
//   launch_fmm_kf*:       explicit kernel matrix out[a][b] = K(A_a, B_b); O is the element type of out, whose
//                         rows (A side) are ld elements apart and whose columns (B side) are contiguous;
//   launch_fmm_large_kf*: the same through the LDS-tiled kernel (operands packed for d > 64).
#define FLK_CAT2(a, b) a##b
#define FLK_CAT(a, b) FLK_CAT2(a, b)
#define FLK_DECLARE_KF(KF)                                                                                        \
    template <typename T>                                                                                         \
    int launch_mmv_small_kf##KF(const PackedView &A, const PackedView &B, const T *vecp, int64_t vec_ld, int tt,  \
                                int64_t a_chunk_blocks, int splits, T *partial, hipStream_t st);                  \
    int launch_mmv_small_f32_wide_kf##KF(const PackedView &A, const PackedView &B, const float *vecp,             \
                                         int64_t vec_ld, int tcols, int64_t a_chunk_blocks, int splits,           \
                                         float *partial, hipStream_t st);                                         \
    int launch_mmv_small_f64_wide_kf##KF(const PackedView &A, const PackedView &B, const double *vecp,            \
                                         int64_t vec_ld, int tcols, int64_t a_chunk_blocks, int splits,           \
                                         double *partial, hipStream_t st);                                        \
    template <typename T>                                                                                         \
    int launch_mmv_large_kf##KF(const PackedView &A, const PackedView &B, const T *vecp, int64_t vec_ld,          \
                                int tcols, int a_tile_blocks, int64_t a_tiles_per_chunk, int splits, T *partial,  \
                                hipStream_t st);                                                                  \
    template <typename T, typename O>                                                                             \
    int launch_fmm_kf##KF(const PackedView &A, const PackedView &B, O *out, int64_t ld, hipStream_t st);          \
    template <typename T, typename O>                                                                             \
    int launch_fmm_large_kf##KF(const PackedView &A, const PackedView &B, O *out, int64_t ld, hipStream_t st);
FLK_DECLARE_KF(0)
FLK_DECLARE_KF(1)
FLK_DECLARE_KF(2)
FLK_DECLARE_KF(3)
FLK_DECLARE_KF(4)
#undef FLK_DECLARE_KF

constexpr int kNumKernelFns = 5;
inline bool valid_kernel_fn(int kf) { return kf >= 0 && kf < kNumKernelFns; }

#define FLK_SWITCH_KF(kf, CALL)                                          \
    switch (kf) {                                                        \
        case 0: return CALL(0);                                          \
        case 1: return CALL(1);                                          \
        case 2: return CALL(2);                                          \
        case 3: return CALL(3);                                          \
        case 4: return CALL(4);                                          \
        default: return fail(FLK_EINVAL, "unknown kernel function %d", kf); \
    }

template <typename T>
inline int launch_mmv_small(int kf, const PackedView &A, const PackedView &B, const T *vecp, int64_t vec_ld, int tt,
                            int64_t a_chunk_blocks, int splits, T *partial, hipStream_t st) {
#define FLK_CALL(KF) launch_mmv_small_kf##KF<T>(A, B, vecp, vec_ld, tt, a_chunk_blocks, splits, partial, st)
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}
template <typename T>
inline int launch_mmv_large(int kf, const PackedView &A, const PackedView &B, const T *vecp, int64_t vec_ld, int tcols,
                            int a_tile_blocks, int64_t a_tiles_per_chunk, int splits, T *partial, hipStream_t st) {
#define FLK_CALL(KF) \
    launch_mmv_large_kf##KF<T>(A, B, vecp, vec_ld, tcols, a_tile_blocks, a_tiles_per_chunk, splits, partial, st)
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}
template <typename T, typename O>
inline int launch_fmm(int kf, const PackedView &A, const PackedView &B, O *out, int64_t ld, hipStream_t st) {
#define FLK_CALL(KF) (launch_fmm_kf##KF<T, O>(A, B, out, ld, st))
    FLK_SWITCH_KF(kf, FLK_CALL)
#undef FLK_CALL
}

}  // namespace flk
