// Explicit kernel matrix out[a][b] = f(A~_a . B~_b + hA_a + hB_b) from two packed operands (f: kernel_fn.h),
// fp32 or fp64 arithmetic, stored as fp32 or fp64 (gfx950).  This is the K(C, C) the preconditioner
// factorises once per fit; it is bound by the HBM writes of the result (or, computed in fp64, by the
// software exp2), so the kernel is kept simple: no LDS, no barriers.
//
// A wave owns FA x FB blocks (64 x 64 entries in fp32, 32 x 64 in fp64) and walks over the features; the
// packed layout is already in MFMA operand order, so each step is one element per lane and operand
// block straight from global memory (the tiles of neighbouring waves overlap and sit in L2), read two
// steps ahead of the MFMAs that consume it.  The epilogue adds the half norms, applies exp2 with the
// clamp K <= 1 (the reference's clamp of the squared distance, falkon/kernels/distance_kernel.py:100)
// and stores: consecutive lanes hold consecutive columns, so every store covers whole 128-byte runs.  The
// stores are non-temporal: the result is written once and never read here, and ordinary stores evicted
// the operand tiles from L2 (M = 50 000, d = 28: 5.9 ms with ordinary stores, 3.8 ms without).
#include "flk_common.h"
#include "kernel_fn.h"
#include "mfma_traits.h"

#ifndef FLK_KF
#define FLK_KF FLK_GAUSSIAN
#endif

namespace flk {

template <typename T> struct FmmCfg;
template <> struct FmmCfg<float>  { static constexpr int FA = 2, FB = 2; };
template <> struct FmmCfg<double> { static constexpr int FA = 2, FB = 4; };
constexpr int kFmmWavesA = 2, kFmmWavesB = 2;

// KF (= FLK_KF) is a template parameter only to give every kernel function's instantiations their own symbols
template <typename T, typename O, int FA, int FB, int KF>
__global__ void __launch_bounds__(64 * kFmmWavesA * kFmmWavesB)
    fmm_kernel(const T *__restrict__ PA, const T *__restrict__ hA, const T *__restrict__ PB, const T *__restrict__ hB,
               int64_t na_blocks, int64_t nb_blocks, int64_t n_a, int64_t n_b, int64_t dpad, int64_t b_tiles,
               O *__restrict__ out, int64_t ld) {
    typedef LTraits<T> TR;
    typedef typename TR::acc_t acc_t;
    typedef typename TR::vec4_t vec4_t;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % TR::BLK, lg = lane / TR::BLK;
    const int64_t steps = dpad / TR::KG;
    const int64_t tile_a = (int64_t)blockIdx.x / b_tiles, tile_b = (int64_t)blockIdx.x % b_tiles;
    const int64_t ablk0 = (tile_a * kFmmWavesA + wave / kFmmWavesB) * FA;
    const int64_t bblk0 = (tile_b * kFmmWavesB + wave % kFmmWavesB) * FB;
    if (ablk0 >= na_blocks || bblk0 >= nb_blocks) return;        // nothing below synchronises across waves

    // lane group lg of a wave consumes the features lg*steps .. lg*steps+steps-1 of a block, one per step
    const T *pa[FA], *pb[FB];
#pragma unroll
    for (int p = 0; p < FA; p++) {
        int64_t blk = ablk0 + p < na_blocks ? ablk0 + p : na_blocks - 1;   // past the end: recompute the last block
        pa[p] = PA + (blk * dpad + (int64_t)lg * steps) * TR::BLK + j;
    }
#pragma unroll
    for (int q = 0; q < FB; q++) {
        int64_t blk = bblk0 + q < nb_blocks ? bblk0 + q : nb_blocks - 1;
        pb[q] = PB + (blk * dpad + (int64_t)lg * steps) * TR::BLK + j;
    }

    acc_t acc[FA][FB];
#pragma unroll
    for (int p = 0; p < FA; p++)
#pragma unroll
        for (int q = 0; q < FB; q++)
#pragma unroll
            for (int r = 0; r < TR::ACCN; r++) acc[p][q][r] = T(0);

    // operands travel two steps ahead of the MFMAs that consume them (three register sets in rotation);
    // reads past the last step repeat it
    T av[3][FA], bv[3][FB];
    auto read_step = [&](int set, int64_t s) {
        const int64_t sc = s < steps ? s : steps - 1;
#pragma unroll
        for (int p = 0; p < FA; p++) av[set][p] = pa[p][sc * TR::BLK];
#pragma unroll
        for (int q = 0; q < FB; q++) bv[set][q] = pb[q][sc * TR::BLK];
    };
    auto mfma_step = [&](int set) {
#pragma unroll
        for (int p = 0; p < FA; p++)
#pragma unroll
            for (int q = 0; q < FB; q++) acc[p][q] = TR::mfma(av[set][p], bv[set][q], acc[p][q]);
    };
    read_step(0, 0);
    read_step(1, 1);
    int64_t s = 0;
    for (; s + 3 <= steps; s += 3) {
        read_step(2, s + 2); mfma_step(0);
        read_step(0, s + 3); mfma_step(1);
        read_step(1, s + 4); mfma_step(2);
    }
    if (s < steps) { read_step(2, s + 2); mfma_step(0); s++; }
    if (s < steps) { mfma_step(1); s++; }

#pragma unroll
    for (int q = 0; q < FB; q++) {
        const int64_t bb = bblk0 + q;
        if (bb >= nb_blocks) break;
        const int64_t col = bb * TR::BLK + TR::out_row(j);
        const T hb = hB[col];                                      // half norms cover the padded rows
#pragma unroll
        for (int p = 0; p < FA; p++) {
            const int64_t ab = ablk0 + p;
            if (ab >= na_blocks) break;
#pragma unroll
            for (int g = 0; g < TR::NG; g++) {
                const int64_t row0 = ab * TR::BLK + TR::group_off(g, lg);   // four consecutive matrix rows
                const vec4_t hn = *(const vec4_t *)(&hA[row0]);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // h - h is 0, or NaN where a row holds a NaN or an infinity: the kernel functions clamp their
                    // argument, which would turn such an entry into a number
                    const T h = hn[e] + hb;
                    const T k = kernel_value<FLK_KF>(acc[p][q][4 * g + e] + h) + (h - h);
                    if (row0 + e < n_a && col < n_b) __builtin_nontemporal_store((O)k, &out[(row0 + e) * ld + col]);
                }
            }
        }
    }
}

template <typename T, typename O>
int FLK_CAT(launch_fmm_kf, FLK_KF)(const PackedView &A, const PackedView &B, O *out, int64_t ld, hipStream_t st) {
    typedef FmmCfg<T> C;
    if (A.dpad != B.dpad || A.d != B.d) return fail(FLK_EINVAL, "fmm: operands packed with different feature counts");
    if (A.n == 0 || B.n == 0) return FLK_OK;
    // beyond the register-resident feature counts the LDS-tiled kernel evaluates K faster (it stages both operand
    // tiles in LDS instead of reading them per step)
    if (A.d > kSmallMaxD) return FLK_CAT(launch_fmm_large_kf, FLK_KF)<T, O>(A, B, out, ld, st);
    const int64_t a_tiles = (A.nblk + kFmmWavesA * C::FA - 1) / (kFmmWavesA * C::FA);
    const int64_t b_tiles = (B.nblk + kFmmWavesB * C::FB - 1) / (kFmmWavesB * C::FB);
    if (a_tiles * b_tiles > (int64_t)0x7fffffff) return fail(FLK_EUNSUPPORTED, "fmm: more tiles than one launch holds");
    hipLaunchKernelGGL((fmm_kernel<T, O, C::FA, C::FB, FLK_KF>), dim3((unsigned)(a_tiles * b_tiles)),
                       dim3(64 * kFmmWavesA * kFmmWavesB), 0, st, (const T *)A.data, (const T *)A.hnorm,
                       (const T *)B.data, (const T *)B.hnorm, A.nblk, B.nblk, A.n, B.n, A.dpad, b_tiles, out, ld);
    FLK_LAUNCH_CHECK("fmm_kernel");
    return FLK_OK;
}
template int FLK_CAT(launch_fmm_kf, FLK_KF)<float, float>(const PackedView &, const PackedView &, float *, int64_t,
                                                          hipStream_t);
template int FLK_CAT(launch_fmm_kf, FLK_KF)<double, double>(const PackedView &, const PackedView &, double *, int64_t,
                                                            hipStream_t);
template int FLK_CAT(launch_fmm_kf, FLK_KF)<double, float>(const PackedView &, const PackedView &, float *, int64_t,
                                                           hipStream_t);

}  // namespace flk
