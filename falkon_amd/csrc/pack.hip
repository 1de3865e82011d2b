// Prologue / epilogue kernels: operand packing, planar right-hand sides, split reduction.
#include "flk_common.h"

namespace flk {

// ---------------------------------------------------------------------------
// pack: X[n,d] (any unit-stride order) -> [nblk][dpad][BLK] scaled by scale/sigma (scale = sqrt(log2 e)
// for the Gaussian, 1 for the other kernels),
// plus hnorm[row] = -1/2 |x~|^2.  One workgroup per block of BLK rows; a
// BLK x 32 tile goes through LDS so that both the read (along the unit stride
// of X) and the write (along rows of the block) are coalesced.
// Row r of an f64 block is stored at position 4*(r%4) + r/4: the 16x16x4 MFMA
// hands lane quarter q the accumulator rows q, q+4, q+8, q+12, and with this
// order those are four consecutive rows of the matrix.
// ---------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ int block_pos(int r);
template <> __device__ __forceinline__ int block_pos<float>(int r) { return r; }
template <> __device__ __forceinline__ int block_pos<double>(int r) { return 4 * (r & 3) + (r >> 2); }

// TI is the caller's element type, T the type of the packed operand (T = double with TI = float serves
// kernel matrices that are computed in double precision from single precision data).
// Packs block blk of one operand; returns the block's half norm of row tid (threads tid < BLK; 0 for the others).
template <typename TI, typename T>
__device__ __forceinline__ T pack_block(int64_t blk, const TI *__restrict__ X, int64_t n, int64_t d, int64_t rs,
                                        int64_t cs, const TI *__restrict__ sigma, int64_t n_sigma, double scale,
                                        T *__restrict__ pdata, T *__restrict__ hnorm, int64_t dpad, bool one_pad) {
    constexpr int BLK = Geo<T>::BLK;
    constexpr int KT = 32;                       // features per LDS tile
    __shared__ T tile[BLK][KT + 1];
    __shared__ double nrm[BLK];
    const int tid = threadIdx.x;
    const int64_t row0 = blk * BLK;
    if (tid < BLK) nrm[tid] = 0.0;
    const bool row_major = (cs == 1);
    for (int64_t k0 = 0; k0 < dpad; k0 += KT) {
        __syncthreads();
        // load + scale
        for (int e = tid; e < BLK * KT; e += 256) {
            int r, k;
            if (row_major) { r = e / KT; k = e % KT; } else { k = e / BLK; r = e % BLK; }
            int64_t row = row0 + r, kk = k0 + k;
            T val = T(0);
            if (row < n && kk < d) {
                double s = scale / (double)sigma[n_sigma == 1 ? 0 : kk];
                val = (T)((double)X[row * rs + kk * cs] * s);
            } else if (one_pad && kk == d) {
                val = T(1);          // padding feature of odd-d fp32 operands: multiplies the folded half norm
            }
            tile[r][k] = val;
        }
        __syncthreads();
        // store feature-major
        for (int e = tid; e < BLK * KT; e += 256) {
            int k = e / BLK, r = e % BLK;
            int64_t kk = k0 + k;
            if (kk < dpad) pdata[(blk * dpad + kk) * BLK + block_pos<T>(r)] = tile[r][k];
        }
        if (tid < BLK) {
            double s = 0.0;
            int kmax = (int)((d - k0) < KT ? (d - k0) : KT);   // real features only
            for (int k = 0; k < kmax; k++) { double x = (double)tile[tid][k]; s += x * x; }
            nrm[tid] += s;
        }
    }
    T h = T(0);
    if (tid < BLK) {
        h = (T)(-0.5 * nrm[tid]);
        hnorm[row0 + tid] = h;
    }
    return h;
}

template <typename TI, typename T>
__global__ void __launch_bounds__(256) pack_kernel(const TI *__restrict__ X, int64_t n, int64_t d, int64_t rs,
                                                   int64_t cs, const TI *__restrict__ sigma, int64_t n_sigma,
                                                   double scale, T *__restrict__ pdata, T *__restrict__ hnorm,
                                                   int64_t dpad, bool one_pad) {
    pack_block<TI, T>(blockIdx.x, X, n, d, rs, cs, sigma, n_sigma, scale, pdata, hnorm, dpad, one_pad);
}

template <typename TI, typename T>
int launch_pack(const TI *X, int64_t n, int64_t d, int64_t rs, int64_t cs, const TI *sigma, int64_t n_sigma,
                double scale, T *pdata, T *hnorm, int64_t dpad, int64_t nblk, bool one_pad, hipStream_t st) {
    if (nblk == 0) return FLK_OK;
    hipLaunchKernelGGL((pack_kernel<TI, T>), dim3((unsigned)nblk), dim3(256), 0, st, X, n, d, rs, cs, sigma, n_sigma, scale,
                       pdata, hnorm, dpad, one_pad);
    FLK_LAUNCH_CHECK("pack_kernel");
    return FLK_OK;
}
template int launch_pack<float, float>(const float *, int64_t, int64_t, int64_t, int64_t, const float *, int64_t,
                                       double, float *, float *, int64_t, int64_t, bool, hipStream_t);
template int launch_pack<double, double>(const double *, int64_t, int64_t, int64_t, int64_t, const double *, int64_t,
                                         double, double *, double *, int64_t, int64_t, bool, hipStream_t);
template int launch_pack<float, double>(const float *, int64_t, int64_t, int64_t, int64_t, const float *, int64_t,
                                        double, double *, double *, int64_t, int64_t, bool, hipStream_t);

// ---------------------------------------------------------------------------
// vec_planar: v[n,t] with element strides (rs, cs) -> vp[t + zero_planes][npad]: rows past n and the
// zero_planes planes past t are zero.  Rows whose half norm (of the operand the vector multiplies) is not
// finite become NaN: their kernel values were clamped to numbers, and 0 * NaN brings the NaN back.
// ---------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ bool finite_value(T x) { return x - x == T(0); }
template <typename T> __device__ __forceinline__ T quiet_nan() { return T(0) / T(0); }
template <> __device__ __forceinline__ float quiet_nan<float>() { return __uint_as_float(0x7fc00000u); }
template <> __device__ __forceinline__ double quiet_nan<double>() { return __longlong_as_double(0x7ff8000000000000ll); }

template <typename T>
__global__ void __launch_bounds__(256) vec_planar_kernel(const T *__restrict__ v, int64_t n, int64_t rs, int64_t cs,
                                                         T *__restrict__ vp, int64_t npad, int64_t tcols,
                                                         const T *__restrict__ row_half_norm) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t t = blockIdx.y;
    if (i >= npad) return;
    T val = (i < n && t < tcols) ? v[i * rs + t * cs] : T(0);
    if (row_half_norm && i < n && t < tcols && !finite_value(row_half_norm[i])) val = quiet_nan<T>();
    vp[t * npad + i] = val;
}

// ---------------------------------------------------------------------------
// The whole prologue of a one-shot product in one launch: workgroups 0 .. nblk1 - 1 pack the output-side operand,
// the others the reduction-side operand, and each of those also writes its BLK rows of the planar right-hand side
// (it holds the rows' half norms, which decide where the vector becomes NaN).  Small products are bound by their
// launches: three launches fewer than pack + pack + vec_planar.
// ---------------------------------------------------------------------------
template <typename T>
struct PackArgs {
    const T *X;
    int64_t n, rs, cs;
    T *pdata, *hnorm;
    int64_t nblk;
};
template <typename T>
__global__ void __launch_bounds__(256) pack_pair_kernel(PackArgs<T> out_side, PackArgs<T> red_side, int64_t d,
                                                        const T *__restrict__ sigma, int64_t n_sigma, double scale,
                                                        int64_t dpad, bool one_pad, const T *__restrict__ v,
                                                        int64_t v_rs, int64_t v_cs, T *__restrict__ vp, int64_t tcols,
                                                        int64_t planes) {
    constexpr int BLK = Geo<T>::BLK;
    __shared__ T hrow[BLK];
    int64_t blk = blockIdx.x;
    if (blk < out_side.nblk) {
        pack_block<T, T>(blk, out_side.X, out_side.n, d, out_side.rs, out_side.cs, sigma, n_sigma, scale, out_side.pdata,
                         out_side.hnorm, dpad, one_pad);
        return;
    }
    blk -= out_side.nblk;
    const T h = pack_block<T, T>(blk, red_side.X, red_side.n, d, red_side.rs, red_side.cs, sigma, n_sigma, scale,
                                 red_side.pdata, red_side.hnorm, dpad, one_pad);
    const int tid = threadIdx.x;
    if (tid < BLK) hrow[tid] = h;
    __syncthreads();
    const int64_t npad = red_side.nblk * BLK;
    for (int64_t e = tid; e < planes * BLK; e += 256) {
        const int r = (int)(e % BLK);
        const int64_t t = e / BLK, i = blk * BLK + r;
        T val = (i < red_side.n && t < tcols) ? v[i * v_rs + t * v_cs] : T(0);
        if (i < red_side.n && t < tcols && !finite_value(hrow[r])) val = quiet_nan<T>();
        vp[t * npad + i] = val;
    }
}
template <typename T>
int launch_pack_pair(const T *X1, int64_t n1, int64_t rs1, int64_t cs1, T *pdata1, T *hnorm1, int64_t nblk1, const T *X2,
                     int64_t n2, int64_t rs2, int64_t cs2, T *pdata2, T *hnorm2, int64_t nblk2, int64_t d, const T *sigma,
                     int64_t n_sigma, double scale, int64_t dpad, bool one_pad, const T *v, int64_t v_rs, int64_t v_cs,
                     T *vp, int64_t tcols, int64_t zero_planes, hipStream_t st) {
    if (nblk1 + nblk2 == 0) return FLK_OK;
    PackArgs<T> a{X1, n1, rs1, cs1, pdata1, hnorm1, nblk1}, b{X2, n2, rs2, cs2, pdata2, hnorm2, nblk2};
    hipLaunchKernelGGL(pack_pair_kernel<T>, dim3((unsigned)(nblk1 + nblk2)), dim3(256), 0, st, a, b, d, sigma, n_sigma,
                       scale, dpad, one_pad, v, v_rs, v_cs, vp, tcols, tcols > 0 ? tcols + zero_planes : 0);
    FLK_LAUNCH_CHECK("pack_pair_kernel");
    return FLK_OK;
}
template int launch_pack_pair<float>(const float *, int64_t, int64_t, int64_t, float *, float *, int64_t, const float *,
                                     int64_t, int64_t, int64_t, float *, float *, int64_t, int64_t, const float *, int64_t,
                                     double, int64_t, bool, const float *, int64_t, int64_t, float *, int64_t, int64_t,
                                     hipStream_t);
template int launch_pack_pair<double>(const double *, int64_t, int64_t, int64_t, double *, double *, int64_t,
                                      const double *, int64_t, int64_t, int64_t, double *, double *, int64_t, int64_t,
                                      const double *, int64_t, double, int64_t, bool, const double *, int64_t, int64_t,
                                      double *, int64_t, int64_t, hipStream_t);

template <typename T>
__global__ void __launch_bounds__(256) zero_fill_kernel(T *__restrict__ p, int64_t count) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) p[i] = T(0);
}
template <typename T>
int launch_zero_fill(T *p, int64_t count, hipStream_t st) {
    if (count <= 0) return FLK_OK;
    hipLaunchKernelGGL(zero_fill_kernel<T>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, p, count);
    FLK_LAUNCH_CHECK("zero_fill_kernel");
    return FLK_OK;
}
template int launch_zero_fill<float>(float *, int64_t, hipStream_t);
template int launch_zero_fill<double>(double *, int64_t, hipStream_t);
template <typename T>
int launch_vec_planar(const T *v, int64_t n, int64_t t, int64_t rs, int64_t cs, T *vp, int64_t npad,
                      int64_t zero_planes, const T *row_half_norm, hipStream_t st) {
    if (npad == 0 || t == 0) return FLK_OK;
    hipLaunchKernelGGL(vec_planar_kernel<T>, dim3((unsigned)((npad + 255) / 256), (unsigned)(t + zero_planes)),
                       dim3(256), 0, st, v, n, rs, cs, vp, npad, t, row_half_norm);
    FLK_LAUNCH_CHECK("vec_planar_kernel");
    return FLK_OK;
}
template int launch_vec_planar<float>(const float *, int64_t, int64_t, int64_t, int64_t, float *, int64_t, int64_t,
                                      const float *, hipStream_t);
template int launch_vec_planar<double>(const double *, int64_t, int64_t, int64_t, int64_t, double *, int64_t, int64_t,
                                       const double *, hipStream_t);

// ---------------------------------------------------------------------------
// finalize: out[b,t] = sum_s partial[s][t][b] (+ addend[b,t]); fixed summation
// order, so results are reproducible run to run (no atomics anywhere).
// With zero_pad the rows n_b..nb_pad of a planar output are cleared as well.
// Output rows whose half norm is not finite (a NaN or an infinity in the data row) become NaN.
// ---------------------------------------------------------------------------
// Sum of the partial results sp0 .. sp1 of one output element in double precision, in order; eight loads in flight
// (one load per addition costs a memory round trip each: 256 partial results of 1000 outputs took 0.4 ms).
template <typename T>
__device__ __forceinline__ double sum_partials(const T *__restrict__ p, int64_t stride, int sp0, int sp1) {
    double s = 0.0;
    int sp = sp0;
    for (; sp + 8 <= sp1; sp += 8) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; u++) x[u] = p[(int64_t)(sp + u) * stride];
#pragma unroll
        for (int u = 0; u < 8; u++) s += (double)x[u];
    }
    for (; sp < sp1; sp++) s += (double)p[(int64_t)sp * stride];
    return s;
}

template <typename T>
__global__ void __launch_bounds__(256) finalize_kernel(const T *__restrict__ partial, int splits, int64_t tt,
                                                       int64_t nb, int64_t nb_pad, const T *__restrict__ addend,
                                                       int64_t add_rs, int64_t add_cs, T *__restrict__ out,
                                                       int64_t out_rs, int64_t out_cs, bool zero_pad,
                                                       const T *__restrict__ row_half_norm) {
    int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t t = blockIdx.y;
    if (b >= nb_pad) return;
    if (b >= nb) {
        if (zero_pad) out[b * out_rs + t * out_cs] = T(0);
        return;
    }
    double s = sum_partials(partial + t * nb_pad + b, tt * nb_pad, 0, splits);
    if (addend) s += (double)addend[b * add_rs + t * add_cs];
    T res = (T)s;
    if (row_half_norm && !finite_value(row_half_norm[b])) res = quiet_nan<T>();
    out[b * out_rs + t * out_cs] = res;
}

// The same for many partial results of few outputs (the K^T u side of a product with few centres: hundreds of splits
// of a thousand rows): 64 outputs per workgroup, each of its NW waves sums its share of the partial results (a
// contiguous range, in order) and the NW sums are added in order, so the result does not depend on timing.  Four waves up
// to kFinalizeWideMin partial results, sixteen beyond (a thousand outputs are sixteen workgroups: with 1737 partial
// results each, four waves per workgroup took 23 us, a quarter of them spent by each wave in one dependent chain).
constexpr int kFinalizeSplitMin = 16;
constexpr int kFinalizeWideMin = 256;
template <typename T, int NW>
__global__ void __launch_bounds__(64 * NW) finalize_split_kernel(const T *__restrict__ partial, int splits, int64_t tt,
                                                                 int64_t nb, int64_t nb_pad, const T *__restrict__ addend,
                                                                 int64_t add_rs, int64_t add_cs, T *__restrict__ out,
                                                                 int64_t out_rs, int64_t out_cs, bool zero_pad,
                                                                 const T *__restrict__ row_half_norm) {
    __shared__ double red[NW][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t b = (int64_t)blockIdx.x * 64 + lane;
    const int64_t t = blockIdx.y;
    const int per = (splits + NW - 1) / NW;
    const int sp0 = wave * per < splits ? wave * per : splits;
    const int sp1 = sp0 + per < splits ? sp0 + per : splits;
    red[wave][lane] = b < nb ? sum_partials(partial + t * nb_pad + b, tt * nb_pad, sp0, sp1) : 0.0;
    __syncthreads();
    if (wave != 0 || b >= nb_pad) return;
    if (b >= nb) {
        if (zero_pad) out[b * out_rs + t * out_cs] = T(0);
        return;
    }
    double s = red[0][lane];
#pragma unroll
    for (int w = 1; w < NW; w++) s += red[w][lane];
    if (addend) s += (double)addend[b * add_rs + t * add_cs];
    T res = (T)s;
    if (row_half_norm && !finite_value(row_half_norm[b])) res = quiet_nan<T>();
    out[b * out_rs + t * out_cs] = res;
}

template <typename T>
int launch_finalize(const T *partial, int splits, int64_t t, int64_t nb, int64_t nb_pad, const T *addend,
                    int64_t add_rs, int64_t add_cs, T *out, int64_t out_rs, int64_t out_cs, bool zero_pad,
                    const T *row_half_norm, hipStream_t st) {
    if (nb_pad == 0 || t == 0) return FLK_OK;
    if (splits >= kFinalizeWideMin)
        hipLaunchKernelGGL((finalize_split_kernel<T, 16>), dim3((unsigned)((nb_pad + 63) / 64), (unsigned)t), dim3(1024), 0, st,
                           partial, splits, t, nb, nb_pad, addend, add_rs, add_cs, out, out_rs, out_cs, zero_pad,
                           row_half_norm);
    else if (splits >= kFinalizeSplitMin)
        hipLaunchKernelGGL((finalize_split_kernel<T, 4>), dim3((unsigned)((nb_pad + 63) / 64), (unsigned)t), dim3(256), 0, st,
                           partial, splits, t, nb, nb_pad, addend, add_rs, add_cs, out, out_rs, out_cs, zero_pad,
                           row_half_norm);
    else
        hipLaunchKernelGGL(finalize_kernel<T>, dim3((unsigned)((nb_pad + 255) / 256), (unsigned)t), dim3(256), 0, st,
                           partial, splits, t, nb, nb_pad, addend, add_rs, add_cs, out, out_rs, out_cs, zero_pad,
                           row_half_norm);
    FLK_LAUNCH_CHECK("finalize_kernel");
    return FLK_OK;
}
template int launch_finalize<float>(const float *, int, int64_t, int64_t, int64_t, const float *, int64_t, int64_t,
                                    float *, int64_t, int64_t, bool, const float *, hipStream_t);
template int launch_finalize<double>(const double *, int, int64_t, int64_t, int64_t, const double *, int64_t, int64_t,
                                     double *, int64_t, int64_t, bool, const double *, hipStream_t);

}  // namespace flk
