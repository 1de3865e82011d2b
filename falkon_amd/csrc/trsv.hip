// Blocked triangular solves with a resident Cholesky factor, for one to four right-hand sides (gfx950).
//
// The preconditioned conjugate-gradient iteration solves with the two M x M factors of the preconditioner four
// times (falkon/preconditioner/flk_preconditioner.py:166-256: invA, invT, invTt, invAt; the reference calls the
// library's trsm there), each with as many right-hand sides as the problem has outputs: one, for config 5.  A
// library trsm with one right-hand side is latency bound (M = 50 000: about 100 ms), while a solve only has to
// read the triangle once: HBM bound, 5 GB in fp32.  The factor is cut into diagonal blocks of `block` rows whose
// inverses the caller computes once; a solve is then a chain over the blocks of
//   a panel product  (the rows of the factor left of / below a diagonal block times the part of x already known,
//                     or, in the pushing form, the panel's transpose times the block just solved), and
//   a block product  x_k = inverse(diagonal block k) r_k,
// two launches per block.  Panels always consist of long contiguous rows (of L where L is stored row-major, of L^T
// where it is stored column-major), so both directions of both layouts need two kernels only:
//   rows_times_vector      out[i] = base[i] - sum_j P[i][j] x[j]     (a workgroup owns 4 rows, reads x once)
//   rows_transposed_times  r[j]  -= sum_i P[i][j] x[i]                (a workgroup owns a strip of columns)
// Neither uses atomics: every sum is taken in a fixed order (four-term fp32 / fp64 products accumulated in double
// precision, then a fixed tree over the lanes and waves), so a solve is reproducible run to run.
#include "flk_common.h"

namespace flk {

constexpr int kTrsvThreads = 256;
constexpr int kTrsvRows = 4;           // rows per workgroup of rows_times_vector
constexpr int kTrsvMaxRhs = 4;

template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct Vec4<double> { typedef double type __attribute__((ext_vector_type(4))); };
template <typename T> struct Vec2;
template <> struct Vec2<float> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct Vec2<double> { typedef double type __attribute__((ext_vector_type(2))); };

// out[i*?] for rows i0 .. i0+nr of P (row i at P + i * ldp, columns c0 .. c1 used):
//   out[t][i] = (base ? base[t][i] : 0) - sign * sum_{j in [c0, c1)} P[i][j] * x[t][j]      with sign = +1 (subtract)
// or, with `plain` set, out[t][i] = sum_j P[i][j] x[t][j] (the product with an inverted diagonal block).
// tri: 0 = all rows use [c0, c1); 1 = lower triangle (row i uses columns up to c0 + i, inclusive);
//      2 = upper triangle (row i uses columns from c0 + i on).  Rows and vectors: right-hand side t at + t * ldv.
// VEC: elements per load (4 when every row start and c0 are multiples of 4 elements and 16-byte aligned, else 1).
template <typename T, int NT, int VEC>
__global__ void __launch_bounds__(kTrsvThreads) rows_times_vector(const T *__restrict__ P, int64_t ldp, int64_t nr,
                                                                   int64_t c0, int64_t c1, int tri, const T *__restrict__ x,
                                                                   int64_t ldx, const T *__restrict__ base, int64_t ldb,
                                                                   T *__restrict__ out, int64_t ldo, int plain,
                                                                   const T *__restrict__ sub, int nsub, int64_t sub_stride,
                                                                   int64_t ldsub) {
    __shared__ double red[kTrsvThreads / 64][kTrsvRows][NT];
    const int64_t i0 = (int64_t)blockIdx.x * kTrsvRows;
    int64_t lo = c0, hi = c1;
    if (tri == 1) { const int64_t last = i0 + kTrsvRows - 1 < nr - 1 ? i0 + kTrsvRows - 1 : nr - 1; hi = c0 + last + 1; }
    if (tri == 2) lo = c0 + (i0 / VEC) * VEC;
    if (hi > c1) hi = c1;
    double acc[kTrsvRows][NT];
#pragma unroll
    for (int r = 0; r < kTrsvRows; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[r][t] = 0.0;
    const T *rows[kTrsvRows];
#pragma unroll
    for (int r = 0; r < kTrsvRows; r++) rows[r] = P + (i0 + r < nr ? i0 + r : nr - 1) * ldp;

    if constexpr (VEC == 4) {
        typedef typename Vec4<T>::type V;
        const int64_t full = lo + ((hi - lo) / 4) * 4;
#pragma unroll 2
        for (int64_t j = lo + 4 * (int64_t)threadIdx.x; j < full; j += 4 * kTrsvThreads) {
            V xv[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                xv[t] = *(const V *)(x + t * ldx + j);
                for (int g = 0; g < nsub; g++) xv[t] -= *(const V *)(sub + g * sub_stride + t * ldsub + j);
            }
#pragma unroll
            for (int r = 0; r < kTrsvRows; r++) {
                const V p = __builtin_nontemporal_load((const V *)(rows[r] + j));
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const T s = p[0] * xv[t][0] + p[1] * xv[t][1] + p[2] * xv[t][2] + p[3] * xv[t][3];
                    acc[r][t] += (double)s;
                }
            }
        }
        for (int64_t j = full + threadIdx.x; j < hi; j += kTrsvThreads)
#pragma unroll
            for (int t = 0; t < NT; t++) {
                T xe = x[t * ldx + j];
                for (int g = 0; g < nsub; g++) xe -= sub[g * sub_stride + t * ldsub + j];
#pragma unroll
                for (int r = 0; r < kTrsvRows; r++) acc[r][t] += (double)(rows[r][j] * xe);
            }
    } else {
        for (int64_t j = lo + threadIdx.x; j < hi; j += kTrsvThreads)
#pragma unroll
            for (int t = 0; t < NT; t++) {
                T xe = x[t * ldx + j];
                for (int g = 0; g < nsub; g++) xe -= sub[g * sub_stride + t * ldsub + j];
#pragma unroll
                for (int r = 0; r < kTrsvRows; r++) acc[r][t] += (double)(rows[r][j] * xe);
            }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int r = 0; r < kTrsvRows; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) {
            double s = acc[r][t];
            for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off, 64);
            if (lane == 0) red[wave][r][t] = s;
        }
    __syncthreads();
    if (threadIdx.x < kTrsvRows * NT) {
        const int r = threadIdx.x / NT, t = threadIdx.x % NT;
        if (i0 + r < nr) {
            double s = 0.0;
            for (int w = 0; w < kTrsvThreads / 64; w++) s += red[w][r][t];
            const double b = (base != nullptr) ? (double)base[t * ldb + i0 + r] : 0.0;
            out[t * ldo + i0 + r] = (T)(plain ? s : b - s);
        }
    }
}

// acc[g][t][j] += sum_{i in row group g} P[i][j] * x[t][i]   for the columns j in [0, nc) of the panel (row i at
// P + i * ldp): the pushing form's update of the part of the right-hand side that is still to be solved.  The rows of
// the panel are cut into groups of kTrsvGroupRows (blockIdx.y); a workgroup owns a strip of 64 * VEC columns of one
// group and adds its sums into that group's own plane of acc (plane g at + g * acc_stride, right-hand side t at
// + t * ldacc), which nobody else writes: no atomics, and every panel keeps thousands of workgroups busy whatever its
// width.  The consumer subtracts the planes from the right-hand side when it solves a block (rows_times_vector's `sub`).
constexpr int kTrsvGroupRows = 512;
template <typename T, int NT, int VEC>
__global__ void __launch_bounds__(kTrsvThreads) rows_transposed_times(const T *__restrict__ P, int64_t ldp, int64_t nr,
                                                                       int64_t nc, const T *__restrict__ x, int64_t ldx,
                                                                       T *__restrict__ acc_out, int64_t acc_stride,
                                                                       int64_t ldacc, int group_rows) {
    constexpr int kWaves = kTrsvThreads / 64;
    __shared__ double red[kWaves][NT][64 * VEC];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: row indices stay scalar
    const int64_t j0 = ((int64_t)blockIdx.x * 64 + lane) * VEC;
    const int64_t r0 = (int64_t)blockIdx.y * group_rows;
    const int64_t r1 = r0 + group_rows < nr ? r0 + group_rows : nr;
    double acc[NT][VEC];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[t][e] = 0.0;
    const bool whole = j0 + VEC <= nc;
    constexpr int kUnroll = 16;
    int64_t i = r0 + wave;
    if (whole) {
        for (; i + (kUnroll - 1) * kWaves < r1; i += kUnroll * kWaves) {
            T p[kUnroll][VEC];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                const T *q = P + (i + u * kWaves) * ldp + j0;
                if constexpr (VEC == 2) {
                    const typename Vec2<T>::type v = __builtin_nontemporal_load((const typename Vec2<T>::type *)q);
                    p[u][0] = v[0]; p[u][1] = v[1];
                } else {
                    p[u][0] = __builtin_nontemporal_load(q);
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++)
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const T xv = x[t * ldx + i + u * kWaves];     // the same for every lane of the wave
#pragma unroll
                    for (int e = 0; e < VEC; e++) acc[t][e] += (double)(p[u][e] * xv);
                }
        }
    }
    for (; i < r1; i += kWaves)
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const T xv = x[t * ldx + i];
#pragma unroll
            for (int e = 0; e < VEC; e++)
                if (j0 + e < nc) acc[t][e] += (double)(P[i * ldp + j0 + e] * xv);
        }
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < VEC; e++) red[wave][t][lane * VEC + e] = acc[t][e];
    __syncthreads();
    // 64 * VEC columns x NT right-hand sides, summed over the waves in order
    T *plane = acc_out + (int64_t)blockIdx.y * acc_stride;
    for (int idx = threadIdx.x; idx < NT * 64 * VEC; idx += kTrsvThreads) {
        const int t = idx / (64 * VEC), c = idx % (64 * VEC);
        const int64_t j = (int64_t)blockIdx.x * 64 * VEC + c;
        if (j < nc) {
            double s = 0.0;
            for (int w = 0; w < kWaves; w++) s += red[w][t][c];
            plane[t * ldacc + j] = (T)((double)plane[t * ldacc + j] + s);
        }
    }
}

template <typename T>
__global__ void fill_zero_kernel(T *__restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = (T)0;
}

template <typename T>
static bool aligned_for(const void *p, int64_t ld, int elems) {
    return ((uintptr_t)p % (elems * sizeof(T))) == 0 && ld % elems == 0;
}

template <typename T, int NT>
static int launch_rows_times_vector(const T *P, int64_t ldp, int64_t nr, int64_t c0, int64_t c1, int tri, const T *x,
                                    int64_t ldx, const T *base, int64_t ldb, T *out, int64_t ldo, int plain,
                                    const T *sub, int nsub, int64_t sub_stride, int64_t ldsub, hipStream_t st) {
    if (nr <= 0) return FLK_OK;
    const dim3 grid((unsigned)((nr + kTrsvRows - 1) / kTrsvRows));
    const bool vec = aligned_for<T>(P, ldp, 4) && aligned_for<T>(x, ldx, 4) && c0 % 4 == 0 &&
                     (nsub == 0 || (aligned_for<T>(sub, ldsub, 4) && sub_stride % 4 == 0));
    if (vec)
        hipLaunchKernelGGL((rows_times_vector<T, NT, 4>), grid, dim3(kTrsvThreads), 0, st, P, ldp, nr, c0, c1, tri, x, ldx,
                           base, ldb, out, ldo, plain, sub, nsub, sub_stride, ldsub);
    else
        hipLaunchKernelGGL((rows_times_vector<T, NT, 1>), grid, dim3(kTrsvThreads), 0, st, P, ldp, nr, c0, c1, tri, x, ldx,
                           base, ldb, out, ldo, plain, sub, nsub, sub_stride, ldsub);
    FLK_LAUNCH_CHECK("rows_times_vector");
    return FLK_OK;
}

template <typename T, int NT>
static int launch_rows_transposed_times(const T *P, int64_t ldp, int64_t nr, int64_t nc, const T *x, int64_t ldx, T *acc,
                                        int64_t acc_stride, int64_t ldacc, hipStream_t st) {
    if (nr <= 0 || nc <= 0) return FLK_OK;
    const int group_rows = kTrsvGroupRows;
    const unsigned groups = (unsigned)((nr + group_rows - 1) / group_rows);
    // strips of 128 columns only where they still give every compute unit a workgroup (measured at M = 50 000:
    // 1.05 ms per solve against 1.07 with 64-column strips throughout; groups of 256 or 1024 rows: 1.07 .. 1.12)
    const bool vec = aligned_for<T>(P, ldp, 2) && (nc / 128) * groups >= 256;
    if (vec) {
        const dim3 grid((unsigned)((nc + 127) / 128), groups);
        hipLaunchKernelGGL((rows_transposed_times<T, NT, 2>), grid, dim3(kTrsvThreads), 0, st, P, ldp, nr, nc, x, ldx, acc,
                           acc_stride, ldacc, group_rows);
    } else {
        const dim3 grid((unsigned)((nc + 63) / 64), groups);
        hipLaunchKernelGGL((rows_transposed_times<T, NT, 1>), grid, dim3(kTrsvThreads), 0, st, P, ldp, nr, nc, x, ldx, acc,
                           acc_stride, ldacc, group_rows);
    }
    FLK_LAUNCH_CHECK("rows_transposed_times");
    return FLK_OK;
}

// Elements of `work` a solve needs: one plane of t x m per row group of a panel (the pushing form's partial sums; the
// form that looks back uses t x m of it as scratch for one block at a time).
int64_t tri_solve_work_elems(int64_t m, int64_t t, int64_t block) {
    const int64_t groups = (block + kTrsvGroupRows - 1) / kTrsvGroupRows;
    return (groups > 1 ? groups : 1) * t * m;
}

// One solve.  L: m x m lower triangular, element (i, j) at L[i * ld + j] (row_major) or L[i + j * ld]; only the part
// strictly below the diagonal blocks is read.  dinv / dinv_t: the inverses of the diagonal blocks and their
// transposes, block k at + k * block * block, row-major with leading dimension `block` (the last block may be
// smaller; its rows still have that leading dimension).  transposed == 0: L x = b, else L^T x = b.
// b, x: t columns of m elements, column c at + c * ldb / ldx.  work: tri_solve_work_elems elements.
template <typename T, int NT>
static int tri_solve_nt(const T *L, int64_t m, int64_t ld, int row_major, const T *dinv, const T *dinv_t, int64_t block,
                        int transposed, const T *b, int64_t ldb, T *x, int64_t ldx, T *work, hipStream_t st) {
    const int64_t nblk = (m + block - 1) / block;
    // the panel of block k: contiguous rows of L (row-major: L[k0:k1, 0:k0]) or of L^T (column-major:
    // (L^T)[k0:k1, k1:m]); "looks back" = the panel multiplies what is already solved
    const bool ascending = !transposed;
    const bool looks_back = (row_major != 0) != (transposed != 0);
    const int groups = (int)((block + kTrsvGroupRows - 1) / kTrsvGroupRows);
    const int64_t plane = (int64_t)NT * m;          // one row group's partial sums: [t][m]
    if (!looks_back && nblk > 1) {
        const int64_t n = groups * plane;
        hipLaunchKernelGGL(fill_zero_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, work, n);
        FLK_LAUNCH_CHECK("fill_zero_kernel");
    }
    for (int64_t step = 0; step < nblk; step++) {
        const int64_t k = ascending ? step : nblk - 1 - step;
        const int64_t k0 = k * block, k1 = k0 + block < m ? k0 + block : m, nb = k1 - k0;
        const T *panel = row_major ? L + k0 * ld : L + k0 * ld + k1;        // row i of the panel at + i * ld
        const int64_t pc = row_major ? k0 : m - k1;                          // its columns
        const int64_t solved0 = row_major ? 0 : k1;                          // the rows of x / r its columns index
        const T *dk = (transposed ? dinv_t : dinv) + k * block * block;
        const int tri = transposed ? 2 : 1;                                  // inverse of lower is lower; its transpose upper
        int rc;
        if (looks_back) {
            // work_k = b_k - panel x[solved]; x_k = dinv_k work_k  (work holds one block at a time: rows k0..k1)
            if (pc > 0) {
                rc = launch_rows_times_vector<T, NT>(panel, ld, nb, 0, pc, 0, x + solved0, ldx, b + k0, ldb, work + k0, m, 0,
                                                     nullptr, 0, 0, 0, st);
                if (rc != FLK_OK) return rc;
                rc = launch_rows_times_vector<T, NT>(dk, block, nb, 0, nb, tri, work + k0, m, nullptr, 0, x + k0, ldx, 1,
                                                     nullptr, 0, 0, 0, st);
            } else {
                rc = launch_rows_times_vector<T, NT>(dk, block, nb, 0, nb, tri, b + k0, ldb, nullptr, 0, x + k0, ldx, 1,
                                                     nullptr, 0, 0, 0, st);
            }
            if (rc != FLK_OK) return rc;
        } else {
            // x_k = dinv_k (b_k - what the panels of the blocks solved so far pushed here); then push panel^T x_k
            rc = launch_rows_times_vector<T, NT>(dk, block, nb, 0, nb, tri, b + k0, ldb, nullptr, 0, x + k0, ldx, 1,
                                                 work + k0, nblk > 1 ? groups : 0, plane, m, st);
            if (rc != FLK_OK) return rc;
            rc = launch_rows_transposed_times<T, NT>(panel, ld, nb, pc, x + k0, ldx, work + solved0, plane, m, st);
            if (rc != FLK_OK) return rc;
        }
    }
    return FLK_OK;
}

template <typename T>
int launch_tri_solve(const T *L, int64_t m, int64_t ld, int row_major, const T *dinv, const T *dinv_t, int64_t block,
                     int transposed, const T *b, int64_t ldb, T *x, int64_t ldx, int64_t t, T *work, hipStream_t st) {
    switch (t) {
        case 1: return tri_solve_nt<T, 1>(L, m, ld, row_major, dinv, dinv_t, block, transposed, b, ldb, x, ldx, work, st);
        case 2: return tri_solve_nt<T, 2>(L, m, ld, row_major, dinv, dinv_t, block, transposed, b, ldb, x, ldx, work, st);
        case 3: return tri_solve_nt<T, 3>(L, m, ld, row_major, dinv, dinv_t, block, transposed, b, ldb, x, ldx, work, st);
        case 4: return tri_solve_nt<T, 4>(L, m, ld, row_major, dinv, dinv_t, block, transposed, b, ldb, x, ldx, work, st);
    }
    return fail(FLK_EUNSUPPORTED, "flk_tri_solve: %lld right-hand sides (1 .. %d per call)", (long long)t, kTrsvMaxRhs);
}
template int launch_tri_solve<float>(const float *, int64_t, int64_t, int, const float *, const float *, int64_t, int,
                                     const float *, int64_t, float *, int64_t, int64_t, float *, hipStream_t);
template int launch_tri_solve<double>(const double *, int64_t, int64_t, int, const double *, const double *, int64_t, int,
                                      const double *, int64_t, double *, int64_t, int64_t, double *, hipStream_t);

}  // namespace flk
