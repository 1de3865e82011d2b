// Cholesky factorisation of one small diagonal tile, together with the inverse of its factor (gfx950).
//
// The preconditioner factorises two M x M matrices (falkon/preconditioner/flk_preconditioner.py:115,152:
// potrf_wrapper).  Blocked, nearly all of that work is matrix products, but the diagonal tiles remain a chain of
// M dependent column steps, and the library routine spends 3 us on each of them (a 4096-row diagonal block: 12.8 ms
// for 2.3e10 flop).  This kernel does the chain for a tile of up to 128 rows inside one workgroup, with the tile
// in registers: a right-looking factorisation (per column: the pivot's square root, the scaled column, the update of the
// trailing lower triangle) and, in the same sweep, the inverse of the factor by forward elimination.  The caller uses
// the inverse to turn the triangular solve of the panel below the tile into a matrix product.
#include "flk_common.h"

namespace flk {

constexpr int kPotrfThreads = 512;
constexpr int kPotrfTile = 128;        // rows of a tile: 32 x 16 threads own 4 x 8 elements each
constexpr int kPotrfOwnRows = kPotrfTile / 32, kPotrfOwnCols = kPotrfTile / 16;

// Square root of a positive pivot and its reciprocal.  Single precision: the hardware's reciprocal square root as the
// seed and one correction each (the library's sqrt and division cost some twenty dependent instructions per column
// step, on the critical path of a chain of 128 steps); double precision: the library routines.
__device__ __forceinline__ void pivot_root(float d, float &l, float &rl) {
    const float y = __builtin_amdgcn_rsqf(d);
    const float g = d * y;
    l = __builtin_fmaf(__builtin_fmaf(-g, g, d), 0.5f * y, g);
    rl = __builtin_fmaf(__builtin_fmaf(-l, y, 1.0f), y, y);
}
__device__ __forceinline__ void pivot_root(double d, double &l, double &rl) {
    l = sqrt(d);
    rl = 1.0 / l;
}

// A: n x n (n <= 128), element (i, j) at A[i * lda + j]; the lower triangle is read and overwritten with the factor,
// the rest is left alone.  inv: n x n at inv[i * ldinv + j], the inverse of the factor with zeros above the diagonal.
// info: left alone on success; a pivot that is not positive (or is NaN) at row j stores info_base + j + 1 there
// unless it already holds a failure, and the outputs are then NaN from that row on.
//
// Thread (ti, tc) of the 32 x 16 grid (two waves per SIMD: a lone wave issues a vector instruction every six cycles)
// keeps the elements (ti + 32a, tc + 16b), a = 0 .. 3, b = 0 .. 7, of the tile (r) and of the inverse under
// construction (x, starting from the identity) in registers for the whole kernel, so every thread has work until the
// last column.  Column step j: the owners of column j publish it, and the owners of row j of x publish that row,
// through LDS (double buffered: one barrier per step); every thread then scales what it needs by 1 / l_jj itself and
// applies  r[i][c] -= l_ij l_cj  (j < c <= i)  and  x[i][c] -= l_ij x_jc  (c <= j < i): the right-looking
// factorisation and the forward elimination of L X = I in one sweep.  Entries a thread never needs (above the
// diagonal, rows past n) hold values that are never read.
template <typename T>
__global__ void __launch_bounds__(kPotrfThreads) potrf_tile_kernel(T *__restrict__ A, int n, int64_t lda,
                                                                    T *__restrict__ inv, int64_t ldinv,
                                                                    int *__restrict__ info, int info_base) {
    constexpr int N = kPotrfTile, QA = kPotrfOwnRows, QB = kPotrfOwnCols;
    __shared__ T colbuf[2][N], rowbuf[2][N];
    const int tid = threadIdx.x, ti = tid >> 4, tc = tid & 15;
    T r[QA][QB], x[QA][QB];
#pragma unroll
    for (int a = 0; a < QA; a++)
#pragma unroll
        for (int b = 0; b < QB; b++) {
            const int i = ti + 32 * a, c = tc + 16 * b;
            r[a][b] = (i < n && c <= i) ? A[i * lda + c] : T(0);
            x[a][b] = i == c ? T(1) : T(0);
        }
#pragma unroll
    for (int jb = 0; jb < QB; jb++) {
        const int ra = jb >> 1;                                 // the block of 32 rows that holds row j
        for (int jj = 0; jj < 16; jj++) {
            const int j = 16 * jb + jj, jr = 16 * (jb & 1) + jj;
            if (j >= n) break;                                  // the same for every thread
            T *cb = colbuf[j & 1], *rb = rowbuf[j & 1];
            if (tc == jj) {
#pragma unroll
                for (int a = ra; a < QA; a++) cb[ti + 32 * a] = r[a][jb];       // column j, rows 32 ra .. (the pivot among them)
            }
            if (ti == jr) {
#pragma unroll
                for (int b = 0; b <= jb; b++) rb[tc + 16 * b] = x[ra][b];       // row j of x, columns .. 16 jb + 15
            }
            __syncthreads();
            const T d = cb[j];
            T l, rl;
            if (d > T(0)) {
                pivot_root(d, l, rl);
            } else {
                if (tid == 0 && *info == 0) *info = info_base + j + 1;
                l = rl = __builtin_nan("");
            }
            // what this thread needs of column j and of row j of x, scaled by 1 / l_jj; only the blocks that hold row
            // and column j have entries on both sides of them (zeros there switch the updates off)
            T lrow[QA], lcol[QB], xrow[QB];
#pragma unroll
            for (int a = ra; a < QA; a++) lrow[a] = cb[ti + 32 * a] * rl;                    // l_ij for my rows
#pragma unroll
            for (int b = jb; b < QB; b++) lcol[b] = cb[tc + 16 * b] * rl;                    // l_cj for my columns
#pragma unroll
            for (int b = 0; b <= jb; b++) xrow[b] = rb[tc + 16 * b] * rl;                    // x_jc, scaled
            if (ti <= jr) lrow[ra] = T(0);
            if (tc <= jj) lcol[jb] = T(0);
            if (tc > jj) xrow[jb] = T(0);
            if (tc == jj) {
#pragma unroll
                for (int a = ra + 1; a < QA; a++) r[a][jb] = lrow[a];
                if (ti > jr) r[ra][jb] = lrow[ra];
                else if (ti == jr) r[ra][jb] = l;
            }
            if (ti == jr) {
#pragma unroll
                for (int b = 0; b <= jb; b++) x[ra][b] = xrow[b];
            }
#pragma unroll
            for (int a = ra; a < QA; a++) {
#pragma unroll
                for (int b = jb; b <= 2 * a + 1; b++) r[a][b] -= lrow[a] * lcol[b];
#pragma unroll
                for (int b = 0; b <= jb; b++) x[a][b] -= lrow[a] * xrow[b];
            }
        }
    }
#pragma unroll
    for (int a = 0; a < QA; a++)
#pragma unroll
        for (int b = 0; b < QB; b++) {
            const int i = ti + 32 * a, c = tc + 16 * b;
            if (i < n && c < n) {
                if (c <= i) A[i * lda + c] = r[a][b];
                inv[i * ldinv + c] = c <= i ? x[a][b] : T(0);
            }
        }
}

template <typename T>
int launch_potrf_tile(T *A, int64_t n, int64_t lda, T *inv, int64_t ldinv, int *info, int info_base, hipStream_t st) {
    if (n > kPotrfTile) return fail(FLK_EINVAL, "flk_potrf_tile: %lld rows (at most %d)", (long long)n, kPotrfTile);
    hipLaunchKernelGGL(potrf_tile_kernel<T>, dim3(1), dim3(kPotrfThreads), 0, st, A, (int)n, lda, inv, ldinv, info, info_base);
    FLK_LAUNCH_CHECK("potrf_tile_kernel");
    return FLK_OK;
}
template int launch_potrf_tile<float>(float *, int64_t, int64_t, float *, int64_t, int *, int, hipStream_t);
template int launch_potrf_tile<double>(double *, int64_t, int64_t, double *, int64_t, int *, int, hipStream_t);
int potrf_tile_rows(int) { return kPotrfTile; }

}  // namespace flk
