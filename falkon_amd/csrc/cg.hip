// The vector work of one conjugate-gradient iteration in one launch, on device-resident scalars.
//
// The reference's solver (falkon/optim/conjgrad.py:125-163) issues per iteration: a column-wise dot product, a
// division, two addcmul updates, a squared norm, a comparison whose result the host waits for, another division and
// a scaled add: eight small launches and one host synchronisation.  Here one workgroup per right-hand side does all
// of it; step lengths, residual norms and convergence flags never leave the device, so the host can enqueue
// iterations without waiting (and look at the flags only every few iterations).
#include "flk_common.h"

namespace flk {

constexpr int kCgThreads = 1024;

// Sum over the workgroup in a fixed order (lane tree inside a wave, then the 16 wave sums in order): the result
// does not depend on timing, so a solve is reproducible run to run.
__device__ __forceinline__ double block_sum(double x, double *lds) {
    for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();                       // lds may still be read from the previous reduction
    if (lane == 0) lds[wave] = x;
    __syncthreads();
    double s = 0.0;
    for (int w = 0; w < kCgThreads / 64; w++) s += lds[w];
    return s;
}

// state: [0] set once every column has converged (all later launches return at once), [1] iterations applied,
// [2 + p*t + c] convergence flag of column c written by the iteration of parity p, [2 + 2t + c] column c is frozen
// (differential convergence: a converged column is no longer updated).
// mode 0: whole iteration with Q = A P.  mode 1: first half only (step length, X += alpha P) before the residual
// is recomputed from scratch; mode 2: second half with Q = A X: R = B - Q, then as mode 0 from the residual norm on.
template <typename T>
__global__ void __launch_bounds__(kCgThreads) cg_update_kernel(int mode, T *__restrict__ X, T *__restrict__ R,
                                                               T *__restrict__ P, const T *__restrict__ Q,
                                                               const T *__restrict__ B, int64_t m, int t, int64_t rs,
                                                               int64_t cs, T *__restrict__ rsold, int *__restrict__ state,
                                                               int parity, double eps, double tol2, int differential) {
    __shared__ double lds[kCgThreads / 64];
    const int c = blockIdx.x;
    const int *prev = state + 2 + (parity ^ 1) * t;
    int *cur = state + 2 + parity * t;
    int *frozen = state + 2 + 2 * t;
    // every column converged in the previous iteration (or earlier): the solve is over, nothing is touched any more
    bool done = state[0] != 0;
    if (!done) {
        done = true;
        for (int i = 0; i < t; i++) done = done && prev[i] != 0;
    }
    if (done) {
        if (c == 0 && threadIdx.x == 0) state[0] = 1;
        if (threadIdx.x == 0 && mode != 1) cur[c] = 1;
        return;
    }
    if (differential && frozen[c]) {       // this column left the solve when it converged
        if (threadIdx.x == 0 && mode != 1) cur[c] = 1;
        return;
    }
    const int64_t off = (int64_t)c * cs;
    const double rs_old = (double)rsold[c];
    if (mode != 2) {
        double acc = 0.0;
        for (int64_t i = threadIdx.x; i < m; i += kCgThreads) acc += (double)P[i * rs + off] * (double)Q[i * rs + off];
        const double pap = block_sum(acc, lds);
        const T alpha = (T)(rs_old / (pap + eps));
        if (mode == 1) {
            for (int64_t i = threadIdx.x; i < m; i += kCgThreads) X[i * rs + off] += P[i * rs + off] * alpha;
            return;
        }
        acc = 0.0;
        for (int64_t i = threadIdx.x; i < m; i += kCgThreads) {
            const int64_t e = i * rs + off;
            X[e] += P[e] * alpha;
            const T r = R[e] - Q[e] * alpha;
            R[e] = r;
            acc += (double)r * (double)r;
        }
        const double rs_new = block_sum(acc, lds);
        const T beta = (T)(rs_new / (rs_old + eps));
        for (int64_t i = threadIdx.x; i < m; i += kCgThreads) {
            const int64_t e = i * rs + off;
            P[e] = P[e] * beta + R[e];
        }
        if (threadIdx.x == 0) {
            const int conv = rs_new < tol2;
            cur[c] = conv;
            if (differential && conv) frozen[c] = 1;
            rsold[c] = (T)rs_new;
            if (c == 0) state[1] += 1;
        }
        return;
    }
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < m; i += kCgThreads) {
        const int64_t e = i * rs + off;
        const T r = B[e] - Q[e];
        R[e] = r;
        acc += (double)r * (double)r;
    }
    const double rs_new = block_sum(acc, lds);
    const T beta = (T)(rs_new / (rs_old + eps));
    for (int64_t i = threadIdx.x; i < m; i += kCgThreads) {
        const int64_t e = i * rs + off;
        P[e] = P[e] * beta + R[e];
    }
    if (threadIdx.x == 0) {
        const int conv = rs_new < tol2;
        cur[c] = conv;
        if (differential && conv) frozen[c] = 1;
        rsold[c] = (T)rs_new;
        if (c == 0) state[1] += 1;
    }
}

template <typename T>
int launch_cg_update(int mode, T *X, T *R, T *P, const T *Q, const T *B, int64_t m, int64_t t, int64_t rs, int64_t cs,
                     T *rsold, int *state, int parity, double eps, double tol2, int differential, hipStream_t st) {
    if (m == 0 || t == 0) return FLK_OK;
    hipLaunchKernelGGL(cg_update_kernel<T>, dim3((unsigned)t), dim3(kCgThreads), 0, st, mode, X, R, P, Q, B, m, (int)t, rs,
                       cs, rsold, state, parity, eps, tol2, differential);
    FLK_LAUNCH_CHECK("cg_update_kernel");
    return FLK_OK;
}
template int launch_cg_update<float>(int, float *, float *, float *, const float *, const float *, int64_t, int64_t,
                                     int64_t, int64_t, float *, int *, int, double, double, int, hipStream_t);
template int launch_cg_update<double>(int, double *, double *, double *, const double *, const double *, int64_t, int64_t,
                                      int64_t, int64_t, double *, int *, int, double, double, int, hipStream_t);

}  // namespace flk
