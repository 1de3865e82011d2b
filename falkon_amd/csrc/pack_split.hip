// Packing for the bf16x3 mode: X[n,d] (fp32, any unit-stride order) -> three bfloat16 planes of the scaled rows in
// MFMA operand order, with (1.0, half norm) in the last two features (see split_common.h).
#include "split_common.h"

namespace flk {

__device__ __forceinline__ unsigned bf16_rne(float x) {
    const unsigned u = __float_as_uint(x);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float bf16_value(unsigned b) { return __uint_as_float(b << 16); }

// x = hi + mid + lo, each piece the bfloat16 nearest to what the previous pieces leave (the subtractions are exact)
__device__ __forceinline__ void split3(float x, unsigned &hi, unsigned &mid, unsigned &lo) {
    hi = bf16_rne(x);
    const float r1 = x - bf16_value(hi);
    mid = bf16_rne(r1);
    lo = bf16_rne(r1 - bf16_value(mid));
}

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

// one thread per (block, k-step, lane): 8 features of one row
__global__ void __launch_bounds__(256) pack_split_kernel(const float *__restrict__ X, int64_t n, int64_t d, int64_t rs,
                                                         int64_t cs, const float *__restrict__ sigma, int64_t n_sigma,
                                                         double scale, uintx4 *__restrict__ P, int ks_count,
                                                         int64_t nblk) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int lane = (int)(gid & 63);
    const int64_t rest = gid >> 6;
    const int ks = (int)(rest % ks_count);
    const int64_t blk = rest / ks_count;
    if (blk >= nblk) return;
    const int64_t row = blk * 32 + (lane & 31);
    const int half = lane >> 5;
    const int64_t dpad = (int64_t)ks_count * 16;
    const bool live = row < n;
    // the thread that owns the last two features needs the row's half norm: sum of squares of the scaled,
    // fp32-rounded features in fp64 (the same values the other threads split)
    float hval = 0.f;
    if (live && ks == ks_count - 1 && half == 1) {
        double nrm = 0.0;
        for (int64_t k = 0; k < d; k++) {
            const float xs = (float)((double)X[row * rs + k * cs] * (scale / (double)sigma[n_sigma == 1 ? 0 : k]));
            nrm += (double)xs * (double)xs;
        }
        hval = (float)(-0.5 * nrm);
    }
    uintx4 out[3];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int64_t f = (int64_t)ks * 16 + half * 8 + e;
        float val = 0.f;
        if (live) {
            if (f < d) val = (float)((double)X[row * rs + f * cs] * (scale / (double)sigma[n_sigma == 1 ? 0 : f]));
            else if (f == dpad - 2) val = 1.0f;
            else if (f == dpad - 1) val = hval;
        }
        unsigned p[3];
        split3(val, p[0], p[1], p[2]);
#pragma unroll
        for (int c = 0; c < 3; c++) {
            if (e & 1) out[c][e >> 1] |= p[c] << 16;
            else out[c][e >> 1] = p[c];
        }
    }
    uintx4 *dst = P + ((blk * ks_count + ks) * 3) * 64 + lane;
    dst[0] = out[0];
    dst[64] = out[1];
    dst[128] = out[2];
}

int launch_pack_split(const float *X, int64_t n, int64_t d, int64_t rs, int64_t cs, const float *sigma, int64_t n_sigma,
                      double scale, void *packed, hipStream_t st) {
    const int64_t nblk = (n + 31) / 32;
    if (nblk == 0) return FLK_OK;
    const int64_t ks = split_ksteps(d);
    const int64_t threads = nblk * ks * 64;
    hipLaunchKernelGGL(pack_split_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, X, n, d, rs, cs,
                       sigma, n_sigma, scale, (uintx4 *)packed, (int)ks, nblk);
    FLK_LAUNCH_CHECK("pack_split_kernel");
    return FLK_OK;
}

}  // namespace flk
