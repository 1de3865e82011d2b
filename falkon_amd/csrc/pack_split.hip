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

// One workgroup per block of 32 rows walks over the k-steps two at a time: a 32 x 32 tile of scaled values goes
// through LDS, so that the read follows the unit stride of X (along a row, or along the rows of a column-major
// matrix) and every lane of the writing waves finds its 8 features in LDS.  The squares are summed per row on the
// way (in fp64, of the fp32-rounded values the pieces are made from), so the half norm is known when the last
// k-step, which carries it, is written.
__global__ void __launch_bounds__(256) pack_split_kernel(const float *__restrict__ X, int64_t n, int64_t d, int64_t rs,
                                                         int64_t cs, const float *__restrict__ sigma, int64_t n_sigma,
                                                         double scale, uintx4 *__restrict__ P, float *__restrict__ hnorm,
                                                         int ks_count) {
    constexpr int KT = 32;                       // features per LDS tile = two k-steps
    __shared__ float tile[32][KT + 1];
    __shared__ double nrm[32];
    const int tid = threadIdx.x;
    const int64_t blk = blockIdx.x;
    const int64_t row0 = blk * 32;
    const int64_t dpad = (int64_t)ks_count * 16;
    if (tid < 32) nrm[tid] = 0.0;
    const bool row_major = (cs == 1);
    for (int64_t k0 = 0; k0 < dpad; k0 += KT) {
        __syncthreads();
        for (int e = tid; e < 32 * KT; e += 256) {
            int r, k;
            if (row_major) { r = e / KT; k = e % KT; } else { k = e / 32; r = e % 32; }
            const int64_t row = row0 + r, f = k0 + k;
            float val = 0.f;
            if (row < n && f < d) val = (float)((double)X[row * rs + f * cs] * (scale / (double)sigma[n_sigma == 1 ? 0 : f]));
            tile[r][k] = val;
        }
        __syncthreads();
        if (tid < 32) {
            double acc = 0.0;
            const int kmax = (int)((d - k0) < KT ? (d - k0 > 0 ? d - k0 : 0) : KT);
            for (int k = 0; k < kmax; k++) { const double x = (double)tile[tid][k]; acc += x * x; }
            nrm[tid] += acc;
        }
        __syncthreads();
        // threads 0..127: k-step k0 / 16 + tid / 64, lane tid % 64 of the packed layout
        const int sub = tid >> 6, lane = tid & 63;
        const int ks = (int)(k0 / 16) + sub;
        if (tid < 128 && ks < ks_count) {
            const int r = lane & 31, half = lane >> 5;
            const bool live = row0 + r < n;
            uintx4 out[3];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int64_t f = (int64_t)ks * 16 + half * 8 + e;
                float val = tile[r][sub * 16 + half * 8 + e];
                if (live && f == dpad - 2) val = 1.0f;
                else if (live && f == dpad - 1) val = (float)(-0.5 * nrm[r]);
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
    }
    if (tid < 32) hnorm[row0 + tid] = (float)(-0.5 * nrm[tid]);   // zero on the padding rows
}

int launch_pack_split(const float *X, int64_t n, int64_t d, int64_t rs, int64_t cs, const float *sigma, int64_t n_sigma,
                      double scale, void *packed, hipStream_t st) {
    const int64_t nblk = (n + 31) / 32;
    if (nblk == 0) return FLK_OK;
    hipLaunchKernelGGL(pack_split_kernel, dim3((unsigned)nblk), dim3(256), 0, st, X, n, d, rs, cs, sigma, n_sigma, scale,
                       (uintx4 *)packed, (float *)((char *)packed + split_data_bytes(n, d)), (int)split_ksteps(d));
    FLK_LAUNCH_CHECK("pack_split_kernel");
    return FLK_OK;
}

}  // namespace flk
