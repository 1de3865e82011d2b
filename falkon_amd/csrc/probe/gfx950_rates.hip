// Instruction-rate probes for gfx950 (MI355X): the measurements the product kernels' design rests on.
//   part 1: fp32 v_exp / v_fma / v_add alone, interleaved, and beside fp32 MFMA from the same and from another wave
//           (do the vector ALU and the fp32 matrix instructions overlap?  They do not.)
//   part 2: the product kernel's instruction mix per 32x32 tile group, issued in phases (as the kernel does) against
//           software-pipelined with the previous tile's epilogue
//   part 3: fp64 vector instruction rates, fp64 MFMA, and their overlap
// Not part of the library.  Build and run:
//   hipcc --offload-arch=gfx950 -O3 -mllvm -amdgpu-mfma-vgpr-form=1 -o gfx950_rates falkon_amd/csrc/probe/gfx950_rates.hip
//   ./gfx950_rates
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
template <typename F> float timeit(F f, int reps = 5) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  f(); f(); CK(hipDeviceSynchronize());
  float best = 1e30f;
  for (int r = 0; r < reps; r++) { CK(hipEventRecord(e0)); f(); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); float ms; CK(hipEventElapsedTime(&ms, e0, e1)); if (ms < best) best = ms; }
  return best;
}

namespace p1 {

// mode bits per wave role: what the wave executes per iteration
//  E = 16 independent v_exp_f32, F = 16 independent v_fma_f32, A = 16 v_add_f32, M = NM mfma (4 chains)
template <int NE, int NF, int NA, int NM, bool INTERLEAVE>
__device__ __forceinline__ void body(float (&x)[16], float (&y)[16], floatx16 (&acc)[4], float a, float b, int iters) {
  for (int it = 0; it < iters; it++) {
    if constexpr (INTERLEAVE) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        if (i < NE) asm volatile("v_exp_f32 %0, %1" : "=v"(y[i]) : "v"(x[i]));
        if (i < NF) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(x[i]) : "v"(a), "v"(b));
        if (i < NA) asm volatile("v_add_f32 %0, %1, %0" : "+v"(x[i]) : "v"(b));
      }
    } else {
#pragma unroll
      for (int i = 0; i < NE; i++) asm volatile("v_exp_f32 %0, %1" : "=v"(y[i]) : "v"(x[i]));
#pragma unroll
      for (int i = 0; i < NF; i++) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(x[i]) : "v"(a), "v"(b));
#pragma unroll
      for (int i = 0; i < NA; i++) asm volatile("v_add_f32 %0, %1, %0" : "+v"(x[i]) : "v"(b));
    }
#pragma unroll
    for (int c = 0; c < NM; c++) acc[c & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[c & 3], 0, 0, 0);
  }
}

// all waves of the workgroup run the same stream
template <int NE, int NF, int NA, int NM, bool IL>
__global__ void __launch_bounds__(512) same(float *out, int iters) {
  float x[16], y[16]; floatx16 acc[4];
  for (int i = 0; i < 16; i++) { x[i] = -1e-3f * (threadIdx.x + i); y[i] = 0.f; }
  for (int c = 0; c < 4; c++) for (int r = 0; r < 16; r++) acc[c][r] = 0.f;
  float a = 0.999f + threadIdx.x * 1e-9f, b = 1e-5f;
  body<NE, NF, NA, NM, IL>(x, y, acc, a, b, iters);
  float s = 0; for (int i = 0; i < 16; i++) s += x[i] + y[i];
  for (int c = 0; c < 4; c++) for (int r = 0; r < 16; r++) s += acc[c][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// waves 0..3 (one per SIMD) run MFMA only, waves 4..7 run the VALU stream only
template <int NE, int NF, int NA, int NM>
__global__ void __launch_bounds__(512) split_roles(float *out, int iters) {
  float x[16], y[16]; floatx16 acc[4];
  for (int i = 0; i < 16; i++) { x[i] = -1e-3f * (threadIdx.x + i); y[i] = 0.f; }
  for (int c = 0; c < 4; c++) for (int r = 0; r < 16; r++) acc[c][r] = 0.f;
  float a = 0.999f + threadIdx.x * 1e-9f, b = 1e-5f;
  if (threadIdx.x < 256) body<0, 0, 0, NM, false>(x, y, acc, a, b, iters);
  else body<NE, NF, NA, 0, false>(x, y, acc, a, b, iters);
  float s = 0; for (int i = 0; i < 16; i++) s += x[i] + y[i];
  for (int c = 0; c < 4; c++) for (int r = 0; r < 16; r++) s += acc[c][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}


int run() {
  hipDeviceProp_t p; CK(hipGetDeviceProperties(&p, 0));
  const int cus = p.multiProcessorCount; const double clk = p.clockRate * 1e3;
  float *dout; CK(hipMalloc(&dout, (size_t)cus * 4 * 512 * 4));
  const int iters = 4000;
  printf("device %s CUs=%d clock=%.0f MHz; cycles per iteration per SIMD (one 512-thread WG per CU = 2 waves/SIMD unless said)\n", p.name, cus, clk / 1e6);
#define RUN_SAME(NE, NF, NA, NM, IL, WGS, THREADS, label) { float ms = timeit([&]{ same<NE,NF,NA,NM,IL><<<cus*(WGS),THREADS>>>(dout, iters); }); \
    printf("%-58s %8.1f cyc/iter/wave-slot (waves/SIMD=%d)\n", label, ms*1e-3*clk/iters, (WGS)*(THREADS)/256); }
  RUN_SAME(16,0,0,0,false,1,256,"16 exp, 1 wave/SIMD");
  RUN_SAME(16,0,0,0,false,1,512,"16 exp, 2 waves/SIMD");
  RUN_SAME(16,0,0,0,false,2,512,"16 exp, 4 waves/SIMD");
  RUN_SAME(0,16,0,0,false,1,256,"16 fma, 1 wave/SIMD");
  RUN_SAME(0,16,0,0,false,1,512,"16 fma, 2 waves/SIMD");
  RUN_SAME(0,16,0,0,false,2,512,"16 fma, 4 waves/SIMD");
  RUN_SAME(0,0,16,0,false,1,512,"16 add, 2 waves/SIMD");
  RUN_SAME(16,16,0,0,false,1,256,"16 exp then 16 fma, 1 wave/SIMD");
  RUN_SAME(16,16,0,0,true,1,256,"16 x (exp,fma) interleaved, 1 wave/SIMD");
  RUN_SAME(16,16,0,0,false,1,512,"16 exp then 16 fma, 2 waves/SIMD");
  RUN_SAME(16,16,0,0,true,1,512,"16 x (exp,fma) interleaved, 2 waves/SIMD");
  RUN_SAME(16,16,16,0,false,1,512,"16 exp, 16 fma, 16 add blocks, 2 waves/SIMD");
  RUN_SAME(16,16,16,0,true,1,512,"16 x (exp,fma,add) interleaved, 2 waves/SIMD");
  RUN_SAME(0,0,0,14,false,1,256,"14 mfma, 1 wave/SIMD");
  RUN_SAME(0,0,0,14,false,1,512,"14 mfma, 2 waves/SIMD");
  RUN_SAME(16,16,16,14,false,1,256,"14 mfma + 16 exp,fma,add blocks, 1 wave/SIMD");
  RUN_SAME(16,16,16,14,false,1,512,"14 mfma + 16 exp,fma,add blocks, 2 waves/SIMD");
  RUN_SAME(16,16,16,14,true,1,512,"14 mfma + 16 x (exp,fma,add) interleaved, 2 waves/SIMD");
  RUN_SAME(16,0,0,14,false,1,512,"14 mfma + 16 exp, 2 waves/SIMD");
  RUN_SAME(0,16,0,14,false,1,512,"14 mfma + 16 fma, 2 waves/SIMD");
#define RUN_SPLIT(NE, NF, NA, NM, label) { float ms = timeit([&]{ split_roles<NE,NF,NA,NM><<<cus,512>>>(dout, iters); }); \
    printf("%-58s %8.1f cyc/iter\n", label, ms*1e-3*clk/iters); }
  RUN_SPLIT(16,0,0,14,"roles: wave A 14 mfma | wave B 16 exp");
  RUN_SPLIT(0,16,0,14,"roles: wave A 14 mfma | wave B 16 fma");
  RUN_SPLIT(16,16,16,14,"roles: wave A 14 mfma | wave B 16 exp,fma,add");
  RUN_SPLIT(16,16,16,0,"roles: wave A idle | wave B 16 exp,fma,add");
  RUN_SPLIT(0,0,0,14,"roles: wave A 14 mfma | wave B idle");
  printf("done\n");
  return 0;
}

}  // namespace p1
#undef RUN
#undef RUN_SAME
#undef RUN_SPLIT
#undef MFMA
#undef EXP
#undef FMAC
#undef ADD

namespace p2 {
// tile's epilogue) instruction streams, 2 waves per SIMD, gfx950.
#define MFMA(acc) asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define EXP(y, x) asm volatile("v_exp_f32 %0, %1" : "=v"(y) : "v"(x))
#define FMAC(o, k, v) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(o) : "v"(k), "v"(v))
#define ADD(y, x, h) asm volatile("v_add_f32 %0, %1, %2" : "=v"(y) : "v"(x), "v"(h))

// MODE 0: phases, 4 chains interleaved (as the product kernel today), NADD adds per accumulator register
// MODE 1: per tile: 14 mfma of tile q interleaved with the epilogue (exp, fmac [, add]) of tile q-1; VPER valu groups after each mfma
template <int MODE, bool WITH_ADD, int DP>
__global__ void __launch_bounds__(512) stream(float *out, int iters) {
  floatx16 acc[4]; float o[4] = {0, 0, 0, 0}; float k;
  for (int c = 0; c < 4; c++) for (int r = 0; r < 16; r++) acc[c][r] = -1e-3f * (threadIdx.x + r);
  float a = 1e-3f * threadIdx.x, b = 1e-4f, hb = -0.5f, v = 0.25f;
  float hn[16]; for (int r = 0; r < 16; r++) hn[r] = -1e-2f * r;
  for (int it = 0; it < iters; it++) {
    if constexpr (MODE == 0) {
      if (WITH_ADD) {
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
          for (int r = 0; r < 16; r++) ADD(acc[q][r], hn[r], hb);
      }
#pragma unroll
      for (int s = 0; s < DP; s++)
#pragma unroll
        for (int q = 0; q < 4; q++) MFMA(acc[q]);
#pragma unroll
      for (int q = 0; q < 4; q++)
#pragma unroll
        for (int r = 0; r < 16; r++) { EXP(k, acc[q][r]); FMAC(o[q], k, v); }
    } else {
      // tile q's chain interleaved with tile q-1's epilogue (previous iteration's tile 3 for q = 0)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int p = (q + 3) & 3;
        // the epilogue of p reads acc[p]; afterwards acc[p] is re-initialised for its next chain
        int r = 0;
#pragma unroll
        for (int s = 0; s < DP; s++) {
          MFMA(acc[q]);
          // spread 16 register epilogues over DP mfma slots
          const int upto = (16 * (s + 1)) / DP;
#pragma unroll
          for (; r < upto; r++) {
            EXP(k, acc[p][r]); FMAC(o[p], k, v);
            if (WITH_ADD) ADD(acc[p][r], hn[r], hb);
          }
        }
      }
    }
  }
  float s = o[0] + o[1] + o[2] + o[3];
  for (int c = 0; c < 4; c++) for (int r = 0; r < 16; r++) s += acc[c][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}


int run() {
  hipDeviceProp_t p; CK(hipGetDeviceProperties(&p, 0));
  const int cus = p.multiProcessorCount; const double clk = p.clockRate * 1e3;
  float *dout; CK(hipMalloc(&dout, (size_t)cus * 4 * 512 * 4));
  const int iters = 3000;
#define RUN(MODE, ADDS, DP, WGS, label) { float ms = timeit([&]{ stream<MODE,ADDS,DP><<<cus*(WGS),512>>>(dout, iters); }); \
    double cyc = ms*1e-3*clk/iters/(2.0*(WGS)); \
    printf("%-64s %8.1f cycles per 4-tile unit per wave (mfma alone %d; waves/SIMD=%d)\n", label, cyc, DP*4*64, 2*(WGS)); }
  RUN(0,true,14,1,"d=28 phases: 64 add | 56 mfma | 64 (exp,fmac)");
  RUN(0,false,14,1,"d=28 phases: 56 mfma | 64 (exp,fmac)");
  RUN(1,true,14,1,"d=28 pipelined: mfma chain q with (exp,fmac,add) of q-1");
  RUN(1,false,14,1,"d=28 pipelined: mfma chain q with (exp,fmac) of q-1");
  RUN(0,false,5,1,"d=10 phases: 20 mfma | 64 (exp,fmac)");
  RUN(1,false,5,1,"d=10 pipelined");
  RUN(0,true,5,1,"d=10 phases with adds");
  RUN(1,true,5,1,"d=10 pipelined with adds");
  RUN(0,true,14,2,"d=28 phases with adds, 4 waves/SIMD");
  RUN(1,true,14,2,"d=28 pipelined with adds, 4 waves/SIMD");
  printf("done\n");
  return 0;
}

}  // namespace p2
#undef RUN
#undef RUN_SAME
#undef RUN_SPLIT
#undef MFMA
#undef EXP
#undef FMAC
#undef ADD

namespace p3 {

// KIND: 0 fma_f64, 1 add_f64, 2 mul_f64, 3 ldexp_f64, 4 max_f64, 5 int and/shift (b32), 6 ds_read_b64 random, 7 cvt_i32_f64
template <int KIND, int NV, int NM>
__global__ void __launch_bounds__(512) stream(double *out, int iters) {
  __shared__ double tab[2048];
  for (int i = threadIdx.x; i < 2048; i += blockDim.x) tab[i] = 1.0 + i * 1e-4;
  __syncthreads();
  double x[16]; doublex4 acc[4]; int n[16];
  for (int i = 0; i < 16; i++) { x[i] = -1e-3 * (threadIdx.x + i); n[i] = threadIdx.x * 37 + i * 101; }
  for (int c = 0; c < 4; c++) for (int r = 0; r < 4; r++) acc[c][r] = 0.0;
  double a = 0.999 + threadIdx.x * 1e-9, b = 1e-5;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      if (KIND == 0) asm volatile("v_fma_f64 %0, %1, %2, %0" : "+v"(x[i]) : "v"(a), "v"(b));
      if (KIND == 1) asm volatile("v_add_f64 %0, %1, %0" : "+v"(x[i]) : "v"(b));
      if (KIND == 2) asm volatile("v_mul_f64 %0, %1, %0" : "+v"(x[i]) : "v"(a));
      if (KIND == 3) asm volatile("v_ldexp_f64 %0, %0, %1" : "+v"(x[i]) : "v"(n[i] & 1));
      if (KIND == 4) asm volatile("v_max_f64 %0, %1, %0" : "+v"(x[i]) : "v"(b));
      if (KIND == 5) asm volatile("v_and_b32 %0, 2047, %0\n v_lshlrev_b32 %0, 3, %0" : "+v"(n[i]));
      if (KIND == 6) { double v; asm volatile("ds_read_b64 %0, %1\n s_waitcnt lgkmcnt(0)" : "=v"(v) : "v"((n[i] * 8) & 16376)); x[i] += v; n[i] += 613; }
      if (KIND == 7) asm volatile("v_cvt_i32_f64 %0, %1" : "=v"(n[i]) : "v"(x[i]));
    }
#pragma unroll
    for (int c = 0; c < NM; c++) acc[c & 3] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[c & 3], 0, 0, 0);
  }
  double s = 0; for (int i = 0; i < 16; i++) s += x[i] + n[i];
  for (int c = 0; c < 4; c++) for (int r = 0; r < 4; r++) s += acc[c][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}


int run() {
  hipDeviceProp_t p; CK(hipGetDeviceProperties(&p, 0));
  const int cus = p.multiProcessorCount; const double clk = p.clockRate * 1e3;
  double *dout; CK(hipMalloc(&dout, (size_t)cus * 4 * 512 * 8));
  const int iters = 3000;
#define RUN(KIND, NV, NM, WGS, label) { float ms = timeit([&]{ stream<KIND,NV,NM><<<cus*(WGS),512>>>(dout, iters); }); \
    double cyc = ms*1e-3*clk/iters; \
    printf("%-56s %8.1f cycles/iter/SIMD = %6.2f per VALU wave-instr, waves/SIMD=%d\n", label, cyc, NV ? (cyc - 0.0)/(NV*2.0*(WGS)) : 0.0, 2*(WGS)); }
  RUN(0,16,0,1,"16 v_fma_f64");
  RUN(0,16,0,2,"16 v_fma_f64 (4 waves)");
  RUN(1,16,0,1,"16 v_add_f64");
  RUN(2,16,0,1,"16 v_mul_f64");
  RUN(3,16,0,1,"16 v_ldexp_f64");
  RUN(4,16,0,1,"16 v_max_f64");
  RUN(5,16,0,1,"16 x (v_and_b32 + v_lshlrev_b32)  [2 instrs each]");
  RUN(7,16,0,1,"16 v_cvt_i32_f64");
  RUN(6,16,0,1,"16 ds_read_b64 scattered + wait + add_f64");
  RUN(0,0,8,1,"8 mfma_f64 16x16x4 (4 chains)");
  RUN(0,0,8,2,"8 mfma_f64 16x16x4 (4 chains), 4 waves");
  RUN(0,16,8,1,"8 mfma_f64 + 16 v_fma_f64");
  RUN(5,16,8,1,"8 mfma_f64 + 16 x (and, lshl) int ops");
  printf("done\n");
  return 0;
}

}  // namespace p3
#undef RUN
#undef RUN_SAME
#undef RUN_SPLIT
#undef MFMA
#undef EXP
#undef FMAC
#undef ADD

int main() {
  printf("---- part 1: fp32 vector instructions and fp32 MFMA ----\n"); p1::run();
  printf("---- part 2: phases against software pipelining ----\n"); p2::run();
  printf("---- part 3: fp64 ----\n"); p3::run();
  return 0;
}
