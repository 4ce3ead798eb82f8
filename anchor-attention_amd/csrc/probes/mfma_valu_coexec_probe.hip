// Timing probe (not part of the library): how well do the matrix pipe and the vector ALU of a gfx950 SIMD overlap?
//
// Part 1: cycles per instruction of v_add_f32 and v_exp_f32 issued by one wave per SIMD.
// Part 2: work-groups of eight waves, i.e. two waves per SIMD (waves w and w+4 share SIMD w); each wave runs one of
//         several instruction streams made of independent 32x32x16 bf16 MFMAs and v_fmac_f32 on register operands.
//         Reported: nanoseconds per iteration (8 MFMAs and/or 48 vector instructions of one wave).
//
//   make -C anchor-attention_amd/csrc probes && anchor-attention_amd/csrc/_probes/mfma_valu_coexec_probe
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
#define CK(x)                                                                    \
  do {                                                                           \
    hipError_t e = (x);                                                          \
    if (e != hipSuccess) {                                                       \
      printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__);       \
      exit(1);                                                                   \
    }                                                                            \
  } while (0)

// ---- part 1 ------------------------------------------------------------------------------------
// MODE 0: 64 independent v_add_f32; 1: 64 v_add_f32 in one dependent chain; 2: 64 independent v_exp_f32; 3: dependent v_exp_f32;
// 4: 32 v_exp_f32 and 32 v_add_f32 alternating, all independent (does the transcendental unit run beside the ordinary one?)
template <int MODE>
__global__ void __launch_bounds__(256) valu_rate(int iters, float* out, float seed, long long* clk) {
  float x[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = seed + i + threadIdx.x;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
    if (MODE == 4) {
      float* y = x + 8;
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          asm volatile("v_exp_f32 %0, %0" : "+v"(x[i]));
          asm volatile("v_add_f32 %0, %0, %1" : "+v"(y[i]) : "v"(seed));
        }
    } else if (MODE == 0 || MODE == 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = MODE == 0 ? x[i] + seed : __builtin_amdgcn_exp2f(x[i]);
    } else {
#pragma unroll
      for (int r = 0; r < 64; ++r) {
        x[0] = MODE == 1 ? x[0] + seed : __builtin_amdgcn_exp2f(x[0]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (threadIdx.x == 0 && blockIdx.x == 7) clk[0] = clock64() - t0;
  float s = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += x[i];
  if (s == 12345.678f) out[0] = s;
}

template <int MODE>
static void run_rate(const char* name) {
  float* d;
  long long* dc;
  CK(hipMalloc(&d, 4));
  CK(hipMalloc(&dc, 16));
  const int iters = 100000;
  valu_rate<MODE><<<256, 256>>>(iters, d, 0.5f, dc);
  CK(hipDeviceSynchronize());
  long long hc;
  CK(hipMemcpy(&hc, dc, 8, hipMemcpyDeviceToHost));
  printf("%-62s %6.2f clk per instruction\n", name, (double)hc / iters / 64);
  CK(hipFree(d));
  CK(hipFree(dc));
}

// ---- part 2 ------------------------------------------------------------------------------------
#define MFMA(acc) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define VALU(x) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(x) : "v"(c1), "v"(c2))

// role: 0 idle, 1 MFMAs only (four independent accumulators), 2 vector only, 3 interleaved (1 MFMA + 6 vector),
//       4 bursts (8 MFMAs, then 48 vector), 5 interleaved (1 MFMA + 3 vector),
//       6 MFMAs only, one dependent chain (every MFMA accumulates onto the previous one's result), 7 two alternating chains
template <int ROLE_LO, int ROLE_HI>
__global__ void __launch_bounds__(512) coexec(int iters, float* out, float c1, float c2) {
  const int wave = threadIdx.x >> 6;
  const int role = wave < 4 ? ROLE_LO : ROLE_HI;
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(threadIdx.x * 0.001f);
    b[i] = (__bf16)(i * 0.01f);
  }
  floatx16 acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
  float x0 = threadIdx.x, x1 = 1, x2 = 2, x3 = 3, x4 = 4, x5 = 5;
  if (role == 1) {
    for (int it = 0; it < iters; ++it) { MFMA(acc0); MFMA(acc1); MFMA(acc2); MFMA(acc3); MFMA(acc0); MFMA(acc1); MFMA(acc2); MFMA(acc3); }
  } else if (role == 2) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 8; ++j) { VALU(x0); VALU(x1); VALU(x2); VALU(x3); VALU(x4); VALU(x5); }
    }
  } else if (role == 3) {
    for (int it = 0; it < iters; ++it) {
#define STEP6(acc) MFMA(acc); VALU(x0); VALU(x1); VALU(x2); VALU(x3); VALU(x4); VALU(x5);
      STEP6(acc0) STEP6(acc1) STEP6(acc2) STEP6(acc3) STEP6(acc0) STEP6(acc1) STEP6(acc2) STEP6(acc3)
    }
  } else if (role == 4) {
    for (int it = 0; it < iters; ++it) {
      MFMA(acc0); MFMA(acc1); MFMA(acc2); MFMA(acc3); MFMA(acc0); MFMA(acc1); MFMA(acc2); MFMA(acc3);
#pragma unroll
      for (int j = 0; j < 8; ++j) { VALU(x0); VALU(x1); VALU(x2); VALU(x3); VALU(x4); VALU(x5); }
    }
  } else if (role == 6) {
    for (int it = 0; it < iters; ++it) { MFMA(acc0); MFMA(acc0); MFMA(acc0); MFMA(acc0); MFMA(acc0); MFMA(acc0); MFMA(acc0); MFMA(acc0); }
  } else if (role == 7) {
    for (int it = 0; it < iters; ++it) { MFMA(acc0); MFMA(acc1); MFMA(acc0); MFMA(acc1); MFMA(acc0); MFMA(acc1); MFMA(acc0); MFMA(acc1); }
  } else if (role == 5) {
    for (int it = 0; it < iters; ++it) {
#define STEP3(acc) MFMA(acc); VALU(x0); VALU(x1); VALU(x2);
      STEP3(acc0) STEP3(acc1) STEP3(acc2) STEP3(acc3) STEP3(acc0) STEP3(acc1) STEP3(acc2) STEP3(acc3)
    }
  }
  float r = x0 + x1 + x2 + x3 + x4 + x5;
  for (int i = 0; i < 16; ++i) r += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  if (r == 12345.678f) out[0] = r;
}

template <int LO, int HI>
static void run_coexec(const char* name) {
  float* d;
  CK(hipMalloc(&d, 4));
  const int iters = 4000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  coexec<LO, HI><<<256, 512>>>(10, d, 0.5f, 0.25f);
  CK(hipEventRecord(e0));
  coexec<LO, HI><<<256, 512>>>(iters, d, 0.5f, 0.25f);
  CK(hipEventRecord(e1));
  CK(hipDeviceSynchronize());
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  printf("%-62s %8.1f ns per iteration\n", name, ms * 1e6 / iters);
  CK(hipFree(d));
}

int main() {
  printf("one wave per SIMD, cycles per vector instruction:\n");
  run_rate<0>("v_add_f32, independent");
  run_rate<1>("v_add_f32, one dependent chain");
  run_rate<2>("v_exp_f32, independent");
  run_rate<3>("v_exp_f32, one dependent chain");
  run_rate<4>("v_exp_f32 and v_add_f32 alternating (per instruction)");
  printf("per iteration and wave: MFMA stream = 8 MFMAs 32x32x16 bf16 (256 matrix-pipe cycles), vector stream = 48 v_fmac_f32\n");
  run_coexec<1, 0>("one wave per SIMD: MFMAs only");
  run_coexec<6, 0>("one wave per SIMD: MFMAs only, one dependent chain");
  run_coexec<7, 0>("one wave per SIMD: MFMAs only, two alternating chains");
  run_coexec<6, 6>("two waves per SIMD: both one dependent chain");
  run_coexec<2, 0>("one wave per SIMD: vector only");
  run_coexec<3, 0>("one wave per SIMD: interleaved 1 MFMA + 6 vector");
  run_coexec<4, 0>("one wave per SIMD: bursts 8 MFMAs then 48 vector");
  run_coexec<1, 2>("two waves per SIMD: one MFMAs only, one vector only");
  run_coexec<1, 1>("two waves per SIMD: both MFMAs only");
  run_coexec<2, 2>("two waves per SIMD: both vector only");
  run_coexec<3, 3>("two waves per SIMD: both interleaved 1 MFMA + 6 vector");
  run_coexec<4, 4>("two waves per SIMD: both bursts 8 MFMAs then 48 vector");
  run_coexec<5, 5>("two waves per SIMD: both interleaved 1 MFMA + 3 vector");
  return 0;
}
