// Timing probe (not part of the library): what does one global -> LDS direct load (global_load_lds_dwordx4, 64 lanes x
// 16 bytes = 1 KB) cost the wave that issues it, and how many bytes per cycle does a CU take in this way?
//
// One work-group per CU; each wave issues 64 loads of 1 KB from a buffer that fits the L2 (every wave walks its own
// 64 KB), then waits for all of them.  Variants: the LDS destination (M0) rewritten before every load or left alone;
// ordinary loads into registers for comparison; 1, 4 or 8 waves per work-group.  Reported per variant: cycles between the
// first issue and the last issue (what the issuing wave loses), cycles until all data has arrived, and the bytes per
// cycle the CU received.
//
//   make -C anchor-attention_amd/csrc probes && anchor-attention_amd/csrc/_probes/lds_dma_issue_probe
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#define CK(x)                                                                    \
  do {                                                                           \
    hipError_t e = (x);                                                          \
    if (e != hipSuccess) {                                                       \
      printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__);       \
      exit(1);                                                                   \
    }                                                                            \
  } while (0)

typedef __attribute__((address_space(3))) char lds_char;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// MODE 0: LDS-direct loads, M0 written once; 1: M0 rewritten before every load; 2: ordinary 16-byte loads into registers
template <int MODE, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) issue_probe(const char* src, long long* out, unsigned* sink, int reps) {
  __shared__ __attribute__((aligned(16))) char buf[WAVES][8 * 1024];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const unsigned lds0 = (unsigned)(uintptr_t)(lds_char*)buf[wave];
  const char* base = src + ((size_t)(blockIdx.x * WAVES + wave) % 256) * 65536;  // 16 MB in all: stays in the L2s
  long long t_issue = 0, t_done = 0;
  u32x4 acc = {0, 0, 0, 0};
  for (int r = 0; r < reps; ++r) {
    __syncthreads();
    const long long t0 = clock64();
#pragma unroll
    for (int i = 0; i < 64; ++i) {
      const unsigned off = (unsigned)(i * 1024 + lane * 16);
      if (MODE == 2) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(base + off);
        acc ^= v;
      } else {
        const unsigned dst = MODE == 1 ? lds0 + (unsigned)((i & 7) * 1024) : lds0;
        asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "{m0}"(dst), "v"(off), "s"(base) : "memory");
      }
    }
    const long long t1 = clock64();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const long long t2 = clock64();
    if (r > 0) { t_issue += t1 - t0; t_done += t2 - t0; }
  }
  if (lane == 0 && blockIdx.x == 17) { out[2 * wave] = t_issue / (reps - 1); out[2 * wave + 1] = t_done / (reps - 1); }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345u) sink[0] = buf[wave][lane];
}

// Second question: what do the arriving loads cost the LDS?  Waves 0-3 (one per SIMD) read LDS back to back (16 bytes per
// lane, rows of 256 bytes with the chunks swizzled: conflict-free, 4 cycles per instruction when alone); waves 4-7 issue
// global -> LDS loads (WITH_DMA) or nothing.  Reported: cycles per LDS read of a reading wave.
template <bool WITH_DMA>
__global__ void __launch_bounds__(512) contention_probe(const char* src, long long* out, unsigned* sink, int reps) {
  __shared__ __attribute__((aligned(16))) char rd[32 * 1024];
  __shared__ __attribute__((aligned(16))) char wr[4][8 * 1024];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 32 * 1024 / 4; i += 512) reinterpret_cast<unsigned*>(rd)[i] = i;
  __syncthreads();
  long long t = 0;
  u32x4 acc = {0, 0, 0, 0};
  if (wave < 4) {
    const int c32 = lane & 31, half = lane >> 5;
    const unsigned a0 = (unsigned)(uintptr_t)(lds_char*)rd + c32 * 256 + (((half) ^ (c32 & 15)) << 4);
    for (int r = 0; r < reps; ++r) {
      const long long t0 = clock64();
#pragma unroll 1
      for (int j = 0; j < 32; ++j) {
        u32x4 v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
          asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v[i]) : "v"(a0), "n"((i % 4) * 8192 + (i / 4) * 32));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < 16; ++i) acc ^= v[i];
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (r > 0) t += clock64() - t0;
    }
    if (lane == 0 && blockIdx.x == 17) out[wave] = t / (reps - 1);
  } else if (WITH_DMA) {
    const unsigned lds0 = (unsigned)(uintptr_t)(lds_char*)wr[wave - 4];
    const char* base = src + ((size_t)(blockIdx.x * 4 + wave - 4) % 256) * 65536;
    for (int r = 0; r < reps; ++r) {
#pragma unroll 1
      for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const unsigned off = (unsigned)((j * 8 + i) * 1024 + lane * 16);
          asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "{m0}"(lds0 + (unsigned)(i * 1024)), "v"(off), "s"(base) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
    }
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345u) sink[0] = rd[lane] + wr[0][lane];
}

template <bool WITH_DMA>
static void run_contention(const char* name, const char* src, long long* d_out, unsigned* d_sink) {
  contention_probe<WITH_DMA><<<256, 512>>>(src, d_out, d_sink, 20);
  CK(hipDeviceSynchronize());
  long long h[4];
  CK(hipMemcpy(h, d_out, sizeof(h), hipMemcpyDeviceToHost));
  long long worst = 0;
  for (int w = 0; w < 4; ++w) worst = h[w] > worst ? h[w] : worst;
  printf("%-58s %6.2f clk per ds_read_b128 of a reading wave (512 reads of 1 KB)\n", name, worst / 512.0);
}

template <int MODE, int WAVES>
static void run(const char* name, const char* src, long long* d_out, unsigned* d_sink) {
  issue_probe<MODE, WAVES><<<256, 64 * WAVES>>>(src, d_out, d_sink, 20);
  CK(hipDeviceSynchronize());
  long long h[16];
  CK(hipMemcpy(h, d_out, sizeof(h), hipMemcpyDeviceToHost));
  long long issue = 0, done = 0;
  for (int w = 0; w < WAVES; ++w) { issue = h[2 * w] > issue ? h[2 * w] : issue; done = h[2 * w + 1] > done ? h[2 * w + 1] : done; }
  printf("%-58s %d waves: %6.1f clk per load until issued, %6.1f until arrived, %5.1f B/clk per CU\n", name, WAVES, issue / 64.0,
         done / 64.0, WAVES * 65536.0 / done);
}

int main() {
  char* src;
  long long* d_out;
  unsigned* d_sink;
  CK(hipMalloc(&src, 16 << 20));
  CK(hipMemset(src, 1, 16 << 20));
  CK(hipMalloc(&d_out, 256));
  CK(hipMalloc(&d_sink, 4));
  run<0, 1>("global_load_lds_dwordx4, M0 left alone", src, d_out, d_sink);
  run<1, 1>("global_load_lds_dwordx4, M0 rewritten per load", src, d_out, d_sink);
  run<2, 1>("global_load_dwordx4 into registers", src, d_out, d_sink);
  run<0, 4>("global_load_lds_dwordx4, M0 left alone", src, d_out, d_sink);
  run<1, 4>("global_load_lds_dwordx4, M0 rewritten per load", src, d_out, d_sink);
  run<2, 4>("global_load_dwordx4 into registers", src, d_out, d_sink);
  run<0, 8>("global_load_lds_dwordx4, M0 left alone", src, d_out, d_sink);
  run<1, 8>("global_load_lds_dwordx4, M0 rewritten per load", src, d_out, d_sink);
  run<2, 8>("global_load_dwordx4 into registers", src, d_out, d_sink);
  run_contention<false>("four waves reading LDS, nothing else", src, d_out, d_sink);
  run_contention<true>("four waves reading LDS, four waves loading global -> LDS", src, d_out, d_sink);
  return 0;
}
