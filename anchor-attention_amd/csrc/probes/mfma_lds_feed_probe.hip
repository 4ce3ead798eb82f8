// Timing probe (not part of the library): how fast can the two waves of a SIMD issue 32x32x16 bf16 MFMAs whose A operand
// comes from LDS, read the way the flash kernel reads its K tile (one ds_read_b128 per MFMA, rows of 256 bytes with
// XOR-swizzled 16-byte chunks) and its V tile (two transposing ds_read_b64_tr_b16 per MFMA)?  Work-groups of four waves
// with 64 KB of LDS, 512 of them; the hardware does not pair them evenly over the CUs, so the figure to read is "max":
// cycles per MFMA and wave of the work-groups that shared their SIMDs with another one for the whole run (bound: 64).
//
//   make -C anchor-attention_amd/csrc probes && anchor-attention_amd/csrc/_probes/mfma_lds_feed_probe
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;
typedef __attribute__((address_space(3))) bf16x8 lds_bf16x8;
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
#define F __builtin_amdgcn_sched_barrier(0)
// MODE 0: 16 MFMAs, register operands, 4 accumulators
// MODE 1: 16 MFMAs, one ds_read_b128 each (K style), two chains of 8
// MODE 2: 16 MFMAs, 8 ds_read_b128: every A operand feeds two MFMAs (two B operands, four chains of 4... 2 accs x 2)
// MODE 3: 16 MFMAs, A = two ds_read_b64_tr_b16 each (V style), 4 accumulators
// MODE 4: 16 MFMAs, V style, every A operand feeds two MFMAs (8 accumulators)
// MODE 5: one tile: 16 K-style + 16 V-style MFMAs
// MODE 6: two query sets: 32 K-style + 32 V-style MFMAs from the same 32 A operands
template <int MODE, int DIST>
__global__ void __launch_bounds__(256, 2) k(int iters, float* out, long long* clk) {
  __shared__ __attribute__((aligned(16))) char lds[65536];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 16384; i += 256) ((unsigned*)lds)[i] = 0x3c003c00u + (i * 2654435761u >> 20);
  __syncthreads();
  const long long t0 = clock64();
  bf16x8 b0, b1;
  for (int i = 0; i < 8; ++i) { b0[i] = (__bf16)(i * 0.01f + tid * 0.001f); b1[i] = (__bf16)(i * 0.02f - tid * 0.001f); }
  floatx16 acc[8] = {};
  const int c32 = lane & 31, half = lane >> 5;
  unsigned krd[8], vrd[4];
  const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  for (int ks = 0; ks < 8; ++ks) krd[ks] = base + c32 * 256 + (((2 * ks + half) ^ (c32 & 15)) << 4);
  {
    const int r0 = 4 * half + ((lane & 15) >> 2);
    const int y0 = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    for (int m = 0; m < 4; ++m) vrd[m] = base + 32768 + r0 * 256 + (((4 * m + y0) ^ (r0 << 1)) << 4) + 8 * (lane & 1);
  }
#define KRD(t) (*(const lds_bf16x8*)(uintptr_t)(krd[(t) & 7] + (unsigned)(8192 * ((t) >> 3))))
#define VSRC(i) (vrd[(i) & 3] + (unsigned)((32 * ((i) >> 3) + 16 * (((i) >> 2) & 1)) * 256))
#define VRD(i, dst) { shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(uintptr_t)(VSRC(i))); \
                      shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(uintptr_t)(VSRC(i) + 2048u)); \
                      shortx8 j = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); dst = *reinterpret_cast<bf16x8*>(&j); }
#define MF(c, a, b) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
#pragma unroll
      for (int t = 0; t < 16; ++t) { MF(acc[t & 3], b1, b0); F; }
    } else if (MODE == 1 || MODE == 2) {
      bf16x8 ka[16];
#pragma unroll
      for (int t = 0; t < DIST; ++t) ka[t] = KRD(t);
      F;
      constexpr int NA = MODE == 1 ? 16 : 8;
#pragma unroll
      for (int t = 0; t < NA; ++t) {
        if (t + DIST < NA) ka[t + DIST] = KRD(t + DIST);
        if (MODE == 1) { MF(acc[t >> 3], ka[t], b0); }
        else { MF(acc[0], ka[t], b0); F; MF(acc[1], ka[t], b1); }
        F;
      }
    } else if (MODE == 3 || MODE == 4) {
      bf16x8 va[16];
      constexpr int NA = MODE == 3 ? 16 : 8;
#pragma unroll
      for (int t = 0; t < DIST; ++t) VRD(t, va[t]);
      F;
#pragma unroll
      for (int t = 0; t < NA; ++t) {
        if (t + DIST < NA) VRD(t + DIST, va[t + DIST]);
        if (MODE == 3) { MF(acc[t & 3], va[t], b0); }
        else { MF(acc[t & 3], va[t], b0); F; MF(acc[4 + (t & 3)], va[t], b1); }
        F;
      }
    } else {
      bf16x8 op[32];
#pragma unroll
      for (int t = 0; t < DIST; ++t) op[t] = KRD(t);
      F;
#pragma unroll
      for (int t = 0; t < 32; ++t) {
        if (t + DIST < 16) op[t + DIST] = KRD(t + DIST);
        else if (t + DIST < 32) VRD(t + DIST - 16, op[t + DIST]);
        if (t < 16) {
          MF(acc[4 + (t >> 3)], op[t], b0);
          if (MODE == 6) { F; MF(acc[6 + (t >> 3)], op[t], b1); }
        } else {
          MF(acc[t & 3], op[t], b0);
          if (MODE == 6) { F; MF(acc[4 + (t & 3)], op[t], b1); }
        }
        F;
      }
    }
  }
  if (tid == 0) { clk[2 * blockIdx.x] = clock64() - t0; clk[2 * blockIdx.x + 1] = wall_clock64(); }
  float r = 0;
  for (int j = 0; j < 8; ++j)
    for (int i = 0; i < 16; ++i) r += acc[j][i];
  if (r == 12345.678f) out[0] = r;
}
template <int MODE, int DIST>
void run(const char* name, int n_mfma) {
  float* d; CK(hipMalloc(&d, 4)); long long* dc; CK(hipMalloc(&dc, 16 * 512));
  const int iters = 4000;
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  k<MODE, DIST><<<512, 256>>>(10, d, dc);
  CK(hipEventRecord(e0));
  k<MODE, DIST><<<512, 256>>>(iters, d, dc);
  CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  static long long h[1024]; CK(hipMemcpy(h, dc, 16 * 512, hipMemcpyDeviceToHost));
  long long mn = h[0], mx = h[0], wmin = h[1], wmax = h[1]; double hc = 0;
  for (int i = 0; i < 512; ++i) { hc += h[2 * i] / 512.0; if (h[2*i] < mn) mn = h[2*i]; if (h[2*i] > mx) mx = h[2*i]; if (h[2*i+1] < wmin) wmin = h[2*i+1]; if (h[2*i+1] > wmax) wmax = h[2*i+1]; }
  // two waves per SIMD: the pipe-bound figure is 2 x 32 clk per MFMA of one wave
  printf("%-64s dist %d: %6.1f clk per MFMA and wave (min %.1f max %.1f; pipe bound 64.0), %.2f ns, end spread %lld ticks\n", name, DIST, hc / iters / n_mfma, (double)mn / iters / n_mfma, (double)mx / iters / n_mfma, ms * 1e6 / iters / n_mfma, wmax - wmin);
  CK(hipFree(d)); CK(hipFree(dc));
}
int main() {
  run<0, 4>("register operands", 16);
  run<1, 4>("K style: one ds_read_b128 per MFMA", 16);
  run<1, 6>("K style: one ds_read_b128 per MFMA", 16);
  run<2, 4>("K style: one ds_read_b128 per TWO MFMAs", 16);
  run<3, 4>("V style: two ds_read_b64_tr_b16 per MFMA", 16);
  run<3, 6>("V style: two ds_read_b64_tr_b16 per MFMA", 16);
  run<4, 4>("V style: two ds_read_b64_tr_b16 per TWO MFMAs", 16);
  run<5, 4>("tile: 16 K-style + 16 V-style MFMAs", 32);
  run<5, 6>("tile: 16 K-style + 16 V-style MFMAs", 32);
  run<6, 4>("tile, two query sets: 64 MFMAs from 32 operands", 64);
  return 0;
}
