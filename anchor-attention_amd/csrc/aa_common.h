// Shared device/host helpers for the AnchorAttention gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.44269504f;  // the literal the operator's definition multiplies by

// ---- 16-bit element types --------------------------------------------------------------------
// The operator takes bf16 tensors (what its callers use) or fp16 tensors (which the definition also admits: every
// ".to(dtype)" of it then rounds to fp16).  A kernel is written once against one of these two descriptions of the
// element type: unpacking a pair from a dword, round-to-nearest-even packing, and the matching MFMA.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

struct Bf16 {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ float lo(uint32_t u) { return __uint_as_float(u << 16); }
  static __device__ __forceinline__ float hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
  static __device__ __forceinline__ float from16(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
  // round-to-nearest-even float -> bf16, two at a time (v_cvt_pk_bf16_f32 on gfx950)
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    floatx2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    return *reinterpret_cast<uint32_t*>(&h);
  }
  static __device__ __forceinline__ float round(float a) { return lo(pack(a, 0.f)); }  // float -> nearest bf16 -> float
  // (a * b).to(bf16) as the operator's definition compiles: a float32 product, then the rounding
  static __device__ __forceinline__ float round_product(float a, float b) { return round(a * b); }
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

struct F16 {
  typedef f16x8 vec8;
  static __device__ __forceinline__ float lo(uint32_t u) { return (float)(*reinterpret_cast<f16x2*>(&u))[0]; }
  static __device__ __forceinline__ float hi(uint32_t u) { return (float)(*reinterpret_cast<f16x2*>(&u))[1]; }
  static __device__ __forceinline__ float from16(uint16_t h) { return lo((uint32_t)h); }
  // round-to-nearest-even float -> fp16, two at a time (v_cvt_pk_f16_f32 on gfx950); overflow gives infinity
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    floatx2 f = {a, b};
    f16x2 h = __builtin_convertvector(f, f16x2);
    return *reinterpret_cast<uint32_t*>(&h);
  }
  static __device__ __forceinline__ float round(float a) { return lo(pack(a, 0.f)); }
  // (a * b).to(fp16) as the operator's definition compiles: ONE rounding of the exact product (the multiply and the
  // cast become a single mixed-precision instruction).  Written out so that it does not depend on what this compiler
  // fuses: the product is exact in double; it is brought to float32 with round-to-odd, after which the
  // round-to-nearest-even to fp16 is the correct rounding of the exact value.
  static __device__ __forceinline__ float round_product(float a, float b) {
    const double d = (double)a * (double)b;
    float f = (float)d;
    const double back = (double)f;
    if (back != d) {  // inexact (also: overflow to infinity)
      uint32_t u = __float_as_uint(f);
      if ((u & 1u) == 0u) {  // even: the odd neighbour on d's side
        const bool negative = (u >> 31) != 0u, larger = d > back;
        u = (negative != larger) ? u + 1u : u - 1u;
      }
      f = __uint_as_float(u);
    }
    return round(f);
  }
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Work-group barrier for LDS hand-over only: waits for this wave's LDS traffic, then synchronises.
// Unlike __syncthreads() it does not wait for outstanding global loads, so prefetches issued before
// the barrier stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// value held by the lane 32 positions away (the two halves of a wave share MFMA columns)
__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// max of a value and its counterpart 32 lanes away, without a trip through LDS: v_permlane32_swap hands every
// lane the lower half's value (result 0) and the upper half's value (result 1)
__device__ __forceinline__ float max_with_other_half(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// ---- geometry --------------------------------------------------------------------------------
// Index lists are packed per (batch, query head): big block bb can select at most
// cap(bb) = bb*S - 2*bs keys (candidates are [bs, bb*S - bs)), and its list starts at
// tri(bb) = sum_{x<bb} cap(x) entries into the head's slab.
__host__ __device__ inline int64_t coords_tri(int64_t bb, int64_t S, int64_t bs) {
  return bb <= 1 ? 0 : S * (bb - 1) * bb / 2 - 2 * bs * (bb - 1);
}

// XCD-aware work-group renumbering.  Consecutive hardware work-group ids go round-robin over the 8 XCDs (each
// with its own L2).  The work consists of `n_units` units (a KV head of one batch element) of `per_unit`
// work-groups each, ordered heaviest first inside a unit; work-groups of one unit read the same K/V rows or pooled
// queries.  Returns the logical index unit * per_unit + idx such that
//   n_units % 8 == 0 : every XCD owns n_units / 8 whole units, in order;
//   8 % n_units == 0 : s = 8 / n_units XCDs share a unit and take its rows alternately (row = idx / inner, the
//                      `inner` work-groups of a row stay together), so that each gets the same mix of heavy and light;
//   otherwise        : the hardware order is kept.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t wg, uint32_t n_units, uint32_t per_unit, uint32_t inner) {
  const uint32_t total = n_units * per_unit;
  const uint32_t xcd = wg % 8u, k = wg / 8u;
  if (total % 8u != 0u) return wg;
  if (n_units % 8u == 0u) return xcd * (total / 8u) + k;
  if (8u % n_units == 0u) {
    const uint32_t s = 8u / n_units;
    if ((per_unit / inner) % s == 0u) return (xcd / s) * per_unit + ((k / inner) * s + xcd % s) * inner + k % inner;
  }
  return wg;
}

// ---- error plumbing (host) -------------------------------------------------------------------
enum Status : int {
  kOk = 0,
  kBadArgument = 1,   // null pointer, non-positive size, inconsistent head counts
  kUnsupported = 2,   // a size the kernels are not written for (head_dim, block_size, step)
  kMisaligned = 3,    // pointer or stride breaks the 16-byte row alignment the loads assume
  kLaunchFailed = 4,  // the HIP runtime refused the launch
};
void set_error(const char* fmt, ...);

}  // namespace aa
