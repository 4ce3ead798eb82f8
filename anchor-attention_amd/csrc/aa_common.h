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

// ---- bf16 <-> float -------------------------------------------------------------------------
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// round-to-nearest-even float -> bf16, two at a time (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  floatx2 f = {a, b};
  bf16x2 h = __builtin_convertvector(f, bf16x2);
  return *reinterpret_cast<uint32_t*>(&h);
}
// float -> nearest bf16 -> float
__device__ __forceinline__ float rn16(float a) { return bf16_lo(pack_bf16(a, 0.f)); }

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
