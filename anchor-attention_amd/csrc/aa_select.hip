// Stage 2 of the AnchorAttention prefill path on gfx950: pooling, score-and-threshold, compaction.
//
//  pool     qbar = bf16(mean of 128 raw query rows), abar = bf16(mean of 128 anchors); float32 sums in
//           ascending row order so the result is reproducible bit for bit.
//  scores   K-stationary: one work-group per (batch, KV head, 512 keys); each of its four waves keeps a
//           128-key tile in registers as the MFMA B operand, and the pooled query rows of EVERY query
//           head of the KV group and EVERY later big block stream past them (A operand, 32 pooled rows
//           per MFMA, staged once per work-group in LDS).  Each K row is thus read once per KV head
//           instead of once per (query head, big block).
//           In the 32x32 accumulator a lane holds one key column; OR-ing its registers over the pooled
//           rows of a big block and a wave ballot give a 32-bit key mask per (q head, big block, key
//           block) with no LDS and no atomics.
//  thresholds  the as-specified test "float(bf16(raw * scale)) + theta >= anchor" is monotone in the raw
//           float32 dot product, so for every pooled row there is one float32 number x* with
//           "test passes  <=>  raw >= x*".  A tiny kernel finds x* per pooled row by bisection over
//           the ordered float32 bit patterns, evaluating the test exactly as written; the score
//           kernel's epilogue is then a single compare per element.
//  compact  one wave per (batch, q head, big block) turns that big block's mask row into an ascending
//           index list with popcounts and a wave prefix sum.
#include "aa_common.h"
#include "aa_kernels.h"

namespace aa {

// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(64) pool_kernel(const PoolArgs p) {
  const int lane = threadIdx.x;
  const int c = lane & 15;
  const int n_pr = p.n_ctx / p.block_size;
  const int pr = 4 * blockIdx.x + (lane >> 4);
  const int h = blockIdx.y, b = blockIdx.z;
  if (pr >= n_pr) return;
  const int bs = p.block_size;
  const __bf16* base = p.q + b * p.q_sb + h * p.q_sh + (int64_t)pr * bs * p.q_sn + 8 * c;
  const int64_t bh = (int64_t)b * p.n_q_heads + h;
  const float* mb = p.M + bh * p.n_ctx + (int64_t)pr * bs;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float am = 0.f;
#pragma unroll 8
  for (int t = 0; t < bs; ++t) {
    const uint4 raw = *reinterpret_cast<const uint4*>(base + (int64_t)t * p.q_sn);
    acc[0] += bf16_lo(raw.x); acc[1] += bf16_hi(raw.x);
    acc[2] += bf16_lo(raw.y); acc[3] += bf16_hi(raw.y);
    acc[4] += bf16_lo(raw.z); acc[5] += bf16_hi(raw.z);
    acc[6] += bf16_lo(raw.w); acc[7] += bf16_hi(raw.w);
    if (c == 0) am += mb[t];
  }
  const float d = (float)bs;
  uint4 o;
  o.x = pack_bf16(acc[0] / d, acc[1] / d);
  o.y = pack_bf16(acc[2] / d, acc[3] / d);
  o.z = pack_bf16(acc[4] / d, acc[5] / d);
  o.w = pack_bf16(acc[6] / d, acc[7] / d);
  *reinterpret_cast<uint4*>(p.qbar + (bh * n_pr + pr) * 128 + 8 * c) = o;
  if (c == 0) {
    const uint32_t w = pack_bf16(am / d, 0.f);
    reinterpret_cast<uint16_t*>(p.abar)[bh * n_pr + pr] = (uint16_t)(w & 0xffffu);
  }
}

hipError_t launch_pool(const PoolArgs& a, hipStream_t stream) {
  const int n_pr = a.n_ctx / a.block_size;
  hipLaunchKernelGGL(pool_kernel, dim3((n_pr + 3) / 4, a.n_q_heads, a.batch), dim3(64), 0, stream, a);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Smallest float32 x with  float(bf16(x * scale2)) + theta >= anchor  (NaN if there is none).
__device__ __forceinline__ bool select_test(const float x, const float scale2, const float theta, const float anchor) {
  const float sc = rn16(x * scale2);  // float32 product, then bf16
  return (sc + theta) >= anchor;      // float32 add and compare, non-strict
}
__device__ __forceinline__ float ordered_to_float(const uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);  // monotone bijection uint32 -> float32
}

__global__ void __launch_bounds__(256) select_threshold_kernel(const __bf16* __restrict__ abar, float* __restrict__ thr, const int n,
                                                                const float scale2, const float theta) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float anchor = bf16_lo(reinterpret_cast<const uint16_t*>(abar)[i]);
  // ordered keys: 0x007fffff <-> -inf, 0xff800000 <-> +inf (NaNs lie outside that range)
  uint32_t lo = 0x007fffffu, hi = 0xff800000u;
  float out;
  if (!select_test(ordered_to_float(hi), scale2, theta, anchor)) {
    out = __uint_as_float(0x7fc00000u);  // no float passes: NaN compares false with everything
  } else {
    while (lo < hi) {  // invariant: test(hi) is true
      const uint32_t mid = lo + ((hi - lo) >> 1);
      if (select_test(ordered_to_float(mid), scale2, theta, anchor)) hi = mid; else lo = mid + 1;
    }
    out = ordered_to_float(hi);
  }
  thr[i] = out;
}

hipError_t launch_select_thresholds(const SelectArgs& a, hipStream_t stream) {
  const int n = a.batch * a.n_q_heads * (a.n_ctx / a.block_size);
  hipLaunchKernelGGL(select_threshold_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, a.abar, a.thr, n, a.scale2, a.theta_log2);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// STEP = pooled rows per big block (16 or 32); 32 / STEP (head, big block) items share one MFMA.
// Work-group = 4 waves = 512 keys: wave w keeps key tile 4*T + w in registers (MFMA B operand) and all
// four waves multiply the same stream of pooled-query groups, which is staged once per work-group in
// LDS (double-buffered, one barrier per group) together with the groups' thresholds.
constexpr int kARowStride = 136;  // bf16 per staged pooled-query row: 272 B, conflict-free for row-per-lane 16-byte reads

constexpr int kKB = 2;  // 32-key blocks a wave keeps in registers (2: 64 keys, 64 VGPRs -> two work-groups per CU)

template <int STEP>
__global__ void __launch_bounds__(256, 2) select_scores_kernel(const SelectArgs p) {
  constexpr int kItems = 32 / STEP;
  constexpr int kWavesPerTile = 4 / kKB;      // waves that share one 128-key tile
  constexpr int kTilesPerWg = 4 / kWavesPerTile;
  __shared__ __attribute__((aligned(16))) __bf16 a_lds[2][32 * kARowStride];
  __shared__ __attribute__((aligned(16))) float thr_lds[2][32];

  // Work-groups are renumbered so that each XCD owns a contiguous range ordered (batch, KV head, super-tile): the
  // pooled queries a work-group streams are those of its KV head's query heads (1 MiB per KV head at 128k tokens),
  // which then stay in that XCD's L2 instead of every XCD cycling through all heads' pooled queries.
  const int n_bb = p.n_ctx / p.big_block;
  const int n_t = p.n_ctx / 128;
  const int n_super = n_t / kTilesPerWg;
  uint32_t vid = xcd_remap(blockIdx.x, p.batch * p.n_kv_heads, n_super, 1);
  const int T = vid % n_super;  // key super-tile (kTilesPerWg * 128 keys); ascending = heaviest first
  vid /= n_super;
  const int kvh = vid % p.n_kv_heads, b = vid / p.n_kv_heads;
  const int n_pr = n_t;  // pooled rows per head (block_size == 128)
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, c32 = lane & 31;

  // key tile t is a candidate for big block bb iff tile_lo <= t <= STEP*bb - tile_slack,
  // i.e. t >= tile_lo and bb >= (t + tile_slack + STEP - 1) / STEP
  const int tw = kTilesPerWg * T + wave / kWavesPerTile;          // this wave's 128-key tile
  const int kb0 = kKB * (wave % kWavesPerTile);                   // its first 32-key block inside the tile
  const int bb_min_w = tw < p.tile_lo ? n_bb : (tw + p.tile_slack + STEP - 1) / STEP;
  if (kTilesPerWg * T + kTilesPerWg - 1 < p.tile_lo) return;      // no tile of the work-group is ever a candidate
  const int t_first = max(p.tile_lo, kTilesPerWg * T);            // first candidate tile of the work-group
  const int bb_lo = (t_first + p.tile_slack + STEP - 1) / STEP;   // smallest big block any wave needs
  if (bb_lo >= n_bb) return;
  const int group = p.n_q_heads / p.n_kv_heads;
  const int n_items = group * (n_bb - bb_lo);
  const int n_groups = (n_items + kItems - 1) / kItems;

  const __bf16* kp = p.k + b * p.k_sb + kvh * p.k_sh;
  bf16x8 kreg[kKB][8];
#pragma unroll
  for (int kb = 0; kb < kKB; ++kb) {
    const __bf16* row = kp + (int64_t)(tw * 128 + 32 * (kb0 + kb) + c32) * p.k_sn + 8 * half;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) kreg[kb][ks] = *reinterpret_cast<const bf16x8*>(row + 16 * ks);
  }

  // staging: thread t carries 32 bytes (chunks 2*(t&7), 2*(t&7)+1) of pooled row t>>3 of the group; row r of a
  // group is pooled row (r % STEP) of item grp*kItems + r/STEP; threads 0..31 also carry the row's threshold
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  u32x4 st0, st1;
  float st_thr = 0.f;
  auto stage_load = [&](const int grp) {
    const int r = tid >> 3;
    const int item = min(grp * kItems + r / STEP, n_items - 1);
    const int64_t prow = ((int64_t)b * p.n_q_heads + kvh * group + item % group) * n_pr + (bb_lo + item / group) * STEP + r % STEP;
    const __bf16* src = p.qbar + prow * 128 + 16 * (tid & 7);
    st0 = *reinterpret_cast<const u32x4*>(src);
    st1 = *reinterpret_cast<const u32x4*>(src + 8);
    if (tid < 32) {
      const int item2 = min(grp * kItems + tid / STEP, n_items - 1);
      st_thr = p.thr[((int64_t)b * p.n_q_heads + kvh * group + item2 % group) * n_pr + (bb_lo + item2 / group) * STEP + tid % STEP];
    }
  };
  auto stage_store = [&](const int buf) {
    __bf16* dst = &a_lds[buf][(tid >> 3) * kARowStride + 16 * (tid & 7)];
    *reinterpret_cast<u32x4*>(dst) = st0;
    *reinterpret_cast<u32x4*>(dst + 8) = st1;
    if (tid < 32) thr_lds[buf][tid] = st_thr;
  };

  stage_load(0);
  stage_store(0);
  __syncthreads();

  for (int grp = 0; grp < n_groups; ++grp) {
    const int buf = grp & 1;
    if (grp + 1 < n_groups) stage_load(grp + 1);

    // does this wave's key tile belong to the candidate range of either item of the group?
    bool item_ok[kItems];
    bool any_ok = false;
#pragma unroll
    for (int it = 0; it < kItems; ++it) {
      const int item = grp * kItems + it;
      item_ok[it] = item < n_items && (bb_lo + item / group) >= bb_min_w;
      any_ok |= item_ok[it];
    }
    if (any_ok) {
      bf16x8 a[8];
      const __bf16* arow = &a_lds[buf][c32 * kARowStride + 8 * half];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) a[ks] = *reinterpret_cast<const bf16x8*>(arow + 16 * ks);
      // raw-score thresholds of the accumulator rows this lane holds: row i = 8*(r/4) + 4*half + r%4
      float thr[16];
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const floatx4 w = *reinterpret_cast<const floatx4*>(&thr_lds[buf][8 * rq + 4 * half]);
        thr[4 * rq + 0] = w[0]; thr[4 * rq + 1] = w[1];
        thr[4 * rq + 2] = w[2]; thr[4 * rq + 3] = w[3];
      }
      uint32_t words[kItems][kKB];
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb) {
        const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        floatx16 c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], kreg[kb][0], zero, 0, 0, 0);
#pragma unroll
        for (int ks = 1; ks < 8; ++ks) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks], kreg[kb][ks], c, 0, 0, 0);
        bool hit[kItems];
#pragma unroll
        for (int it = 0; it < kItems; ++it) hit[it] = false;
#pragma unroll
        for (int r = 0; r < 16; ++r) hit[(8 * (r >> 2)) / STEP] |= (c[r] >= thr[r]);  // rows 0..15 -> item 0, 16..31 -> item 1 (STEP 16)
#pragma unroll
        for (int it = 0; it < kItems; ++it) {
          const uint64_t m = __ballot(hit[it]);
          words[it][kb] = (uint32_t)m | (uint32_t)(m >> 32);  // both halves of the wave hold the same keys
        }
      }
      if (lane == 0) {
#pragma unroll
        for (int it = 0; it < kItems; ++it) {
          if (item_ok[it]) {
            const int item = grp * kItems + it;
            const int hq = kvh * group + item % group;
            const int bb = bb_lo + item / group;
            uint32_t* dst = p.mask + ((((int64_t)b * p.n_q_heads + hq) * n_bb + bb) * n_t + tw) * 4 + kb0;
            if (kKB == 4) {
              *reinterpret_cast<u32x4*>(dst) = u32x4{words[it][0], words[it][1], words[it][kKB - 2], words[it][kKB - 1]};
            } else {
              *reinterpret_cast<u32x2*>(dst) = u32x2{words[it][0], words[it][1]};
            }
          }
        }
      }
    }
    if (grp + 1 < n_groups) stage_store(buf ^ 1);
    __syncthreads();
  }
}

hipError_t launch_select_scores(const SelectArgs& a, hipStream_t stream) {
  const int step = a.big_block / a.block_size;
  const dim3 grid((uint32_t)(a.n_ctx / (128 * kKB)) * a.n_kv_heads * a.batch);
  if (step == 16) hipLaunchKernelGGL(select_scores_kernel<16>, grid, dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(select_scores_kernel<32>, grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(64) select_compact_kernel(const SelectArgs p) {
  const int bb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x;
  const int n_bb = p.n_ctx / p.big_block;
  const int n_t = p.n_ctx / 128;
  const int step = p.big_block / p.block_size;
  const int64_t bh = (int64_t)b * p.n_q_heads + h;
  const int t_lo = p.tile_lo, t_hi = step * bb - p.tile_slack;  // candidate key tiles, inclusive
  int base = 0;
  if (t_hi >= t_lo) {
    const int n_words = 4 * (t_hi - t_lo + 1);
    const uint32_t* mw = p.mask + ((bh * n_bb + bb) * n_t + t_lo) * 4;
    int32_t* out = p.coords + bh * p.coords_per_head + coords_tri(bb, p.big_block, p.block_size);
    for (int w0 = 0; w0 < n_words; w0 += 64) {
      const int wi = w0 + lane;
      uint32_t word = wi < n_words ? mw[wi] : 0u;
      const int pc = __popc(word);
      int incl = pc;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      int pos = base + incl - pc;
      const int key_base = t_lo * 128 + wi * 32;
      while (word) {
        out[pos++] = key_base + (__ffs(word) - 1);
        word &= word - 1;
      }
      base += __shfl(incl, 63, 64);
    }
  }
  if (lane == 0) p.counts[bh * n_bb + bb] = base;
}

hipError_t launch_select_compact(const SelectArgs& a, hipStream_t stream) {
  hipLaunchKernelGGL(select_compact_kernel, dim3(a.n_ctx / a.big_block, a.n_q_heads, a.batch), dim3(64), 0, stream, a);
  return hipGetLastError();
}

}  // namespace aa
