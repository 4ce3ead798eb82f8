// Stage 2 of the AnchorAttention prefill path on gfx950: pooling, score-and-threshold, compaction.
//
//  pool     qbar = bf16(mean of 128 raw query rows), abar = bf16(mean of 128 anchors); float32 sums in
//           ascending row order so the result is reproducible bit for bit.
//  scores   K-stationary: one work-group per (batch, KV head, 256 keys); each of its four waves keeps 64
//           keys in registers as the MFMA B operand, and the pooled query rows of EVERY query head of
//           the KV group and EVERY later big block stream past them (A operand, 32 pooled rows per
//           MFMA, staged once per work-group in LDS, 128 rows per barrier).  Each K row is thus read
//           once per KV head instead of once per (query head, big block).
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
// D = head dimension (128 or 64): D/8 lanes of 16 bytes cover a query row, a wave pools 64 / (D/8) blocks.
template <typename T, int D>
__global__ void __launch_bounds__(64) pool_kernel(const PoolArgs p) {
  constexpr int kLanesPerRow = D / 8, kBlocksPerWave = 64 / kLanesPerRow;
  const int lane = threadIdx.x;
  const int c = lane % kLanesPerRow;
  const int n_pr = p.n_ctx / p.block_size;
  const int pr = kBlocksPerWave * blockIdx.x + lane / kLanesPerRow;
  const int h = blockIdx.y, b = blockIdx.z;
  if (pr >= n_pr) return;
  const int bs = p.block_size;
  const uint16_t* base = p.q + b * p.q_sb + h * p.q_sh + (int64_t)pr * bs * p.q_sn + 8 * c;
  const int64_t bh = (int64_t)b * p.n_q_heads + h;
  const float* mb = p.M + bh * p.n_ctx + (int64_t)pr * bs;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float am = 0.f;
#pragma unroll 8
  for (int t = 0; t < bs; ++t) {
    const uint4 raw = *reinterpret_cast<const uint4*>(base + (int64_t)t * p.q_sn);
    acc[0] += T::lo(raw.x); acc[1] += T::hi(raw.x);
    acc[2] += T::lo(raw.y); acc[3] += T::hi(raw.y);
    acc[4] += T::lo(raw.z); acc[5] += T::hi(raw.z);
    acc[6] += T::lo(raw.w); acc[7] += T::hi(raw.w);
    if (c == 0) am += mb[t];
  }
  const float d = (float)bs;
  uint4 o;
  o.x = T::pack(acc[0] / d, acc[1] / d);
  o.y = T::pack(acc[2] / d, acc[3] / d);
  o.z = T::pack(acc[4] / d, acc[5] / d);
  o.w = T::pack(acc[6] / d, acc[7] / d);
  *reinterpret_cast<uint4*>(p.qbar + (bh * n_pr + pr) * D + 8 * c) = o;
  if (c == 0) {
    const uint32_t w = T::pack(am / d, 0.f);
    reinterpret_cast<uint16_t*>(p.abar)[bh * n_pr + pr] = (uint16_t)(w & 0xffffu);
  }
}

hipError_t launch_pool(const PoolArgs& a, hipStream_t stream) {
  const int n_pr = a.n_ctx / a.block_size;
  const int per_wave = a.head_dim == 128 ? 4 : 8;
  const dim3 grid((n_pr + per_wave - 1) / per_wave, a.n_q_heads, a.batch);
  if (a.head_dim == 128) {
    if (a.dtype == 0) hipLaunchKernelGGL((pool_kernel<Bf16, 128>), grid, dim3(64), 0, stream, a);
    else hipLaunchKernelGGL((pool_kernel<F16, 128>), grid, dim3(64), 0, stream, a);
  } else {
    if (a.dtype == 0) hipLaunchKernelGGL((pool_kernel<Bf16, 64>), grid, dim3(64), 0, stream, a);
    else hipLaunchKernelGGL((pool_kernel<F16, 64>), grid, dim3(64), 0, stream, a);
  }
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Smallest float32 x with  float(round16(x * scale2)) + theta >= anchor  (NaN if there is none); round16 rounds to the
// tensors' 16-bit type.
template <typename T>
__device__ __forceinline__ bool select_test(const float x, const float scale2, const float theta, const float anchor) {
  const float sc = T::round_product(x, scale2);  // the score as (dot * scale).to(dtype) evaluates it for this type
  return (sc + theta) >= anchor;      // float32 add and compare, non-strict
}
__device__ __forceinline__ float ordered_to_float(const uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);  // monotone bijection uint32 -> float32
}

template <typename T>
__global__ void __launch_bounds__(256) select_threshold_kernel(const uint16_t* __restrict__ abar, float* __restrict__ thr, const int n,
                                                                const float scale2, const float theta) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float anchor = T::from16(abar[i]);
  // ordered keys: 0x007fffff <-> -inf, 0xff800000 <-> +inf (NaNs lie outside that range)
  uint32_t lo = 0x007fffffu, hi = 0xff800000u;
  float out;
  if (!select_test<T>(ordered_to_float(hi), scale2, theta, anchor)) {
    out = __uint_as_float(0x7fc00000u);  // no float passes: NaN compares false with everything
  } else {
    while (lo < hi) {  // invariant: test(hi) is true
      const uint32_t mid = lo + ((hi - lo) >> 1);
      if (select_test<T>(ordered_to_float(mid), scale2, theta, anchor)) hi = mid; else lo = mid + 1;
    }
    out = ordered_to_float(hi);
  }
  thr[i] = out;
}

hipError_t launch_select_thresholds(const SelectArgs& a, hipStream_t stream) {
  const int n = a.batch * a.n_q_heads * (a.n_ctx / a.block_size);
  if (a.dtype == 0) hipLaunchKernelGGL(select_threshold_kernel<Bf16>, dim3((n + 255) / 256), dim3(256), 0, stream, a.abar, a.thr, n, a.scale2, a.theta_log2);
  else hipLaunchKernelGGL(select_threshold_kernel<F16>, dim3((n + 255) / 256), dim3(256), 0, stream, a.abar, a.thr, n, a.scale2, a.theta_log2);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// STEP = pooled rows per big block (16 or 32); an "item" is one (query head of the KV group, big block) pair, i.e.
// STEP pooled rows that share one output mask word per 32 keys.
//
// Work-group = 4 waves = one super-tile of 256 keys: wave w keeps keys 64*w .. 64*w+63 of it in registers (MFMA B
// operand, 64 VGPRs) for the whole kernel.  The items that can select those keys - every query head of the KV group
// and every big block from bb_lo on - stream past them as the A operand.  The stream is cut into blocks of 128
// pooled rows; a block travels global -> LDS by LDS-DMA loads (no registers, no LDS store instructions) one whole
// block ahead of its use, so a block's loads have the time of 64 MFMAs per wave to land, and the work-group
// synchronises once per block.  LDS rows are unpadded 256 bytes whose 16-byte chunks are XOR-swizzled with the row
// number on the load side (a lane fetches the chunk that belongs in its slot), which makes the row-per-lane 16-byte
// operand reads conflict-free.  The rows' thresholds ride along (4 bytes per row).
//
// Rows 32*w .. 32*w+31 of a block are brought in by wave w: they belong to 32/STEP whole items, so the item -> (head,
// big block) arithmetic is wave-uniform.
constexpr int kKB = 2;            // 32-key blocks a wave keeps in registers (64 keys, 64 VGPRs)
constexpr int kSelRowBytes = 256; // one pooled row in LDS
#ifndef AA_SEL_WAVES
#define AA_SEL_WAVES 4            // waves per work-group (two waves share a 128-key tile)
#endif
#ifndef AA_SEL_ROWS
#define AA_SEL_ROWS 128           // pooled rows staged per barrier
#endif
#ifndef AA_SEL_WGS
#define AA_SEL_WGS 2              // work-groups per CU the kernel is compiled for
#endif

typedef __attribute__((address_space(3))) char sel_lds_char;
__device__ __forceinline__ uint32_t sel_lds_addr(const void* p) { return (uint32_t)(uintptr_t)(sel_lds_char*)p; }
// 64 lanes x 16 bytes (or x 4 bytes) global -> LDS; lane L's bytes land at lds_dst + 16*L (4*L).  lds_dst is wave-uniform
// and travels in M0; the nop covers the wait state an LDS-DMA instruction needs after a scalar write of M0.
__device__ __forceinline__ void sel_load16_to_lds(const char* base, const uint32_t byte_off, const uint32_t lds_dst) {
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "{m0}"(lds_dst), "v"(byte_off), "s"(base) : "memory");
}
__device__ __forceinline__ void sel_load4_to_lds(const char* base, const uint32_t byte_off, const uint32_t lds_dst) {
  asm volatile("s_nop 0\n\tglobal_load_lds_dword %1, %2" : : "{m0}"(lds_dst), "v"(byte_off), "s"(base) : "memory");
}

// D = head dimension (128 or 64).  With 64 the pooled rows keep their 256-byte pitch in LDS: a row fills eight of its
// sixteen 16-byte slots (the staging lanes whose slot belongs to no chunk fetch a duplicate that is never read), so
// the LDS addressing is that of 128 and only the number of MFMA steps over the head dimension changes.
template <int STEP, int WAVES, int ROWS, typename T, int D>
__global__ void __launch_bounds__(64 * WAVES, AA_SEL_WGS) select_scores_kernel(const SelectArgs p) {
  constexpr int kKS = D / 16;                    // MFMA steps over the head dimension
  constexpr int kItems = 32 / STEP;              // items per 32-row MFMA group
  constexpr int kGroups = ROWS / 32;             // MFMA groups per block
  constexpr int kBlockItems = ROWS / STEP;       // items per block
  constexpr int kRowsPerWave = ROWS / WAVES;     // rows of a block a wave brings in
  constexpr int kItemsPerWave = kRowsPerWave / STEP;
  constexpr int kTilesPerWg = WAVES / 2;         // two waves share one 128-key tile
  static_assert(kRowsPerWave % STEP == 0 && kItemsPerWave >= 1 && kRowsPerWave % 4 == 0, "a wave stages whole items");
  static_assert(ROWS % 64 == 0 && ROWS / 64 <= WAVES, "thresholds are staged 64 per wave");
  // the swizzle is written with the row inside a wave's share on the load side (r & 15) and with the row inside a
  // 32-row group on the read side (c32 & 15): the two agree only when a wave's share is whole groups of 16 rows; and
  // the per-item mask words of a block live in lanes 0..63 of one register pair
  static_assert(kRowsPerWave % 16 == 0, "a wave stages whole groups of 16 rows (the swizzle's period)");
  static_assert(kBlockItems <= 64, "one lane per item of a block");
  __shared__ __attribute__((aligned(16))) char a_lds[2][ROWS * kSelRowBytes];
  __shared__ __attribute__((aligned(16))) float thr_lds[2][ROWS];

  // Work-groups are renumbered so that each XCD owns a contiguous range ordered (batch, KV head, super-tile): the
  // pooled queries a work-group streams are those of its KV head's query heads (1 MiB per KV head at 128k tokens),
  // which then stay in that XCD's L2 instead of every XCD cycling through all heads' pooled queries.
  const int S = p.big_block;
  const int n_bb = p.n_ctx / S;
  const int n_t = p.n_ctx / 128;
  const int n_super = n_t / kTilesPerWg;
  uint32_t vid = xcd_remap(blockIdx.x, p.batch * p.n_kv_heads, n_super, 1);
  const int ST = vid % n_super;  // key super-tile (kTilesPerWg * 128 keys); ascending = heaviest first
  vid /= n_super;
  const int kvh = vid % p.n_kv_heads, b = vid / p.n_kv_heads;
  const int n_pr = p.n_ctx / p.block_size;  // pooled rows per head
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, c32 = lane & 31;

  // Key tile t (keys 128t .. 128t+127) holds candidates of big block bb iff it reaches past key_lo and starts below
  // bb*S - key_slack, i.e. bb >= (128t + key_slack) / S + 1.
  auto tile_bb_min = [&](const int t) { return 128 * t + 128 > p.key_lo ? (128 * t + p.key_slack) / S + 1 : n_bb; };
  const int tw = kTilesPerWg * ST + wave / 2;  // this wave's 128-key tile
  const int kb0 = kKB * (wave % 2);           // its first 32-key block inside the tile
  const int bb_min_w = tile_bb_min(tw);
  int bb_lo = n_bb;                           // smallest big block any wave of the work-group needs
#pragma unroll
  for (int i = 0; i < kTilesPerWg; ++i) bb_lo = min(bb_lo, tile_bb_min(kTilesPerWg * ST + i));
  if (bb_lo >= n_bb) return;
  const int group = p.n_q_heads / p.n_kv_heads;
  const int n_items = group * (n_bb - bb_lo);
  const int n_blocks = (n_items * STEP + ROWS - 1) / ROWS;
  // item -> (head in group, big block): item / group = floor(2*item * ceil(2^31 / group) / 2^32), exact for item < 2^16
  // and group < 2^15 (the host checks both)
  const uint32_t magic = (0x80000000u + (uint32_t)group - 1u) / (uint32_t)group;
  auto item_bb_off = [&](const int item) { return (int)__umulhi(2u * (uint32_t)item, magic); };

  typedef typename T::vec8 vec8;
  const uint16_t* kp = p.k + b * p.k_sb + kvh * p.k_sh;
  vec8 kreg[kKB][kKS];
#pragma unroll
  for (int kb = 0; kb < kKB; ++kb) {
    const uint16_t* row = kp + (int64_t)(tw * 128 + 32 * (kb0 + kb) + c32) * p.k_sn + 8 * half;
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) kreg[kb][ks] = *reinterpret_cast<const vec8*>(row + 16 * ks);
  }

  // ---- staging -------------------------------------------------------------------------------
  // Wave w brings in block rows w*kRowsPerWave ..: its load j fills rows 4j + (lane >> 4) of those; a lane brings
  // chunk (lane & 15) ^ (row & 15).  The rows of one wave are whole items, so the item arithmetic is wave-uniform.
  const char* qbar_base = reinterpret_cast<const char*>(p.qbar);
  const char* thr_base = reinterpret_cast<const char*>(p.thr);
  const int64_t head0 = ((int64_t)b * p.n_q_heads + kvh * group) * n_pr;  // first pooled row of the group's first head
  const uint32_t a_lds0 = sel_lds_addr(a_lds[0]) + wave * kRowsPerWave * kSelRowBytes;
  const uint32_t thr_lds0 = sel_lds_addr(thr_lds[0]);
  auto item_first_row = [&](const int item_unclamped) {  // pooled-row number, within the whole qbar array, of an item's first row
    const int item = min(item_unclamped, n_items - 1);   // past the end: repeat the last item
    const int q = item_bb_off(item);
    return (uint32_t)(head0 + (int64_t)(item - q * group) * n_pr + (int64_t)(bb_lo + q) * STEP);
  };
  auto stage_block = [&](const int blk, const int buf) {
    uint32_t item_row0[kItemsPerWave];
#pragma unroll
    for (int it = 0; it < kItemsPerWave; ++it) item_row0[it] = item_first_row(blk * kBlockItems + wave * kItemsPerWave + it);
#pragma unroll
    for (int j = 0; j < kRowsPerWave / 4; ++j) {
      const int r = 4 * j + (lane >> 4);  // row inside the wave's share
      const uint32_t prow = item_row0[r / STEP] + (uint32_t)(r % STEP);
      const uint32_t chunk = (uint32_t)(((lane & 15) ^ (r & 15)) & (D / 8 - 1));
      sel_load16_to_lds(qbar_base, prow * (uint32_t)(2 * D) + chunk * 16u, a_lds0 + buf * (ROWS * kSelRowBytes) + 4 * j * kSelRowBytes);
    }
    if (wave < ROWS / 64) {  // thresholds of block rows 64*wave + lane
      const int r = 64 * wave + lane;
      const uint32_t prow = item_first_row(blk * kBlockItems + r / STEP) + (uint32_t)(r % STEP);
      sel_load4_to_lds(thr_base, prow * 4u, thr_lds0 + buf * (ROWS * 4) + wave * 256);
    }
  };

  stage_block(0, 0);

  // A operand of MFMA step ks: row c32 of the group, chunk 2*ks + half, swizzled with the row's low four bits
  uint32_t a_rd[kKS];
#pragma unroll
  for (int ks = 0; ks < kKS; ++ks) a_rd[ks] = sel_lds_addr(a_lds[0]) + c32 * kSelRowBytes + (((2 * ks + half) ^ (c32 & 15)) << 4);
  typedef __attribute__((address_space(3))) vec8 lds_vec8_t;
  typedef __attribute__((address_space(3))) floatx4 lds_floatx4_t;
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

  for (int blk = 0; blk < n_blocks; ++blk) {
    const int buf = blk & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of block blk has landed
    __syncthreads();                                   // ... and everyone's; everyone is done with the other buffer
    if (blk + 1 < n_blocks) stage_block(blk + 1, buf ^ 1);
    const uint32_t a_off = buf * (ROWS * kSelRowBytes);
    // The groups of a block are straight-line code (no branch between them), so that the operand reads of one group can
    // overlap the products of the previous one.  Every item is computed, also the few that cannot select this wave's
    // keys (a big block below the tile's first one, the padding past the last item): those are simply not stored.
    // The mask words of item i (wave-uniform ballot results) are dropped into lane i of w_lo / w_hi.
    uint32_t w_lo = 0u, w_hi = 0u;
#pragma unroll
    for (int gi = 0; gi < kGroups; ++gi) {
      vec8 a[kKS];
#pragma unroll
      for (int ks = 0; ks < kKS; ++ks) a[ks] = *(const lds_vec8_t*)(uintptr_t)(a_rd[ks] + a_off + gi * 32 * kSelRowBytes);
      // raw-score thresholds of the accumulator rows this lane holds: row i = 8*(r/4) + 4*half + r%4
      float thr[16];
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const floatx4 w = *(const lds_floatx4_t*)(uintptr_t)(thr_lds0 + buf * (ROWS * 4) + (32 * gi + 8 * rq + 4 * half) * 4);
        thr[4 * rq + 0] = w[0]; thr[4 * rq + 1] = w[1];
        thr[4 * rq + 2] = w[2]; thr[4 * rq + 3] = w[3];
      }
      floatx16 c[kKB];
      const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb) c[kb] = T::mfma(a[0], kreg[kb][0], zero);
#pragma unroll
      for (int ks = 1; ks < kKS; ++ks)
#pragma unroll
        for (int kb = 0; kb < kKB; ++kb) c[kb] = T::mfma(a[ks], kreg[kb][ks], c[kb]);
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb) {
        bool hit[kItems];
#pragma unroll
        for (int it = 0; it < kItems; ++it) hit[it] = false;
#pragma unroll
        for (int r = 0; r < 16; ++r) hit[(8 * (r >> 2)) / STEP] |= (c[kb][r] >= thr[r]);  // rows 0..15 -> item 0, 16..31 -> item 1 (STEP 16)
#pragma unroll
        for (int it = 0; it < kItems; ++it) {
          const uint64_t m = __ballot(hit[it]);
          const uint32_t word = (uint32_t)m | (uint32_t)(m >> 32);  // both halves of the wave hold the same keys
          if (kb == 0) w_lo = lane == gi * kItems + it ? word : w_lo;
          else w_hi = lane == gi * kItems + it ? word : w_hi;
        }
      }
    }
    // lane i stores the two words (this wave's 64 keys) of item blk * kBlockItems + i
    if (lane < kBlockItems) {
      const int item = blk * kBlockItems + lane;
      const int q = item_bb_off(min(item, n_items - 1));
      const int bb = bb_lo + q;
      const int hq = kvh * group + (min(item, n_items - 1) - q * group);
      if (item < n_items && bb >= bb_min_w) {
        uint32_t* dst = p.mask + ((((int64_t)b * p.n_q_heads + hq) * n_bb + bb) * n_t + tw) * 4 + kb0;
        *reinterpret_cast<u32x2*>(dst) = u32x2{w_lo, w_hi};
      }
    }
  }
}

template <typename T, int D>
static void launch_select_scores_for(const SelectArgs& a, hipStream_t stream) {
  constexpr int kWaves = AA_SEL_WAVES, kRows = AA_SEL_ROWS;
  const int step = a.big_block / a.block_size;
  const dim3 grid((uint32_t)(a.n_ctx / (64 * kWaves)) * a.n_kv_heads * a.batch);
  if (step == 16) hipLaunchKernelGGL((select_scores_kernel<16, kWaves, kRows, T, D>), grid, dim3(64 * kWaves), 0, stream, a);
  else hipLaunchKernelGGL((select_scores_kernel<32, kWaves, kRows, T, D>), grid, dim3(64 * kWaves), 0, stream, a);
}

hipError_t launch_select_scores(const SelectArgs& a, hipStream_t stream) {
  if (a.head_dim == 128) {
    if (a.dtype == 0) launch_select_scores_for<Bf16, 128>(a, stream);
    else launch_select_scores_for<F16, 128>(a, stream);
  } else {
    if (a.dtype == 0) launch_select_scores_for<Bf16, 64>(a, stream);
    else launch_select_scores_for<F16, 64>(a, stream);
  }
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// One wave per (batch, query head, big block): the candidate keys [key_lo, bb*S - key_slack) of the big block's mask row
// become an ascending index list (popcount per 32-key word, wave prefix sum, each lane writes its word's set bits).
__global__ void __launch_bounds__(64) select_compact_kernel(const SelectArgs p) {
  const int bb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x;
  const int n_bb = p.n_ctx / p.big_block;
  const int n_t = p.n_ctx / 128;
  const int64_t bh = (int64_t)b * p.n_q_heads + h;
  const int key_lo = p.key_lo, key_hi = bb * p.big_block - p.key_slack;  // candidate keys [key_lo, key_hi)
  int base = 0;
  if (key_hi > key_lo) {
    const int w_lo = key_lo / 32, w_hi = (key_hi + 31) / 32;  // mask words [w_lo, w_hi) of the row
    const uint32_t* mw = p.mask + (bh * n_bb + bb) * n_t * 4;
    int32_t* out = p.coords + bh * p.coords_per_head + coords_tri(bb, p.big_block, p.block_size);
    for (int w0 = w_lo; w0 < w_hi; w0 += 64) {
      const int wi = w0 + lane;
      uint32_t word = wi < w_hi ? mw[wi] : 0u;
      // the first and the last word may reach outside the candidate range (block sizes below 32 keys)
      const int k0 = wi * 32;
      if (k0 < key_lo) word &= key_lo - k0 >= 32 ? 0u : ~0u << (key_lo - k0);
      if (k0 + 32 > key_hi) word &= key_hi <= k0 ? 0u : ~0u >> (k0 + 32 - key_hi);
      const int pc = __popc(word);
      int incl = pc;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      int pos = base + incl - pc;
      while (word) {
        out[pos++] = k0 + (__ffs(word) - 1);
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
