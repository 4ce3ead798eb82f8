// Software-pipelined MFMA flash-attention core for gfx950 (256-row work-groups).
//
// Same mathematics and register formulation as aa_flash.hip (transposed S^T = K Q^T with one query
// per lane, P^T fed to the second MFMA straight from the accumulator registers, V row-major in
// LDS read with the transposing ds_read_b64_tr_b16), but a wave owns 64 query rows (two 32-row
// blocks share every K and V operand read, halving LDS traffic per FLOP) and the key loop is
// pipelined at 32-key granularity inside one wave.  Iteration j:
//
//   A:  K operands of sub-tile j+1 (LDS)  |  row max of S_j, first half of the exps
//       MFMA  S_{j+1} = K_{j+1} Q^T  (16)  interleaved with that vector work
//   (rare) rescale the output accumulators if some row's running max moved
//   B:  MFMA  O^T += V_j^T P_j^T  (16)     |  second half of the exps, V operands (LDS),
//       LDS store of sub-tile j+2 (loaded from HBM/L2 during this iteration), loads of sub-tile j+3
//   barrier
//
// Keys travel through a ring of four 32-key LDS slots, one barrier per sub-tile.
#include "aa_common.h"
#include "aa_kernels.h"

namespace aa {

namespace f2 {

constexpr int kBN = 64;          // keys per schedule tile (two 32-key sub-tiles)
constexpr int kSub = 32;         // keys per LDS slot / pipeline step
constexpr int kRowStride = 152;  // bf16 per K/V row in LDS: 304 B, conflict-free for both read patterns (measured)
constexpr int kOsStride = 136;   // bf16 per output-staging row
constexpr int kSlots = 4;
constexpr int BM = 256;

enum FlashMode : int { kAnchor = 0, kSparse = 1, kDense = 2 };

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

#include "aa_acc_asm.inc"

struct Smem {
  union {
    struct {
      __bf16 k[kSlots][kSub * kRowStride];
      __bf16 v[kSlots][kSub * kRowStride];
    } t;
    __bf16 os[4][64 * kOsStride];  // epilogue staging, reuses the tile space
  };
};

__device__ __forceinline__ bf16x8 scale_q8(const u32x4 raw, const float sm_scale, const bool bf16_chain) {
  const uint32_t w[4] = {raw[0], raw[1], raw[2], raw[3]};
  uint32_t o[4];
  if (bf16_chain) {  // bf16(bf16(q * bf16(sm_scale)) * bf16(log2e))
    const float s16 = rn16(sm_scale), c16 = rn16(kLog2e);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = rn16(bf16_lo(w[i]) * s16), b = rn16(bf16_hi(w[i]) * s16);
      o[i] = pack_bf16(a * c16, b * c16);
    }
  } else {  // float32 products, one rounding
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_bf16((bf16_lo(w[i]) * sm_scale) * kLog2e, (bf16_hi(w[i]) * sm_scale) * kLog2e);
  }
  const u32x4 packed = {o[0], o[1], o[2], o[3]};
  return *reinterpret_cast<const bf16x8*>(&packed);
}

struct TileRegs {  // one 32-key sub-tile in flight: two 16-byte chunks of K and of V per thread
  u32x4 k[2];
  u32x4 v[2];
};

template <int MODE>
__device__ __forceinline__ void tile_load(TileRegs& r, const char* kb, const char* vb, const uint32_t k_row_bytes,
                                          const uint32_t v_row_bytes, const int key0, const int tid, const int32_t* cbase,
                                          const int cnt) {
  const int row0 = tid >> 4;
  const uint32_t col = (tid & 15) * 16;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = row0 + 16 * j;
    uint32_t key;
    if (MODE == kSparse) {
      key = (key0 + row < cnt) ? (uint32_t)cbase[key0 + row] : 0u;  // tail lanes read row 0, masked later
    } else {
      key = (uint32_t)(key0 + row);
    }
    r.k[j] = *reinterpret_cast<const u32x4*>(kb + (key * k_row_bytes + col));
    r.v[j] = *reinterpret_cast<const u32x4*>(vb + (key * v_row_bytes + col));
  }
}

__device__ __forceinline__ void tile_store(const TileRegs& r, __bf16* ks, __bf16* vs, const int tid) {
  const int row0 = tid >> 4, c = tid & 15;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int off = (row0 + 16 * j) * kRowStride + 8 * c;
    *reinterpret_cast<u32x4*>(ks + off) = r.k[j];
    *reinterpret_cast<u32x4*>(vs + off) = r.v[j];
  }
}

// max / sum over the two wave halves that hold the same query column
__device__ __forceinline__ float halves_max(const float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(const float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- score tile ---------------------------------------------------------------------------------
// All MFMAs of this kernel are issued through inline assembly so that their register files can be
// chosen by hand: the pre-scaled queries (B operands, 64 registers) and the output accumulators (128
// registers) live in AGPRs, which only MFMAs can read, and the 256 architectural VGPRs are left to the
// two score tiles and the operand traffic.  The compiler does not know these statements are MFMAs and
// adds no wait states after them: a vector instruction may only read a score tile long after the MFMAs
// that produced it (the pipeline below keeps at least eight other MFMAs in between; the prologue waits
// explicitly).
// (AA_S_MFMA_FIRST_i / AA_S_MFMA_i, i = query block * 8 + k-step, come from aa_acc_asm.inc: the B operand
// of each is the query fragment pinned in a[128+4i : 131+4i])

// K operands (A matrix) of one 32-key sub-tile: eight 16-byte LDS reads shared by both query blocks.
__device__ __forceinline__ void k_operands(bf16x8 (&ka)[8], const __bf16* krow) {
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) ka[ks] = *reinterpret_cast<const bf16x8*>(krow + 16 * ks);
}

// in-lane part of the row max over accumulator registers [4*i, 4*i+4) of both query blocks
__device__ __forceinline__ void max_slice(const floatx16 (&s)[2], const int i, float (&mx)[2]) {
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const float a = fmaxf(fmaxf(s[qb][4 * i], s[qb][4 * i + 1]), fmaxf(s[qb][4 * i + 2], s[qb][4 * i + 3]));
    mx[qb] = (i == 0) ? a : fmaxf(mx[qb], a);
  }
}
// the same over registers [8*i, 8*i+8)
__device__ __forceinline__ void max_half(const floatx16 (&s)[2], const int i, float (&mx)[2]) {
  max_slice(s, 2 * i, mx);
  max_slice(s, 2 * i + 1, mx);
}

// completes the row max across the two wave halves; new running max, rescale factor, "did any max move"
__device__ __forceinline__ bool max_finish(const float (&mx)[2], float (&m_run)[2], float (&alpha)[2]) {
  bool rescale = false;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const float m_new = fmaxf(m_run[qb], halves_max(mx[qb]));
    alpha[qb] = fast_exp2(m_run[qb] - m_new);
    rescale |= (m_new != m_run[qb]);
    m_run[qb] = m_new;
  }
  return rescale;
}

// p = exp2(s - m) for accumulator registers R, R+1 of query block QB: rounded to bf16 as one dword of
// the B operand of the second product; the unrounded values go into the row sum.
template <int QB, int R>
__device__ __forceinline__ void exp_pair(const floatx16 (&s)[2], const float (&m_run)[2], float (&psum)[2], u32x4 (&pw)[2]) {
  const float e0 = fast_exp2(s[QB][R] - m_run[QB]), e1 = fast_exp2(s[QB][R + 1] - m_run[QB]);
  psum[QB] += e0;
  psum[QB] += e1;
  pw[QB][(R & 7) >> 1] = pack_bf16(e0, e1);
}

// The eight 32x32 output accumulators (tuple t = d_block*2 + query_block) live in fixed AGPRs a0..a127
// for the whole kernel and are only ever touched by the inline-assembly helpers of aa_acc_asm.inc:
// inside the loop nothing but MFMAs reads or writes them, which leaves the 256 architectural VGPRs
// to Q, the two score tiles and the operand traffic.  (This translation unit is built with
// -mllvm -amdgpu-mfma-vgpr-form so that the score MFMAs, whose results the vector ALUs consume,
// write VGPRs.)  The compiler cannot see that those statements are MFMAs, so every helper that reads
// or rewrites the accumulators with vector instructions first waits out the MFMA write latency.

// O^T += V^T P^T for one 32-key sub-tile: 16 MFMAs, 16 transposing LDS reads shared by the two query blocks.
__device__ __forceinline__ bf16x8 v_operand(const __bf16* src) {
  const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(src));
  const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(src + 8 * kRowStride));
  const shortx8 av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return *reinterpret_cast<const bf16x8*>(&av);
}

// The four V^T operands (one per 32-column d-block) of MFMA step `st` of a 32-key sub-tile.
__device__ __forceinline__ void v_operands(bf16x8 (&va)[4], const __bf16* vrow, const int st) {
  const __bf16* src = vrow + 16 * st * kRowStride;
#pragma unroll
  for (int db = 0; db < 4; ++db) va[db] = v_operand(src + 32 * db);
}

// O^T += V^T P^T: the two MFMAs (one per query block) that consume V^T operand `va` of d-block DB.
#define AA_PV_PAIR(DB, va, pfrag)                 \
  AA_ACC_MFMA_##DB##A(acc, va, pfrag[0]);         \
  AA_ACC_MFMA_##DB##B(acc, va, pfrag[1]);
#define AA_ACC_MFMA_0A AA_ACC_MFMA_0
#define AA_ACC_MFMA_0B AA_ACC_MFMA_1
#define AA_ACC_MFMA_1A AA_ACC_MFMA_2
#define AA_ACC_MFMA_1B AA_ACC_MFMA_3
#define AA_ACC_MFMA_2A AA_ACC_MFMA_4
#define AA_ACC_MFMA_2B AA_ACC_MFMA_5
#define AA_ACC_MFMA_3A AA_ACC_MFMA_6
#define AA_ACC_MFMA_3B AA_ACC_MFMA_7
#define AA_FENCE() __builtin_amdgcn_sched_barrier(0)

// interleave hint for a block with n_mfma MFMAs and plenty of VALU work: one MFMA, then a few VALU ops
#define AA_SCHED_MFMA_VALU(n_mfma, n_valu)               \
  _Pragma("unroll") for (int i_ = 0; i_ < (n_mfma); ++i_) { \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);    \
    __builtin_amdgcn_sched_group_barrier(0x002, (n_valu), 0); \
  }

template <int MODE>
__global__ void __launch_bounds__(256, 1) flash2_kernel(const FlashArgs p) {
  __shared__ __attribute__((aligned(16))) Smem sm;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5;
  const int c32 = lane & 31;

  // ---- which rows ----------------------------------------------------------------------------
  const int group = p.n_q_heads / p.n_kv_heads;
  const int n_qblk = p.n_ctx / BM;
  uint32_t vid = xcd_remap(blockIdx.x, gridDim.x);
  const int g = vid % group;  vid /= group;
  int qblk = vid % n_qblk;    vid /= n_qblk;
  const int kvh = vid % p.n_kv_heads;
  const int b = vid / p.n_kv_heads;
  const int hq = kvh * group + g;
  qblk = n_qblk - 1 - qblk;  // longest rows first (later big blocks also carry the longest index lists)
  const int R0 = qblk * BM;
  const int S = p.big_block;
  const int bb = R0 / S;
  const int wr0 = R0 + wave * 64;
  const int64_t bh = (int64_t)b * p.n_q_heads + hq;
#ifdef AA_CLOCKS  // timing experiments only: shader-clock and 100 MHz reference stamps
  const long long aa_c0 = clock64(), aa_w0 = wall_clock64();
#endif

  const __bf16* qp = p.q + b * p.q_sb + hq * p.q_sh;
  const char* kbase = reinterpret_cast<const char*>(p.k + b * p.k_sb + kvh * p.k_sh);
  const char* vbase = reinterpret_cast<const char*>(p.v + b * p.v_sb + kvh * p.v_sh);
  const uint32_t k_row_bytes = (uint32_t)p.k_sn * 2u, v_row_bytes = (uint32_t)p.v_sn * 2u;

  // ---- tile schedule -------------------------------------------------------------------------
  // n_tiles: 64-key tiles the work-group streams; n_tiles_w: how many of them this wave computes on
  // (a wave's rows end 64*(3-wave) rows before the work-group's, so its causal limit comes earlier).
  int n_tiles, n_tiles_w, n_init = 0, cnt = 0;
  const int32_t* cbase = nullptr;
  if (MODE == kAnchor) {
    n_init = min(S, R0 + BM) / kBN;
    n_tiles = n_init + (bb >= 1 ? (R0 + BM - bb * S) / kBN : 0);
    n_tiles_w = n_tiles - (3 - wave);
  } else if (MODE == kDense) {
    n_tiles = (R0 + BM) / kBN;
    n_tiles_w = n_tiles - (3 - wave);
  } else {
    cnt = p.counts[bh * (p.n_ctx / S) + bb];
    cbase = p.coords + bh * p.coords_per_head + coords_tri(bb, S, p.block_size);
    n_tiles = (cnt + kBN - 1) / kBN;
    n_tiles_w = n_tiles;
  }
#define AA_TILE_KEY0(i) ((MODE == kAnchor) ? ((i) < n_init ? (i) * kBN : bb * S + ((i) - n_init) * kBN) : (i) * kBN)

  // two register sets carry sub-tiles from global memory to LDS: a sub-tile is loaded five pipeline
  // steps before its keys are multiplied, parked in registers for two steps, then stored
  TileRegs trA, trB;
  if (n_tiles > 0) tile_load<MODE>(trA, kbase, vbase, k_row_bytes, v_row_bytes, AA_TILE_KEY0(0), tid, cbase, cnt);
  if (n_tiles > 0) tile_load<MODE>(trB, kbase, vbase, k_row_bytes, v_row_bytes, AA_TILE_KEY0(0) + kSub, tid, cbase, cnt);

  // ---- queries: B operands, pre-scaled into the exp2 domain (held in AGPRs by the MFMA statements) ----
  bf16x8 qa[2][8];
  {
    const bool chain = (MODE == kAnchor) && (p.scale_mode == 0);
    // each fragment is written once into its own AGPR tuple (a128..a191) so that it is born in the
    // register file the MFMAs read it from and is never copied again
#define AA_Q_LOAD(QB, KS, IDX)                                                                              \
    {                                                                                                        \
      const __bf16* row = qp + (int64_t)(wr0 + 32 * (QB) + c32) * p.q_sn + 8 * half;                         \
      const bf16x8 f = scale_q8(*reinterpret_cast<const u32x4*>(row + 16 * (KS)), p.sm_scale, chain);         \
      const u32x4 w = *reinterpret_cast<const u32x4*>(&f);                                                   \
      AA_Q_PIN_##IDX(qa[QB][KS], w);                                                                         \
    }
    AA_Q_LOAD(0, 0, 0) AA_Q_LOAD(0, 1, 1) AA_Q_LOAD(0, 2, 2) AA_Q_LOAD(0, 3, 3)
    AA_Q_LOAD(0, 4, 4) AA_Q_LOAD(0, 5, 5) AA_Q_LOAD(0, 6, 6) AA_Q_LOAD(0, 7, 7)
    AA_Q_LOAD(1, 0, 8) AA_Q_LOAD(1, 1, 9) AA_Q_LOAD(1, 2, 10) AA_Q_LOAD(1, 3, 11)
    AA_Q_LOAD(1, 4, 12) AA_Q_LOAD(1, 5, 13) AA_Q_LOAD(1, 6, 14) AA_Q_LOAD(1, 7, 15)
#undef AA_Q_LOAD
  }
  // S^T of one 32-key sub-tile for both query blocks: 16 MFMAs
#define AA_QK_SUBTILE(s, ka)                                                     \
  AA_S_MFMA_FIRST_0(s[0], ka[0], qa[0][0]); AA_S_MFMA_FIRST_8(s[1], ka[0], qa[1][0]); \
  AA_S_MFMA_1(s[0], ka[1], qa[0][1]); AA_S_MFMA_9(s[1], ka[1], qa[1][1]);             \
  AA_S_MFMA_2(s[0], ka[2], qa[0][2]); AA_S_MFMA_10(s[1], ka[2], qa[1][2]);             \
  AA_S_MFMA_3(s[0], ka[3], qa[0][3]); AA_S_MFMA_11(s[1], ka[3], qa[1][3]);             \
  AA_S_MFMA_4(s[0], ka[4], qa[0][4]); AA_S_MFMA_12(s[1], ka[4], qa[1][4]);             \
  AA_S_MFMA_5(s[0], ka[5], qa[0][5]); AA_S_MFMA_13(s[1], ka[5], qa[1][5]);             \
  AA_S_MFMA_6(s[0], ka[6], qa[0][6]); AA_S_MFMA_14(s[1], ka[6], qa[1][6]);             \
  AA_S_MFMA_7(s[0], ka[7], qa[0][7]); AA_S_MFMA_15(s[1], ka[7], qa[1][7]);

  // ---- running state -------------------------------------------------------------------------
  float m_run[2], l_run[2];
  floatx16 acc[8];
  if (MODE == kSparse) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int row = wr0 + 32 * qb + c32;
      m_run[qb] = p.M[bh * p.n_ctx + row];
      l_run[qb] = half == 0 ? p.L[bh * p.n_ctx + row] : 0.f;  // the two halves are summed at the end
    }
#define AA_LOAD_TUPLE(T)                                                                                           \
    {                                                                                                                \
      const float* af = p.acc_frag + ((bh * (p.n_ctx / 32) + (wr0 + 32 * ((T) & 1)) / 32) * 16 + ((T) >> 1) * 4) * 256 + lane * 4; \
      float x[16];                                                                                                   \
      _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) {                                                            \
        const floatx4 t4 = *reinterpret_cast<const floatx4*>(af + rg * 256);                                         \
        x[4 * rg + 0] = t4[0]; x[4 * rg + 1] = t4[1]; x[4 * rg + 2] = t4[2]; x[4 * rg + 3] = t4[3];                    \
      }                                                                                                              \
      AA_ACC_SET_##T(acc, x);                                                                                        \
    }
    AA_LOAD_TUPLE(0) AA_LOAD_TUPLE(1) AA_LOAD_TUPLE(2) AA_LOAD_TUPLE(3)
    AA_LOAD_TUPLE(4) AA_LOAD_TUPLE(5) AA_LOAD_TUPLE(6) AA_LOAD_TUPLE(7)
#undef AA_LOAD_TUPLE
  } else {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      m_run[qb] = -INFINITY;
      l_run[qb] = 0.f;
    }
    AA_ACC_ZERO_ALL(acc);
  }

  // per-lane LDS read offsets (bf16 elements)
  const int k_rd = c32 * kRowStride + 8 * half;
  const int v_rd = (4 * half + ((lane & 15) >> 2)) * kRowStride + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // ---- sub-tile schedule: sub-tile sidx covers keys/list positions [key0(sidx), key0(sidx)+32) ----
  const int n_sub = 2 * n_tiles, n_sub_w = 2 * n_tiles_w;
#define AA_SUB_KEY0(sidx) (AA_TILE_KEY0((sidx) >> 1) + kSub * ((sidx) & 1))

  // prologue: sub-tiles 0, 1 and 2 go straight to their LDS slots, sub-tiles 3 and 4 stay in flight
  if (n_sub > 0) {
    tile_store(trA, sm.t.k[0], sm.t.v[0], tid);
    tile_store(trB, sm.t.k[1], sm.t.v[1], tid);
    if (n_sub > 2) {
      tile_load<MODE>(trA, kbase, vbase, k_row_bytes, v_row_bytes, AA_SUB_KEY0(2), tid, cbase, cnt);
      tile_store(trA, sm.t.k[2], sm.t.v[2], tid);
    }
    if (n_sub > 3) tile_load<MODE>(trA, kbase, vbase, k_row_bytes, v_row_bytes, AA_SUB_KEY0(3), tid, cbase, cnt);
    if (n_sub > 4) tile_load<MODE>(trB, kbase, vbase, k_row_bytes, v_row_bytes, AA_SUB_KEY0(4), tid, cbase, cnt);
  }
  __syncthreads();

  floatx16 sA[2], sB[2];  // scores of the even / odd sub-tile
  bf16x8 ka[8];
  float alpha[2] = {1.f, 1.f}, mx[2];
  bool rescale = false;

  // mask for registers [4*i, 4*i+4) of the sub-tile starting at key0s (diagonal in anchor/dense mode,
  // tail of the index list in sparse mode)
  auto mask_slice = [&](floatx16 (&s)[2], const int key0s, const int i) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int r = 4 * i; r < 4 * i + 4; ++r) {
        const int key = key0s + 8 * (r >> 2) + 4 * half + (r & 3);
        const bool dead = (MODE == kSparse) ? (key >= cnt) : (key > wr0 + 32 * qb + c32);
        if (dead) s[qb][r] = -INFINITY;
      }
  };
  auto needs_mask = [&](const int key0s) -> bool { return (MODE == kSparse) ? (key0s + kSub > cnt) : (key0s + kSub - 1 > wr0); };

  if (n_sub_w > 0) {  // scores, mask and row max of sub-tile 0 (not overlapped with anything)
    k_operands(ka, sm.t.k[0] + k_rd);
    AA_QK_SUBTILE(sA, ka)
    AA_ACC_SETTLE();
    const int key0s = AA_SUB_KEY0(0);
    const bool msk = needs_mask(key0s);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (msk) mask_slice(sA, key0s, i);
      max_slice(sA, i, mx);
    }
    rescale = max_finish(mx, m_run, alpha);
    k_operands(ka, sm.t.k[1] + k_rd);  // operands of S_1, consumed by the first pipeline step
  }

// timing experiments only (never defined in the product build)
#if defined(AA_ABLATE) && AA_ABLATE == 1
#define AA_ABL_LOAD && (j) < 1
#define AA_ABL_STORE
#define AA_ABL_SYNC lds_barrier()
#elif defined(AA_ABLATE) && AA_ABLATE == 3
#define AA_ABL_LOAD && (j) < 1
#define AA_ABL_STORE && (j) < 1
#define AA_ABL_SYNC lds_barrier()
#elif defined(AA_ABLATE) && AA_ABLATE == 4
#define AA_ABL_LOAD && (j) < 1
#define AA_ABL_STORE && (j) < 1
#define AA_ABL_SYNC
#else
#define AA_ABL_LOAD
#define AA_ABL_STORE
#define AA_ABL_SYNC lds_barrier()
#endif

  // One pipeline step.  On entry S_cur holds the masked scores of sub-tile j and (m_run, alpha,
  // rescale) already include its row max.  MASKN says whether the step contains the code that masks
  // S_{j+1} (only the last two sub-tiles of a wave can need it).  The scheduling fences pin the
  // interleave by hand - one MFMA, then a handful of vector instructions - because the compiler
  // cannot see that the asm statements are MFMAs and would bunch them behind the vector work.
#define AA_KA(i) ka[i] = *reinterpret_cast<const bf16x8*>(knn + 16 * (i));
#define AA_X(S, QB, R) exp_pair<QB, R>(S, m_run, psum, pw0); AA_FENCE();
#define AA_Y(S, QB, R) exp_pair<QB, R>(S, m_run, psum, pw1); AA_FENCE();
#ifdef AA_CLOCKS
  long long aa_ph[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  long long aa_t = clock64();
#define AA_STAMP(i) { const long long t_ = clock64(); aa_ph[i] += t_ - aa_t; aa_t = t_; }
#else
#define AA_STAMP(i)
#endif
#define AA_PIPE_STEP(j, S_cur, S_nxt, MASKN, TR)                                                                      \
  {                                                                                                                \
    AA_STAMP(4)                                                                                                    \
    if ((j) < n_sub_w) {                                                                                           \
      const __bf16* vcur = sm.t.v[(j) & 3] + v_rd;                                                                 \
      const float a_cur[2] = {alpha[0], alpha[1]};                                                                 \
      float psum[2] = {0.f, 0.f};                                                                                  \
      u32x4 pw0[2], pw1[2];                                                                                        \
      bf16x8 va[4];                                                                                                \
      /* A: S_{j+1} = K_{j+1} Q^T (computed even past the wave's last sub-tile; the result is then unused)  */     \
      /*    with three quarters of the exps of S_j in between                                                */     \
      /*    (its K operands were fetched during the previous step; this step's V^T operands of MFMA step 0  */     \
      /*    are fetched between the first score MFMAs)                                                       */     \
      const __bf16* knn = sm.t.k[((j) + 2) & 3] + k_rd;                                                            \
      AA_FENCE();                                                                                                  \
      /* the first exps run while the operands are on their way from LDS */                                        \
      AA_STAMP(5)                                                                                                  \
      AA_X(S_cur, 0, 0) AA_X(S_cur, 1, 0) AA_X(S_cur, 0, 2) AA_X(S_cur, 1, 2)                                      \
      AA_STAMP(6)                                                                                                  \
      AA_S_MFMA_FIRST_0(S_nxt[0], ka[0], qa[0][0]); AA_FENCE(); va[0] = v_operand(vcur); AA_X(S_cur, 0, 4)         \
      AA_S_MFMA_FIRST_8(S_nxt[1], ka[0], qa[1][0]); AA_FENCE(); va[1] = v_operand(vcur + 32); AA_X(S_cur, 1, 4)    \
      AA_S_MFMA_1(S_nxt[0], ka[1], qa[0][1]); AA_FENCE(); va[2] = v_operand(vcur + 64); AA_X(S_cur, 0, 6)          \
      AA_S_MFMA_9(S_nxt[1], ka[1], qa[1][1]); AA_FENCE(); va[3] = v_operand(vcur + 96); AA_X(S_cur, 1, 6)          \
      AA_S_MFMA_2(S_nxt[0], ka[2], qa[0][2]); AA_FENCE(); AA_Y(S_cur, 0, 8)                                        \
      AA_S_MFMA_10(S_nxt[1], ka[2], qa[1][2]); AA_FENCE(); AA_Y(S_cur, 1, 8)                                       \
      AA_S_MFMA_3(S_nxt[0], ka[3], qa[0][3]); AA_FENCE(); AA_Y(S_cur, 0, 10)                                       \
      AA_S_MFMA_11(S_nxt[1], ka[3], qa[1][3]); AA_FENCE(); AA_Y(S_cur, 1, 10)                                      \
      AA_S_MFMA_4(S_nxt[0], ka[4], qa[0][4]); AA_FENCE(); AA_Y(S_cur, 0, 12)                                       \
      AA_S_MFMA_12(S_nxt[1], ka[4], qa[1][4]); AA_FENCE(); AA_Y(S_cur, 1, 12)                                      \
      AA_S_MFMA_5(S_nxt[0], ka[5], qa[0][5]); AA_FENCE(); AA_Y(S_cur, 0, 14)                                       \
      AA_S_MFMA_13(S_nxt[1], ka[5], qa[1][5]); AA_FENCE(); AA_Y(S_cur, 1, 14)                                      \
      AA_STAMP(7)                                                                                                  \
      AA_S_MFMA_6(S_nxt[0], ka[6], qa[0][6]); AA_FENCE();                                                          \
      _Pragma("unroll") for (int qb = 0; qb < 2; ++qb) l_run[qb] = l_run[qb] * a_cur[qb] + psum[qb];              \
      AA_FENCE();                                                                                                  \
      AA_S_MFMA_14(S_nxt[1], ka[6], qa[1][6]); AA_FENCE();                                                         \
      AA_S_MFMA_7(S_nxt[0], ka[7], qa[0][7]); AA_FENCE();                                                          \
      AA_S_MFMA_15(S_nxt[1], ka[7], qa[1][7]); AA_FENCE();                                                         \
      AA_STAMP(0)                                                                                                  \
      /* keeps those exps on this side of the branch */                                                            \
      asm volatile("" : "+v"(pw0[0]), "+v"(pw0[1]), "+v"(pw1[0]), "+v"(pw1[1]), "+v"(l_run[0]), "+v"(l_run[1]));   \
      if (__builtin_expect(__any(rescale), 0)) { /* multiplying by alpha == 1 is exact: skipped when no max moved */ \
        AA_ACC_SCALE_QB0(acc, a_cur[0]);                                                                           \
        AA_ACC_SCALE_QB1(acc, a_cur[1]);                                                                           \
      }                                                                                                            \
      /* B: second product.  Step 0 with the last quarter of the exps in between; every V^T operand of       */     \
      /*    step 1 is fetched as soon as the step-0 pair that used its registers has been issued.            */     \
      const bf16x8* p0 = reinterpret_cast<const bf16x8*>(pw0);                                                     \
      const bf16x8* p1 = reinterpret_cast<const bf16x8*>(pw1);                                                     \
      const bool nxt = (j) + 1 < n_sub_w;                                                                          \
      const int key0n = AA_SUB_KEY0((j) + 1);                                                                      \
      const bool mskn = (MASKN) && nxt && needs_mask(key0n);                                                       \
      AA_FENCE();                                                                                                  \
      AA_ACC_MFMA_0(acc, va[0], p0[0]); AA_FENCE();                                                                \
      AA_ACC_MFMA_1(acc, va[0], p0[1]); AA_FENCE(); va[0] = v_operand(vcur + 16 * kRowStride);                     \
      AA_ACC_MFMA_2(acc, va[1], p0[0]); AA_FENCE();                                                                \
      AA_ACC_MFMA_3(acc, va[1], p0[1]); AA_FENCE(); va[1] = v_operand(vcur + 16 * kRowStride + 32);                \
      AA_ACC_MFMA_4(acc, va[2], p0[0]); AA_FENCE();                                                                \
      if ((MASKN) && mskn) { mask_slice(S_nxt, key0n, 0); mask_slice(S_nxt, key0n, 1); }                           \
      AA_ACC_MFMA_5(acc, va[2], p0[1]); AA_FENCE(); va[2] = v_operand(vcur + 16 * kRowStride + 64);                \
      max_slice(S_nxt, 0, mx); AA_FENCE();                                                                         \
      AA_ACC_MFMA_6(acc, va[3], p0[0]); AA_FENCE();                                                                \
      if ((MASKN) && mskn) { mask_slice(S_nxt, key0n, 2); mask_slice(S_nxt, key0n, 3); }                           \
      AA_ACC_MFMA_7(acc, va[3], p0[1]); AA_FENCE(); va[3] = v_operand(vcur + 16 * kRowStride + 96);                \
      max_slice(S_nxt, 1, mx); AA_FENCE();                                                                         \
      AA_STAMP(1)                                                                                                  \
      /*    Step 1 with the rest of the row max of S_{j+1} in between (its MFMAs were issued >= 8 MFMAs ago). */    \
      /*    and the K operands of S_{j+2} fetched one per MFMA (their LDS slot was filled two steps ago)       */     \
      AA_ACC_MFMA_0(acc, va[0], p1[0]); AA_FENCE(); AA_KA(0) max_slice(S_nxt, 2, mx); AA_FENCE();                  \
      AA_ACC_MFMA_1(acc, va[0], p1[1]); AA_FENCE(); AA_KA(1) max_slice(S_nxt, 3, mx); AA_FENCE();                  \
      AA_ACC_MFMA_2(acc, va[1], p1[0]); AA_FENCE(); AA_KA(2)                                                       \
      if (nxt) rescale = max_finish(mx, m_run, alpha);                                                             \
      AA_FENCE();                                                                                                  \
      AA_ACC_MFMA_3(acc, va[1], p1[1]); AA_FENCE(); AA_KA(3) AA_FENCE();                                           \
      AA_ACC_MFMA_4(acc, va[2], p1[0]); AA_FENCE(); AA_KA(4) AA_FENCE();                                           \
      AA_ACC_MFMA_5(acc, va[2], p1[1]); AA_FENCE(); AA_KA(5) AA_FENCE();                                           \
      AA_ACC_MFMA_6(acc, va[3], p1[0]); AA_FENCE(); AA_KA(6) AA_FENCE();                                           \
      AA_ACC_MFMA_7(acc, va[3], p1[1]); AA_FENCE(); AA_KA(7) AA_FENCE();                                           \
      AA_STAMP(2)                                                                                                  \
    }                                                                                                              \
    /* sub-tile j+3 (loaded two steps ago) goes to its slot; sub-tile j+5 starts its trip */                            \
    if ((j) + 3 < n_sub AA_ABL_STORE) tile_store(TR, sm.t.k[((j) + 3) & 3], sm.t.v[((j) + 3) & 3], tid);            \
    if ((j) + 5 < n_sub AA_ABL_LOAD) tile_load<MODE>(TR, kbase, vbase, k_row_bytes, v_row_bytes, AA_SUB_KEY0((j) + 5), tid, cbase, cnt); \
    AA_ABL_SYNC;                                                                                                   \
    AA_STAMP(3)                                                                                                    \
  }

  // only the last two sub-tiles of a wave can need masking (the diagonal, or the tail of the index list)
  const int j_mask = n_sub_w - 2;
  for (int j = 0; j < n_sub; j += 2) {
    AA_PIPE_STEP(j, sA, sB, true, trA)
    AA_PIPE_STEP(j + 1, sB, sA, true, trB)
  }
#undef AA_PIPE_STEP
#undef AA_X
#undef AA_KA
#undef AA_Y
#undef AA_SUB_KEY0
#undef AA_TILE_KEY0

#ifdef AA_CLOCKS
  if (MODE == kAnchor && tid == 0 && qblk == n_qblk / 2 && hq == 0 && b == 0) {
    p.L_out[bh * p.n_ctx + p.n_ctx - 1] = (float)(clock64() - aa_c0);
    p.L_out[bh * p.n_ctx + p.n_ctx - 2] = (float)(wall_clock64() - aa_w0);
    p.L_out[bh * p.n_ctx + p.n_ctx - 3] = (float)n_tiles;
    for (int i = 0; i < 8; ++i) p.L_out[bh * p.n_ctx + p.n_ctx - 4 - i] = (float)aa_ph[i];
  }
#endif
  // ---- epilogue --------------------------------------------------------------------------------
  AA_ACC_SETTLE();
  float l_tot[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) l_tot[qb] = halves_sum(l_run[qb]);
  if (MODE == kAnchor) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int row = wr0 + 32 * qb + c32;
      if (half == 0) {
        p.M_out[bh * p.n_ctx + row] = m_run[qb];
        p.L_out[bh * p.n_ctx + row] = l_tot[qb];
      }
    }
#define AA_STORE_TUPLE(T)                                                                                          \
    {                                                                                                                \
      float* af = p.acc_out + ((bh * (p.n_ctx / 32) + (wr0 + 32 * ((T) & 1)) / 32) * 16 + ((T) >> 1) * 4) * 256 + lane * 4; \
      float x[16];                                                                                                   \
      AA_ACC_GET_##T(acc, x);                                                                                        \
      _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) {                                                            \
        const floatx4 t4 = {x[4 * rg + 0], x[4 * rg + 1], x[4 * rg + 2], x[4 * rg + 3]};                             \
        *reinterpret_cast<floatx4*>(af + rg * 256) = t4;                                                             \
      }                                                                                                              \
    }
    AA_STORE_TUPLE(0) AA_STORE_TUPLE(1) AA_STORE_TUPLE(2) AA_STORE_TUPLE(3)
    AA_STORE_TUPLE(4) AA_STORE_TUPLE(5) AA_STORE_TUPLE(6) AA_STORE_TUPLE(7)
#undef AA_STORE_TUPLE
  } else {
    // out = bf16(acc / l): stage the wave's [64][128] tile in LDS, then write whole rows
    __syncthreads();  // every wave is done with the K/V tiles the staging area overlays
    __bf16* os = sm.os[wave];
    const float inv[2] = {1.0f / l_tot[0], 1.0f / l_tot[1]};
#define AA_STAGE_TUPLE(T)                                                                                          \
    {                                                                                                                \
      float x[16];                                                                                                   \
      AA_ACC_GET_##T(acc, x);                                                                                        \
      const float iv = inv[(T) & 1];                                                                                 \
      _Pragma("unroll") for (int rg = 0; rg < 4; ++rg) {                                                            \
        u32x2 w;                                                                                                     \
        w[0] = pack_bf16(x[4 * rg + 0] * iv, x[4 * rg + 1] * iv);                                                    \
        w[1] = pack_bf16(x[4 * rg + 2] * iv, x[4 * rg + 3] * iv);                                                    \
        *reinterpret_cast<u32x2*>(&os[(32 * ((T) & 1) + c32) * kOsStride + 32 * ((T) >> 1) + 8 * rg + 4 * half]) = w; \
      }                                                                                                              \
    }
    AA_STAGE_TUPLE(0) AA_STAGE_TUPLE(1) AA_STAGE_TUPLE(2) AA_STAGE_TUPLE(3)
    AA_STAGE_TUPLE(4) AA_STAGE_TUPLE(5) AA_STAGE_TUPLE(6) AA_STAGE_TUPLE(7)
#undef AA_STAGE_TUPLE
    __syncthreads();
    __bf16* op = p.out + b * p.o_sb + hq * p.o_sh;
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int r = it * 4 + (lane >> 4), c = lane & 15;
      const u32x4 w = *reinterpret_cast<const u32x4*>(&os[r * kOsStride + 8 * c]);
      *reinterpret_cast<u32x4*>(op + (int64_t)(wr0 + r) * p.o_sn + 8 * c) = w;
    }
  }
}

}  // namespace f2

hipError_t launch_flash2(const FlashArgs& a, int mode, hipStream_t stream) {
  const uint32_t grid = (uint32_t)a.batch * a.n_q_heads * (a.n_ctx / f2::BM);
  if (mode == f2::kAnchor) hipLaunchKernelGGL((f2::flash2_kernel<f2::kAnchor>), dim3(grid), dim3(256), 0, stream, a);
  else if (mode == f2::kSparse) hipLaunchKernelGGL((f2::flash2_kernel<f2::kSparse>), dim3(grid), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((f2::flash2_kernel<f2::kDense>), dim3(grid), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace aa
