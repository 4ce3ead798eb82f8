// MFMA flash-attention core for gfx950, used three ways:
//   kAnchor : stage 1 - windowed causal attention over [0,S) U [bb*S, r]; emits M, L, Acc
//   kSparse : stage 3 - resumes from (M, L, Acc) over K/V rows gathered at selected indices
//   kDense  : plain causal attention (baseline)
//
// Formulation.  A wave owns 32 query rows and computes the TRANSPOSED score tile
//   S^T[key][query] = K[key][:] . Q[query][:]      (MFMA A = K rows from LDS, B = Q from registers)
// so that in the 32x32 accumulator layout a lane holds one query column: the soft-max statistics
// of a query are then plain per-lane scalars (one exchange with the lane 32 positions away
// completes the row max).  The second product is computed transposed as well,
//   O^T[d][query] += V^T[d][key] . P^T[key][query]  (A = V^T, B = P^T straight from the S^T
// accumulator registers, rounded to bf16) - P never travels through LDS.
// The contraction slot k = 8*(lane/32) + e of MFMA step st of key block kb is fed from accumulator
// register 8*st + e, i.e. key 32*kb + 16*st + 8*(e/4) + 4*(lane/32) + e%4: two runs of four
// consecutive keys.  V sits row-major in LDS exactly as it is in memory, and each run of four keys
// at one head-dim column is fetched with the transposing LDS read ds_read_b64_tr_b16 (within a group
// of 16 lanes, lane i receives column i of the 4x16 block whose rows the group's lanes point at).
//
// The running row max m is subtracted inside the first product: the score accumulators start from
// -m (a per-lane constant, kept replicated in a 16-register tuple) instead of zero, so the tile
// arrives as S - m and p = exp2(S - m) needs no subtraction.  Only when some row's max grows (rare
// after the first tiles) does the wave take a slow path that shifts the tile, re-bases the tuple and
// rescales the accumulators - which is exact for the lanes whose max did not move (shift 0, factor 1).
//
// Inside a 64-key tile the two 32-key halves are staggered so that matrix and vector work overlap
// within a wave: S0 | S1 with soft-max(S0) | P0.V0 with soft-max(S1) | P1.V1.  The online soft-max
// therefore advances 32 keys at a time.
//
// Work-group = 4 waves = 128 query rows; keys are consumed 64 at a time through a
// double-buffered LDS tile that the memory system fills directly (global_load_lds_dwordx4: no staging
// registers, no LDS store instructions).  Such a load writes lane L's 16 bytes at M0 + 16*L, so LDS rows
// are unpadded 256 bytes; bank conflicts are avoided by XOR-swizzling the 16-byte chunks of a row, which
// costs nothing on the load side (a lane simply fetches the chunk that belongs in its slot):
//   K row r, chunk c  ->  slot c ^ (r & 15)          (row-per-lane 16-byte reads)
//   V row r, chunk c  ->  slot c ^ ((r & 7) << 1)    (transposing 8-byte reads)
// Both choices measure conflict-free for their read pattern (and each is 2-way conflicted for the other's).
#include <type_traits>

#include "aa_common.h"
#include "aa_kernels.h"

namespace aa {

constexpr int kBN = 64;        // keys per LDS tile
constexpr int kRowBytes = 256;   // pitch of a K/V row in LDS (128 16-bit elements, unpadded, chunks swizzled; head dimension 64 fills half)
constexpr int kTileBytes = kBN * kRowBytes;
constexpr int kDist = 4;         // MFMA operands are fetched from LDS this many MFMAs ahead of their use
constexpr int kIdxWin = 1024;    // selected-key indices held in LDS at a time (16 tiles)

enum FlashMode : int { kAnchor = 0, kSparse = 1, kDense = 2 };

// Timing-only ablations.  A build with -DAA_ABLATE=n (`make ablations`) leaves out one ingredient of the kernel so
// that its cost can be measured (bench_ablations.py); such a build computes WRONG results on purpose, reports
// aa_version() >= 1000 and is refused by the Python loader.  0, the default, is the product.
//   1  exp2 of the soft-max replaced by a pass-through        4  (sparse) no tile loop: state in, output out
//   2  no soft-max arithmetic at all (mask, max, exp, sum)    5  (sparse) accumulator state not loaded
//   3  no K/V tile loads inside the tile loop                 6  (sparse) at most two tiles per query block
//                                                             7  (sparse) 4 and 5 together
//   8  no work-group barrier at the end of a tile             9  neither the barrier nor the wait for the tile's loads
//  10  the soft-max is computed in full (same instructions, same energy) but the second product takes a loop-invariant
//      operand instead of P: the dependency scores -> soft-max -> P.V inside a wave is cut, nothing else changes
#ifndef AA_ABLATE
#define AA_ABLATE 0
#endif
#ifndef AA_SPARSE_CHAIN
#define AA_SPARSE_CHAIN 1  // 0: every query block of a stage-3 work-group requests its own first tile, queries and state
#endif

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

template <bool WITH_IDX>
struct FlashSmem {
  struct {
    char k[2][kTileBytes];
    char v[2][kTileBytes];
  } t;  // (the epilogue stages the output in the tile space)
  int32_t idx[WITH_IDX ? kIdxWin : 4];  // sparse mode: window of the big block's index list
};

// Query pre-scaling into the exp2 domain, eight elements at a time.  `chain`: both constants and both products rounded
// to the tensors' 16-bit type (stage 1, whose definition takes sm_scale as a compile-time constant); otherwise float32
// products and one rounding.
template <typename T>
__device__ __forceinline__ typename T::vec8 scale_q8(const u32x4 raw, const float sm_scale, const bool chain) {
  const uint32_t w[4] = {raw[0], raw[1], raw[2], raw[3]};
  uint32_t o[4];
  if (chain) {  // r16(r16(q * r16(sm_scale)) * r16(log2e))
    const float s16 = T::round(sm_scale), c16 = T::round(kLog2e);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = T::round(T::lo(w[i]) * s16), b = T::round(T::hi(w[i]) * s16);
      o[i] = T::pack(a * c16, b * c16);
    }
  } else {  // float32 products, one rounding
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = T::pack((T::lo(w[i]) * sm_scale) * kLog2e, (T::hi(w[i]) * sm_scale) * kLog2e);
  }
  const u32x4 packed = {o[0], o[1], o[2], o[3]};
  return *reinterpret_cast<const typename T::vec8*>(&packed);
}

typedef __attribute__((address_space(3))) char lds_char;
__device__ __forceinline__ uint32_t lds_addr(const void* p) { return (uint32_t)(uintptr_t)(lds_char*)p; }

// 64 lanes x 16 bytes, global -> LDS without passing through registers: lane L's bytes land at
// lds_dst + 16*L (lds_dst is wave-uniform and travels in M0).  Completion is tracked by vmcnt.
__device__ __forceinline__ void load16_to_lds(const char* base, const uint32_t byte_off, const uint32_t lds_dst) {
  // the LDS base is bound to M0 by the constraint, so the compiler knows that M0 is written here; the nop covers the
  // wait state an LDS-DMA instruction needs after a scalar write of M0 (the compiler does not look inside the asm)
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "{m0}"(lds_dst), "v"(byte_off), "s"(base) : "memory");
}

// One K/V tile: wave w fills LDS rows 16*j + 4*w .. +3 (j = 0..3), i.e. thread t brings the chunk that belongs in
// slot (t & 15) of row (t >> 4) + 16*j; tile_fetch_one issues one of the tile's eight loads.  `kb`/`vb` are the
// wave-uniform head bases, `k_col`/`v_col` the byte offset of this thread's (swizzled) chunk inside a row,
// `lds_k`/`lds_v` the LDS address of row 4*w of the destination tile.  Gathered tiles take their row numbers from
// the LDS window of the index list (a dependent global load per tile would put a full memory latency on the
// critical path of every tile); the caller reads a tile's four row numbers per lane (`gather_keys`, see tile_gather_keys)
// before it issues the tile's first load: a wave's LDS reads are served in order with its global -> LDS loads, so a row
// number read after a load would arrive only when that load's data has.
// the row numbers lane `tid` needs for the gathered tile at list position key0 (positions past the count hold 0: row 0,
// masked later)
__device__ __forceinline__ void tile_gather_keys(uint32_t (&keys)[4], const int32_t* idx_win, const int key0, const int tid) {
#pragma unroll
  for (int j = 0; j < 4; ++j) keys[j] = (uint32_t)idx_win[(key0 + (tid >> 4) + 16 * j) & (kIdxWin - 1)];
}

template <int MODE>
__device__ __forceinline__ void tile_fetch_one(const int n, const char* kb, const char* vb, const uint32_t k_row_bytes,
                                               const uint32_t v_row_bytes, const uint32_t k_col, const uint32_t v_col, const int key0,
                                               const uint32_t* gather_keys, const uint32_t lds_k, const uint32_t lds_v,
                                               const uint32_t k_voff, const uint32_t v_voff) {
  const int j = n >> 1;  // load n: K (even n) or V (odd n) rows 16*j + ...
  if (MODE == kSparse) {
    const uint32_t key = gather_keys[j];  // this lane's row of the tile's j-th block of 16 rows
    if ((n & 1) == 0) load16_to_lds(kb, __umul24(key, k_row_bytes) + k_col, lds_k + 16 * j * kRowBytes);
    else load16_to_lds(vb, __umul24(key, v_row_bytes) + v_col, lds_v + 16 * j * kRowBytes);
  } else {
    // consecutive keys: the first row of the tile's j-th block of 16 rows goes into the (scalar) base address, the
    // thread's row inside the block and its chunk are one loop-invariant vector offset - no vector arithmetic per tile
    if ((n & 1) == 0) load16_to_lds(kb + (uint64_t)(uint32_t)(key0 + 16 * j) * k_row_bytes, k_voff, lds_k + 16 * j * kRowBytes);
    else load16_to_lds(vb + (uint64_t)(uint32_t)(key0 + 16 * j) * v_row_bytes, v_voff, lds_v + 16 * j * kRowBytes);
  }
}

// D is the head dimension, 128 or 64.  With 64 the LDS tiles keep their 256-byte row pitch and their swizzles - a row
// then fills eight of its sixteen 16-byte slots, the lanes of a tile load that would bring the other eight fetch a
// duplicate that is never read - so every LDS address below is the same for both sizes, and only the number of MFMA steps
// over the head dimension (kKS per 32 keys of Q.K^T) and of 32-column output blocks (kDB) changes.
template <int MODE, typename T, int D>
__global__ void __launch_bounds__(256, 2) flash_kernel(const FlashArgs p) {
  typedef typename T::vec8 vec8;
  typedef __attribute__((address_space(3))) vec8 lds_vec8;
  __shared__ __attribute__((aligned(16))) FlashSmem<MODE == kSparse> sm;
  constexpr int BM = 128;
  static_assert(D == 128 || D == 64, "head dimension");
  constexpr int kKS = D / 16;       // MFMAs per 32-key block of S^T = K Q^T
  constexpr int kDB = D / 32;       // 32-column blocks of the head dimension: accumulators of O^T
  constexpr int kNS = 2 * kKS;      // S^T slots of a 64-key tile
  constexpr int kNV = 4 * kDB;      // O^T slots of a 64-key tile (two 16-key steps per 32-key block)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5;
  const int c32 = lane & 31;

  // ---- which rows ----------------------------------------------------------------------------
  // A work-group owns 128 query rows - in sparse mode p.q_blocks_per_wg consecutive blocks of 128 rows of one big
  // block, one after the other: they share the big block's index list (fetched once), and the output stores of one
  // block drain while the next one is already loading, instead of every 128 rows paying for a work-group launch, the
  // list's round trip to memory and the wait for its stores.
  const int group = p.n_q_heads / p.n_kv_heads;
  const int nq = MODE == kSparse ? p.q_blocks_per_wg : 1;
  const int n_qunit = p.n_ctx / (BM * nq);
  const int S = p.big_block;
  int g, qunit, kvh, b;
  const uint32_t n_pairs = (uint32_t)(p.batch * p.n_kv_heads) * (uint32_t)(p.n_ctx / S);
  if (MODE == kSparse && n_pairs % 8u == 0u) {
    // Stage 3's work per (KV head, big block) pair is the length of the pair's index lists, which depends on the data:
    // a head whose queries select many keys would keep its XCD busy long after the others have finished if whole
    // heads were tied to XCDs.  So the unit that stays on one XCD (and shares its L2) is the pair - the query blocks of
    // a big block and the heads of a KV group gather the same rows - and consecutive pairs, ordered latest big block
    // first, go round-robin over the XCDs with a rotation, so that every XCD sees every head and every depth.
    const uint32_t per_pair = (uint32_t)group * (uint32_t)(S / (BM * nq));  // work-groups of a pair
    const uint32_t n_units = (uint32_t)(p.batch * p.n_kv_heads);
    const uint32_t xcd = blockIdx.x % 8u, k = blockIdx.x / 8u;
    const uint32_t kp = k / per_pair, within = k % per_pair;
    const uint32_t pair = kp * 8u + (xcd + kp) % 8u;
    const int bb_ = p.n_ctx / S - 1 - (int)(pair / n_units);
    const uint32_t unit = pair % n_units;
    g = within % group;
    qunit = bb_ * (S / (BM * nq)) + (int)(within / group);
    kvh = unit % p.n_kv_heads;
    b = unit / p.n_kv_heads;
  } else {
    uint32_t vid = xcd_remap(blockIdx.x, p.batch * p.n_kv_heads, group * n_qunit, group);
    g = vid % group;  vid /= group;
    qunit = vid % n_qunit;  vid /= n_qunit;
    kvh = vid % p.n_kv_heads;
    b = vid / p.n_kv_heads;
    qunit = n_qunit - 1 - qunit;  // longest rows first (later big blocks also carry the longest index lists)
  }
  const int hq = kvh * group + g;
  const int bb = qunit * nq * BM / S;  // (all blocks of a work-group lie in one big block: the host picks q_blocks_per_wg so)
  const int64_t bh = (int64_t)b * p.n_q_heads + hq;

  const uint16_t* qp = p.q + b * p.q_sb + hq * p.q_sh;
  const char* kbase = reinterpret_cast<const char*>(p.k + b * p.k_sb + kvh * p.k_sh);
  const char* vbase = reinterpret_cast<const char*>(p.v + b * p.v_sb + kvh * p.v_sh);
  const uint32_t k_row_bytes = (uint32_t)p.k_sn * 2u, v_row_bytes = (uint32_t)p.v_sn * 2u;

  // ---- sparse mode: what the query blocks of a work-group share, and what they hand to each other -------
  // All blocks lie in one big block of one head, so they walk the same index list and gather the same tiles.  When the
  // list fits the LDS window, the blocks are chained: the last tile of a block brings the list's first tile into the idle
  // buffer for the next block, whose queries and statistics are requested before the output of the block is staged and
  // whose accumulator state is requested as soon as the staging has emptied the accumulator registers - so the next
  // block starts its first product without a round trip to memory of its own.
  int cnt = 0, cap = 0, sparse_tiles = 0;
  const int32_t* cbase = nullptr;
  if (MODE == kSparse) {
    cap = max(bb * S - 2 * p.block_size, 0);  // capacity of the big block's list (a multiple of 4)
    // (counts and indices come from device memory the caller filled: a count beyond the capacity or an index beyond
    // the context is clamped rather than followed out of bounds)
    cnt = max(0, min(p.counts[bh * (p.n_ctx / S) + bb], cap));
    cbase = p.coords + bh * p.coords_per_head + coords_tri(bb, S, p.block_size);
    sparse_tiles = (cnt + kBN - 1) / kBN;
    if (AA_ABLATE == 4 || AA_ABLATE == 7) sparse_tiles = 0;
    if (AA_ABLATE == 6) sparse_tiles = min(sparse_tiles, 2);
  }
  const bool list_chains = MODE == kSparse && AA_SPARSE_CHAIN && sparse_tiles > 0 && sparse_tiles <= kIdxWin / kBN;
  int cur = 0;             // (sparse) LDS buffer of the next tile to be computed
  bool chained = false;    // (sparse) this block's first tile and state were requested by the previous block
  bool have_queries = false;  // (sparse) so were its queries and statistics
  u32x4 qraw[kKS];
  float m_in = 0.f, l_in = 0.f;
  floatx16 acc[kDB];
  // (sparse) queries and soft-max statistics of the block whose lane row is `row`
  auto request_queries = [&](const int row) __attribute__((always_inline)) {
    const uint16_t* qr = qp + (int64_t)row * p.q_sn + 8 * half;
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) qraw[ks] = *reinterpret_cast<const u32x4*>(qr + 16 * ks);
    m_in = p.M[bh * p.n_ctx + row];
    l_in = half == 0 ? p.L[bh * p.n_ctx + row] : 0.f;  // the two halves are summed at the end
  };
  // (sparse) the accumulator state of that block.  (The accumulator state and the output are touched once each: they
  // are written and read with the non-temporal hint, so that they do not push K/V rows, which many work-groups share,
  // out of the L2.)
  auto request_state = [&](const int row) __attribute__((always_inline)) {
    const float* af = p.acc_frag + ((bh * (p.n_ctx / 32) + row / 32) * (4 * kDB)) * 256 + lane * 4;
#pragma unroll
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        floatx4 t = {0.f, 0.f, 0.f, 0.f};
        if (AA_ABLATE != 5 && AA_ABLATE != 7) t = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(af + (db * 4 + rg) * 256));
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[db][rg * 4 + c] = t[c];
      }
  };

  for (int qb = 0; qb < nq; ++qb) {
  const int R0 = (qunit * nq + qb) * BM;
  const int wr0 = R0 + wave * 32;
  const int my_row = wr0 + c32;

  // ---- sparse mode: the queries and the softmax statistics are requested first ----------------------
  // They depend on nothing, whereas the first K/V tile needs the index list, which needs its own round trip to
  // memory.  The 64 KB of accumulator state follow the first tile's loads (further down) and are not waited for
  // before the first scores are computed.
  float m_run, l_run;
  const uint16_t* qrow = qp + (int64_t)my_row * p.q_sn + 8 * half;
  if (MODE == kSparse && !have_queries) request_queries(my_row);
  const bool feeds_next = list_chains && qb + 1 < nq;  // the next block takes its first tile from this one

  // ---- tile schedule -------------------------------------------------------------------------
  const bool pool = MODE == kAnchor && p.qbar_out != nullptr;
  int n_tiles, n_init = 0;
  if (MODE == kAnchor) {
    n_init = min(S, R0 + BM) / kBN;
    n_tiles = n_init + (bb >= 1 ? (R0 + BM - bb * S) / kBN : 0);
  } else if (MODE == kDense) {
    n_tiles = (R0 + BM) / kBN;
  } else {
    n_tiles = sparse_tiles;
  }
  // first key (anchor, dense) or first list position (sparse) of tile i
#define AA_TILE_KEY0(i) ((MODE == kAnchor) ? ((i) < n_init ? (i) * kBN : bb * S + ((i) - n_init) * kBN) : (i) * kBN)

  // sparse mode: list positions [w0, w0 + kIdxWin) -> LDS (zeros past the count).  The load is bounded by the list's
  // capacity, not by its count, so that it does not have to wait for the count to arrive; what lies past the count is
  // zeroed afterwards.
  auto fill_index_window = [&](const int w0) {
    const int pos = w0 + 4 * tid;
    int4 v = {0, 0, 0, 0};
    if (pos < cap) v = *reinterpret_cast<const int4*>(cbase + pos);  // lists start 16-byte aligned; capacity is a multiple of 4
    if (pos >= cnt) v.x = 0;
    if (pos + 1 >= cnt) v.y = 0;
    if (pos + 2 >= cnt) v.z = 0;
    if (pos + 3 >= cnt) v.w = 0;
    const uint32_t last = (uint32_t)p.n_ctx - 1u;
    v.x = (int)min((uint32_t)v.x, last);
    v.y = (int)min((uint32_t)v.y, last);
    v.z = (int)min((uint32_t)v.z, last);
    v.w = (int)min((uint32_t)v.w, last);
    *reinterpret_cast<int4*>(&sm.idx[4 * tid]) = v;
  };
  // (uniform over the work-group; not conditioned on the count, see above.  Later blocks of the work-group find the
  // list's first window still in place unless the list is longer than the window)
  if (MODE == kSparse && cap > 0 && (qb == 0 || n_tiles > kIdxWin / kBN)) {
    fill_index_window(0);
    __syncthreads();
  }

  // this thread's chunk of a row (swizzled: see the top of the file) and the wave's slice of the LDS tiles
  // (head dimension 64: a row has eight chunks; the lanes whose slot belongs to none of them fetch a duplicate)
  const uint32_t k_col = (uint32_t)(((tid & 15) ^ ((tid >> 4) & 15)) & (D / 8 - 1)) * 16u;
  const uint32_t v_col = (uint32_t)(((tid & 15) ^ (((tid >> 4) & 7) << 1)) & (D / 8 - 1)) * 16u;
  const uint32_t lds_k0 = lds_addr(sm.t.k[0]) + wave * 4 * kRowBytes, lds_v0 = lds_addr(sm.t.v[0]) + wave * 4 * kRowBytes;
  // byte offset of this thread's chunk of row (tid >> 4) of a block of 16 tile rows from the block's first row
  const uint32_t k_voff = (tid >> 4) * k_row_bytes + k_col, v_voff = (tid >> 4) * v_row_bytes + v_col;
  // (anchor mode with pooling) the work-group's raw query rows, fetched like a tile by the last tile's load slots
  const char* qblock = reinterpret_cast<const char*>(qp + (int64_t)R0 * p.q_sn);
  const uint32_t q_row_bytes = (uint32_t)p.q_sn * 2u;
  const uint32_t q_voff = (uint32_t)(tid >> 4) * q_row_bytes + (uint32_t)((tid & 15) & (D / 8 - 1)) * 16u;
  if (n_tiles > 0 && !chained) {
    const uint32_t first = MODE == kSparse ? (uint32_t)cur * kTileBytes : 0u;
    uint32_t keys0[4] = {0u, 0u, 0u, 0u};
    if (MODE == kSparse) tile_gather_keys(keys0, sm.idx, 0, tid);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      tile_fetch_one<MODE>(j, kbase, vbase, k_row_bytes, v_row_bytes, k_col, v_col, AA_TILE_KEY0(0), keys0, lds_k0 + first,
                           lds_v0 + first, k_voff, v_voff);
  }
  // the accumulator state: the youngest loads in flight, first needed by the first P.V product
  if (MODE == kSparse && !chained) request_state(my_row);

  // ---- queries: B operand, pre-scaled into the exp2 domain -----------------------------------
  vec8 qreg[kKS];
  {
    const bool chain = (MODE == kAnchor) && (p.scale_mode == 0);
    if (MODE != kSparse) {
#pragma unroll
      for (int ks = 0; ks < kKS; ++ks) qraw[ks] = *reinterpret_cast<const u32x4*>(qrow + 16 * ks);
    }
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) qreg[ks] = scale_q8<T>(qraw[ks], p.sm_scale, chain);
  }

  // ---- running state (sparse mode loaded it at the top) -----------------------------------------
  if (MODE != kSparse) {
    m_run = -INFINITY;
    l_run = 0.f;
#pragma unroll
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
  } else {
    m_run = m_in;
    l_run = l_in;
  }

  // m_ref is what the score accumulators are pre-loaded with (negated); it equals m_run except before
  // the first tile of a fresh row (m_run = -inf, m_ref = 0)
  float m_ref = (MODE == kSparse) ? m_run : 0.f;
  floatx16 negm;
#pragma unroll
  for (int r = 0; r < 16; ++r) negm[r] = -m_ref;

  if (MODE == kSparse) {
    // Loads complete in order and the accumulator state was requested last, with 4 * kDB load instructions, so "at most
    // that many outstanding" means: everything requested before it - queries, statistics, tile 0 - has arrived.  The
    // state itself may still be on its way while the first scores are computed (the compiler waits where it is first used).
    // (A chained block has nothing to wait for here: its first tile landed before the previous block's last barrier, and
    // the compiler waits for the queries where they are scaled.  The barrier is still needed - the tile about to be
    // requested lands where the other waves staged their output.)
    if (!chained) {
      if (kDB == 4) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    }
    lds_barrier();  // a barrier that does not wait for the loads still in flight
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // tile 0 has landed in LDS
    __syncthreads();
  }

  // per-lane LDS byte offsets.  K: row c32 (+32*kb), chunk 2*ks + half, swizzled with the row's low four bits.
  // (absolute LDS addresses into the current buffer; the 32-key half and the row steps are immediate offsets)
  const uint32_t first_buf = MODE == kSparse ? (uint32_t)cur * kTileBytes : 0u;  // (sparse) where this block's first tile lies
  // (sparse: formed per block from an opaque copy of the lane number - hoisted out of the loop over the work-group's
  // blocks, the pieces of these addresses would occupy registers throughout the tile loop)
  int lane_t = lane;
  if (MODE == kSparse) asm volatile("" : "+v"(lane_t));
  const int c32_t = lane_t & 31, half_t = lane_t >> 5;
  uint32_t k_rd[kKS];
#pragma unroll
  for (int ks = 0; ks < kKS; ++ks) k_rd[ks] = lds_addr(sm.t.k[0]) + first_buf + c32_t * kRowBytes + (((2 * ks + half_t) ^ (c32_t & 15)) << 4);
  // transposing V read i: a group of 16 lanes covers 16 head-dim columns; lane points at row r0 = 4*half + (lane%16)/4
  // (+ multiples of 8, which leave r0 = row & 7 alone), bf16 columns 32*(i&3) + 16*((lane>>4)&1) + 4*(lane&3): chunk
  // 4*(i&3) + y0 with y0 < 4, swizzled with r0 << 1 -> one offset per value of i & 3
  uint32_t v_rd[kDB];
  {
    const int r0 = 4 * half_t + ((lane_t & 15) >> 2);
    const int y0 = 2 * ((lane_t >> 4) & 1) + ((lane_t & 3) >> 1);
#pragma unroll
    for (int m = 0; m < kDB; ++m) v_rd[m] = lds_addr(sm.t.v[0]) + first_buf + r0 * kRowBytes + (((4 * m + y0) ^ (r0 << 1)) << 4) + 8 * (lane_t & 1);
  }


  // key (or list position) that accumulator register r of 32-key half kb of the tile at key0 stands for
#define AA_KEY_OF(kb, r) (key0 + 32 * (kb) + 8 * ((r) >> 2) + 4 * half + ((r) & 3))
  // causal / list-end mask of one 32-key half (only tiles on the diagonal or at the end of a list need it)
#define AA_MASK(sx, kb)                                                              \
  if (MODE != kSparse) {                                                             \
    if (key0 + 32 * (kb) + 31 > wr0) {                                               \
      _Pragma("unroll") for (int r = 0; r < 16; ++r)                                 \
        if (AA_KEY_OF(kb, r) > my_row) sx[r] = -INFINITY;                            \
    }                                                                                \
  } else if (key0 + 32 * (kb) + 32 > cnt) {                                          \
    _Pragma("unroll") for (int r = 0; r < 16; ++r)                                   \
      if (AA_KEY_OF(kb, r) >= cnt) sx[r] = -INFINITY;                                \
  }
  // row max of one half (both halves of the wave hold the same query), relative to m_ref
#define AA_ROWMAX(sx, mx)                                                            \
  {                                                                                  \
    float t0 = fmaxf(fmaxf(sx[0], sx[1]), sx[2]), t1 = fmaxf(fmaxf(sx[3], sx[4]), sx[5]);      \
    float t2 = fmaxf(fmaxf(sx[6], sx[7]), sx[8]), t3 = fmaxf(fmaxf(sx[9], sx[10]), sx[11]);    \
    float t4 = fmaxf(fmaxf(sx[12], sx[13]), sx[14]);                                 \
    t0 = fmaxf(fmaxf(t0, t1), t2);                                                   \
    t3 = fmaxf(fmaxf(t3, t4), sx[15]);                                               \
    t0 = fmaxf(t0, t3);                                                              \
    mx = max_with_other_half(t0);                                                     \
  }
#define AA_EXP2(x) ((AA_ABLATE == 1 || AA_ABLATE == 2) ? (x) : fast_exp2(x))
  // p = exp2(s) for accumulator registers 4c .. 4c+3 of one half, summed and rounded into the P^T fragment words
#define AA_EXP_CHUNK(sx, pw, sum, c)                                                 \
  {                                                                                  \
    const float e0 = AA_EXP2(sx[4 * (c) + 0]), e1 = AA_EXP2(sx[4 * (c) + 1]);        \
    const float e2 = AA_EXP2(sx[4 * (c) + 2]), e3 = AA_EXP2(sx[4 * (c) + 3]);        \
    if (AA_ABLATE != 2) { sum += e0; sum += e1; sum += e2; sum += e3; }              \
    pw[(c) >> 1][2 * ((c) & 1) + 0] = T::pack(e0, e1);                                 \
    pw[(c) >> 1][2 * ((c) & 1) + 1] = T::pack(e2, e3);                                 \
  }
  // V operand fetch i (two transposing reads): i = (kb*2 + st)*kDB + db
#define AA_V_SRC(i) (v_rd[(i) % kDB] + (uint32_t)(rd_off + (32 * ((i) / (2 * kDB)) + 16 * (((i) / kDB) & 1)) * kRowBytes))
#define AA_V_FETCH(i)                                                                                  \
  {                                                                                                    \
    vlo[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(uintptr_t)(AA_V_SRC(i)));                     \
    vhi[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(uintptr_t)(AA_V_SRC(i) + 8u * kRowBytes));    \
  }
#define AA_PV_MFMA(i, pw)                                                                              \
  {                                                                                                    \
    typedef short shortx8 __attribute__((ext_vector_type(8)));                                         \
    const shortx8 av = __builtin_shufflevector(vlo[i], vhi[i], 0, 1, 2, 3, 4, 5, 6, 7);                \
    acc[(i) % kDB] = T::mfma(*reinterpret_cast<const vec8*>(&av),                                      \
                             AA_ABLATE == 10 ? qreg[(i) % kKS] : *reinterpret_cast<const vec8*>(&pw[((i) / kDB) & 1]), acc[(i) % kDB]); \
  }
#define AA_FENCE __builtin_amdgcn_sched_barrier(0)

  // One tile.  The LDS buffer it reads (BUF) is a compile-time constant - the loop below is unrolled by two - so that
  // the buffer's offset is part of every LDS instruction's immediate offset and the read addresses are loop-invariant.
  // Sparse mode, whose tile counts can be odd, keeps one copy of the tile (BUF = -1): the buffer is i & 1 and the read
  // addresses step back and forth between the two buffers.
  int32_t buf_step = (MODE == kSparse && cur) ? -kTileBytes : kTileBytes;
  auto run_tile = [&](auto buf_const, const int i) __attribute__((always_inline)) {
    constexpr int kBuf = decltype(buf_const)::value;
    constexpr uint32_t rd_off = kBuf > 0 ? kBuf * kTileBytes : 0;  // immediate part of the LDS read addresses
    const int buf = kBuf >= 0 ? kBuf : cur;
    const int key0 = AA_TILE_KEY0(i);
    if (MODE == kSparse && i + 1 < n_tiles && ((i + 1) & (kIdxWin / kBN - 1)) == 0) {
      // tile i+1 opens the next window; everyone finished reading the old one before the last barrier
      fill_index_window((i + 1) * kBN);
      __syncthreads();
    }
    // Tile i+1 goes straight into the other buffer (every wave finished reading it before the last barrier).  Its
    // eight load instructions are spread over the first MFMAs of this tile: issued in one burst by all four waves
    // they queue up behind each other in the memory pipeline and every wave stalls for the length of the queue.
    // (the last tile fetches itself once more into the idle buffer, which keeps the instruction stream free of branches -
    // unless the work-group also pools its queries: then the eight load slots of the last tile bring the work-group's
    // 128 raw query rows into the idle buffer instead, rows 0..63 where K tiles go and rows 64..127 where V tiles go,
    // chunks in place)
    // (sparse, chained: the last tile of a block fetches the list's first tile, for the next block)
    const int i_next = i + 1 < n_tiles ? i + 1 : (feeds_next ? 0 : i);
    const int key0_next = AA_TILE_KEY0(i_next);
    const bool fetch_queries = MODE == kAnchor && pool && i + 1 == n_tiles;  // wave-uniform
    // (selects, not branches: the eight slots stay straight-line code; the base address is scalar, and the vector offset
    // is chosen once per tile and operand kind)
    const uint32_t k_voff_sel = fetch_queries ? q_voff : k_voff, v_voff_sel = fetch_queries ? q_voff : v_voff;
    uint32_t keys_next[4] = {0u, 0u, 0u, 0u};  // (sparse) row numbers of the next tile, read before the tile's first load is issued
    if (MODE == kSparse) tile_gather_keys(keys_next, sm.idx, key0_next, tid);
#define AA_FETCH_ONE(n)                                                                                               \
  if (MODE == kAnchor) {                                                                                              \
    const int j_ = (n) >> 1;                                                                                          \
    const char* kv_ = ((n) & 1) ? vbase + (uint64_t)(uint32_t)(key0_next + 16 * j_) * v_row_bytes                     \
                                : kbase + (uint64_t)(uint32_t)(key0_next + 16 * j_) * k_row_bytes;                    \
    const char* q_ = qblock + (uint64_t)(64 * ((n) & 1) + 16 * j_) * q_row_bytes;                                     \
    load16_to_lds(fetch_queries ? q_ : kv_, ((n) & 1) ? v_voff_sel : k_voff_sel,                                      \
                  (((n) & 1) ? lds_v0 : lds_k0) + (buf ^ 1) * kTileBytes + 16 * j_ * kRowBytes);                      \
  } else {                                                                                                            \
    tile_fetch_one<MODE>(n, kbase, vbase, k_row_bytes, v_row_bytes, k_col, v_col, key0_next, keys_next,               \
                         lds_k0 + (buf ^ 1) * kTileBytes, lds_v0 + (buf ^ 1) * kTileBytes, k_voff, v_voff);           \
  }
    // (a wave whose rows all lie above this tile - two of the four waves on the last tile of a causal work-group -
    // runs it fully masked: it would only wait at the barrier for the others anyway)
    {
      floatx16 s0, s1;
      vec8 ka[kNS];                // K operand of slot n = kb*kKS + ks
      shortx4 vlo[kNV], vhi[kNV];  // V operand of slot kNS + i, i = (kb*2 + st)*kDB + db
      u32x4 pw0[2], pw1[2];        // P^T fragments (bf16 pairs) of the two halves
      float mx0, mx1, sum0 = 0.f, sum1 = 0.f, shift0 = 0.f, alpha1 = 1.f;
#define AA_K_FETCH(t) ka[t] = *(const lds_vec8*)(uintptr_t)(k_rd[(t) % kKS] + (uint32_t)(rd_off + 32 * ((t) / kKS) * kRowBytes))

      // The MFMAs of a tile are slots 0 .. kNS + kNV - 1 (head dimension 128: 16 for S^T, then 16 for O^T); the operand of
      // slot n is fetched from LDS while slot n - kDist is issued.  The scheduling fences keep that distance: left
      // alone, the reads sink next to their use and every MFMA then waits out a full LDS latency.
#define AA_OPERAND_FETCH(n)                          \
  {                                                  \
    if ((n) < kNS) {                                 \
      AA_K_FETCH((n) % kNS);                         \
    } else if ((n) < kNS + kNV) {                    \
      AA_V_FETCH(((n) - kNS) % kNV)                  \
    }                                                \
  }
#define AA_S_MFMA(sx, n) sx = T::mfma(ka[n], qreg[(n) % kKS], ((n) % kKS) == 0 ? negm : sx)
      // Each half-tile product is kKS (S^T) or 2*kDB (O^T) MFMAs long; the soft-max of the other half sits between them:
      // a quarter of the MFMAs, the row max, half of the MFMAs with the four exp chunks spread over them, the last quarter.
      constexpr int kSPre = kKS / 4, kSMid = kKS / 2, kVPre = kDB / 2, kVMid = kDB;
#pragma unroll
      for (int n = 0; n < kDist; ++n) AA_OPERAND_FETCH(n)
      AA_FENCE;

      // ---- phase A: S0^T = K0 Q^T (and the next tile's eight loads) -------------------------------
#pragma unroll
      for (int n = 0; n < kKS; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_S_MFMA(s0, n);
        if (AA_ABLATE != 3) {
#pragma unroll
          for (int u = 0; u < 8 / kKS; ++u) { AA_FETCH_ONE(n * (8 / kKS) + u) }
        }
        AA_FENCE;
      }

      // ---- phase B: S1^T = K1 Q^T, with the soft-max of S0 between the MFMAs ---------------------
#pragma unroll
      for (int n = kKS; n < kKS + kSPre; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_S_MFMA(s1, n);
        AA_FENCE;
      }
      if (AA_ABLATE != 2) {
        AA_MASK(s0, 0)
        AA_ROWMAX(s0, mx0)
      } else {
        mx0 = -INFINITY;
      }
      const bool moved0 = __any(m_ref + mx0 > m_run);
      if (moved0) {
        // slow path: some row's max grew.  Lanes whose max did not move get shift 0 and alpha 1 (exact).
        // S1 is being accumulated on top of the old -m_ref and is shifted once it is complete.
        const float m_new = fmaxf(m_run, m_ref + mx0);
        const float alpha = fast_exp2(m_run - m_new);
        shift0 = m_new - m_ref;
        m_run = m_new;
        m_ref = m_new;
        l_run *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) s0[r] -= shift0;
#pragma unroll
        for (int r = 0; r < 16; ++r) negm[r] = -m_new;
#pragma unroll
        for (int db = 0; db < kDB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[db][r] *= alpha;
      }
      AA_FENCE;
#pragma unroll
      for (int n = kKS + kSPre; n < kKS + kSPre + kSMid; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_S_MFMA(s1, n);
#pragma unroll
        for (int u = 0; u < 4 / kSMid; ++u) { AA_EXP_CHUNK(s0, pw0, sum0, (n - kKS - kSPre) * (4 / kSMid) + u) }
        AA_FENCE;
      }
      l_run += sum0;
#pragma unroll
      for (int n = kKS + kSPre + kSMid; n < kNS; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_S_MFMA(s1, n);
        AA_FENCE;
      }

      // ---- phase C: O^T += V0^T P0^T, with the soft-max of S1 between the MFMAs --------------------
#pragma unroll
      for (int n = kNS; n < kNS + kVPre; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_PV_MFMA(n - kNS, pw0)
        AA_FENCE;
      }
      if (moved0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s1[r] -= shift0;
      }
      if (AA_ABLATE != 2) {
        AA_MASK(s1, 1)
        AA_ROWMAX(s1, mx1)
      } else {
        mx1 = -INFINITY;
      }
      const bool moved1 = __any(m_ref + mx1 > m_run);
      if (moved1) {
        // as above, except that O^T is rescaled only after the P0 V0 products in flight have been added
        const float m_new = fmaxf(m_run, m_ref + mx1);
        alpha1 = fast_exp2(m_run - m_new);
        const float shift = m_new - m_ref;
        m_run = m_new;
        m_ref = m_new;
        l_run *= alpha1;
#pragma unroll
        for (int r = 0; r < 16; ++r) s1[r] -= shift;
#pragma unroll
        for (int r = 0; r < 16; ++r) negm[r] = -m_new;
      }
      AA_FENCE;
#pragma unroll
      for (int n = kNS + kVPre; n < kNS + kVPre + kVMid; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_PV_MFMA(n - kNS, pw0)
#pragma unroll
        for (int u = 0; u < 4 / kVMid; ++u) { AA_EXP_CHUNK(s1, pw1, sum1, (n - kNS - kVPre) * (4 / kVMid) + u) }
        AA_FENCE;
      }
      l_run += sum1;
#pragma unroll
      for (int n = kNS + kVPre + kVMid; n < kNS + 2 * kDB; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_PV_MFMA(n - kNS, pw0)
        AA_FENCE;
      }
      if (moved1) {
#pragma unroll
        for (int db = 0; db < kDB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[db][r] *= alpha1;
      }

      // ---- phase D: O^T += V1^T P1^T ---------------------------------------------------------------
#pragma unroll
      for (int n = kNS + 2 * kDB; n < kNS + kNV; ++n) {
        AA_OPERAND_FETCH(n + kDist)
        AA_PV_MFMA(n - kNS, pw1)
        AA_FENCE;
      }
      if (AA_ABLATE == 10) {  // P is still formed: it only has to exist by the end of the tile
        asm volatile("" ::"v"(pw0[0]), "v"(pw0[1]), "v"(pw1[0]), "v"(pw1[1]));
      }
#undef AA_OPERAND_FETCH
#undef AA_S_MFMA
#undef AA_K_FETCH
    }
#undef AA_FETCH_ONE

    if (kBuf < 0) {  // the read addresses follow the tiles into the other buffer
#pragma unroll
      for (int ks = 0; ks < kKS; ++ks) k_rd[ks] += buf_step;
#pragma unroll
      for (int m = 0; m < kDB; ++m) v_rd[m] += buf_step;
      buf_step = -buf_step;
      cur ^= 1;
    }
    if (AA_ABLATE != 9) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of tile i+1 has landed in LDS
    if (AA_ABLATE != 8 && AA_ABLATE != 9) __syncthreads();
  };
  if (MODE == kSparse) {
    for (int i = 0; i < n_tiles; ++i) run_tile(std::integral_constant<int, -1>{}, i);
  } else {
    // 128 query rows and 64-key tiles: the window of a query block always holds an even number of tiles
    for (int i = 0; i < n_tiles; i += 2) {
      run_tile(std::integral_constant<int, 0>{}, i);
      run_tile(std::integral_constant<int, 1>{}, i + 1);
    }
  }
#undef AA_TILE_KEY0
#undef AA_KEY_OF
#undef AA_MASK
#undef AA_ROWMAX
#undef AA_EXP_CHUNK
#undef AA_V_SRC
#undef AA_V_FETCH
#undef AA_PV_MFMA
#undef AA_FENCE

  // ---- epilogue --------------------------------------------------------------------------------
  const float l_tot = l_run + xor32(l_run);
  if (MODE == kAnchor) {
    if (half == 0) {
      p.M_out[bh * p.n_ctx + my_row] = m_run;
      p.L_out[bh * p.n_ctx + my_row] = l_tot;
    }
    float* af = p.acc_out + ((bh * (p.n_ctx / 32) + my_row / 32) * (4 * kDB)) * 256 + lane * 4;
#pragma unroll
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        floatx4 t;
#pragma unroll
        for (int c = 0; c < 4; ++c) t[c] = acc[db][rg * 4 + c];
        __builtin_nontemporal_store(t, reinterpret_cast<floatx4*>(af + (db * 4 + rg) * 256));
      }
    if (pool) {
      // Mean-pooling of the work-group's raw queries (brought into the idle tile buffer by the last tile's load slots) and
      // of its anchors: float32 sums over block_size rows in ascending row order, divided by block_size, rounded to
      // bf16 - the same operations in the same order as pool_kernel, so the results are the same bit for bit.
      const int pbuf = n_tiles & 1;  // where the queries went
      float* mlds = reinterpret_cast<float*>(sm.t.k[pbuf ^ 1]);
      if (half == 0) mlds[wave * 32 + c32] = m_run;
      __syncthreads();
      const int bs = p.block_size, n_pooled = BM / bs;  // pooled rows of this work-group (1 for block_size 128)
      const int n_pr = p.n_ctx / bs;
      const float d = (float)bs;
      if (tid < D) {
        // waves 0 and 1: one head-dim column per thread (the ordered sum is a serial chain per column, so the shorter
        // the chain per thread the sooner the work-group retires)
        for (int pp = 0; pp < n_pooled; ++pp) {
          float a0 = 0.f;
          for (int r0 = pp * bs; r0 < (pp + 1) * bs; r0 += 16) {  // 16 rows at a time (never across the K/V halves): reads first, then the ordered sums
            const char* rowp = (r0 < 64 ? sm.t.k[pbuf] : sm.t.v[pbuf]) + (r0 & 63) * kRowBytes + 2 * tid;
            uint16_t w[16];
#pragma unroll
            for (int t = 0; t < 16; ++t) w[t] = *reinterpret_cast<const uint16_t*>(rowp + t * kRowBytes);
#pragma unroll
            for (int t = 0; t < 16; ++t) a0 += T::from16(w[t]);
          }
          reinterpret_cast<uint16_t*>(p.qbar_out)[((bh * n_pr) + R0 / bs + pp) * D + tid] = (uint16_t)(T::pack(a0 / d, 0.f) & 0xffffu);
        }
      } else if (tid >= 128 && tid - 128 < n_pooled) {
        // meanwhile, in wave 2: one thread per pooled anchor
        const int pp = tid - 128;
        float am = 0.f;
        for (int r0 = pp * bs; r0 < (pp + 1) * bs; r0 += 16) {
          float w[16];
#pragma unroll
          for (int t = 0; t < 16; t += 4) *reinterpret_cast<floatx4*>(&w[t]) = *reinterpret_cast<const floatx4*>(&mlds[r0 + t]);
#pragma unroll
          for (int t = 0; t < 16; ++t) am += w[t];
        }
        reinterpret_cast<uint16_t*>(p.abar_out)[bh * n_pr + R0 / bs + pp] = (uint16_t)(T::pack(am / d, 0.f) & 0xffffu);
      }
    }
  } else {
    // out = bf16(acc / l): the wave stages its [32][D] tile in LDS - 32 rows of the tile pitch, 16-byte chunks swizzled
    // with the row like a K tile - and writes whole rows.  The staging area is private to the wave (only a wave-local wait
    // lies between its writes and its reads) and lies in the tile buffer the loop consumed last, which every wave has
    // finished reading (the tile's closing barrier): waves 0, 1 in its K half, waves 2, 3 in its V half.  In sparse mode
    // the other buffer may already hold the next block's first tile.
    const bool more = MODE == kSparse && qb + 1 < nq;
    if (more) request_queries(my_row + BM);  // (the registers of this block's raw queries are long free)
    char* ob = (MODE == kSparse ? (wave < 2 ? sm.t.k[cur ^ 1] : sm.t.v[cur ^ 1]) + (wave & 1) * 32 * kRowBytes
                                : sm.t.k[0] + wave * 32 * kRowBytes);
    constexpr int kChunkMask = D / 8 - 1;
    // (the staging offsets are the same for every block of the work-group; computed from an opaque copy of the lane
    // number they are formed here, a few instructions per block, instead of occupying registers throughout the tile loop)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int c32_e = lane_e & 31, half_e = lane_e >> 5;
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        u32x2 w;
        w[0] = T::pack(acc[db][rg * 4 + 0] * inv, acc[db][rg * 4 + 1] * inv);
        w[1] = T::pack(acc[db][rg * 4 + 2] * inv, acc[db][rg * 4 + 3] * inv);
        *reinterpret_cast<u32x2*>(ob + c32_e * kRowBytes + (((4 * db + rg) ^ (c32_e & kChunkMask)) << 4) + 8 * half_e) = w;
      }
    // the accumulator registers are free: the next block's state can be on its way while this block's output leaves
    if (more && list_chains) request_state(my_row + BM);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave's LDS writes are done (and stay above this line)
    uint16_t* op = p.out + b * p.o_sb + hq * p.o_sh;
    constexpr int kLanesPerRow = D / 8, kRowsPerStore = 64 / kLanesPerRow;  // a row is D/8 pieces of 16 bytes
#pragma unroll
    for (int it = 0; it < 32 / kRowsPerStore; ++it) {
      const int r = it * kRowsPerStore + lane_e / kLanesPerRow, c = lane_e % kLanesPerRow;
      const u32x4 w = *reinterpret_cast<const u32x4*>(ob + r * kRowBytes + ((c ^ (r & kChunkMask)) << 4));
      __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(op + (int64_t)(wr0 + r) * p.o_sn + 8 * c));
    }
    chained = more && list_chains;
    have_queries = more;
  }
  }  // query blocks of the work-group
}

#ifndef AA_SPARSE_QBLOCKS
#define AA_SPARSE_QBLOCKS 4  // 128-row query blocks a stage-3 work-group handles one after the other (when the big block allows)
#endif

template <int MODE>
static hipError_t launch(const FlashArgs& args, hipStream_t stream) {
  FlashArgs a = args;
  a.q_blocks_per_wg = 1;
  if (MODE == kSparse) {
    const int per_big_block = a.big_block / 128;  // even for every supported geometry
    a.q_blocks_per_wg = per_big_block % AA_SPARSE_QBLOCKS == 0 ? AA_SPARSE_QBLOCKS : (per_big_block % 2 == 0 ? 2 : 1);
  }
  const dim3 grid((uint32_t)a.batch * a.n_q_heads * (a.n_ctx / (128 * a.q_blocks_per_wg))), block(256);
  if (a.head_dim == 128) {
    if (a.dtype == 0) hipLaunchKernelGGL((flash_kernel<MODE, Bf16, 128>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((flash_kernel<MODE, F16, 128>), grid, block, 0, stream, a);
  } else {  // 64: the C-ABI layer admits nothing else
    if (a.dtype == 0) hipLaunchKernelGGL((flash_kernel<MODE, Bf16, 64>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((flash_kernel<MODE, F16, 64>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

hipError_t launch_flash(const FlashArgs& a, int mode, hipStream_t stream) {
  if (mode == kAnchor) return launch<kAnchor>(a, stream);
  if (mode == kSparse) return launch<kSparse>(a, stream);
  return launch<kDense>(a, stream);
}

}  // namespace aa
