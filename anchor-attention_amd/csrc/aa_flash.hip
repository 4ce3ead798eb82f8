// MFMA flash-attention core for gfx950, used three ways:
//   kAnchor : stage 1 - windowed causal attention over [0,S) U [bb*S, r]; emits M, L, Acc
//   kSparse : stage 3 - resumes from (M, L, Acc) over K/V rows gathered at selected indices
//   kDense  : plain causal attention (baseline)
//
// Formulation.  A wave owns 32*QB query rows and computes the TRANSPOSED score tile
//   S^T[key][query] = K[key][:] . Q[query][:]      (MFMA A = K rows from LDS, B = Q from registers)
// so that in the 32x32 accumulator layout a lane holds one query column: the soft-max statistics
// of a query are then plain per-lane scalars (one exchange with the lane 32 positions away
// completes the row max).  The second product is computed transposed as well,
//   O^T[d][query] += V^T[d][key] . P^T[key][query]  (A = V^T from LDS, B = P^T straight from the
// S^T accumulator registers, rounded to bf16) - P never travels through LDS.
// The contraction slot k = 8*(lane/32) + e of MFMA step s of key block kb is fed from accumulator
// register 8*s + e, i.e. key 32*kb + 16*s + 8*(e/4) + 4*(lane/32) + e%4.  V^T is therefore
// written to LDS with bits 2 and 3 of the key index swapped ("slot" order), which makes every
// lane's eight V^T operands one contiguous 16-byte LDS read.
//
// Work-group = 4 waves = 128*QB query rows; keys are consumed 64 at a time through a
// double-buffered LDS tile (K row-major, padded to 272-byte rows; V^T padded to 144-byte rows, both
// conflict-free for 16-byte reads by 8 consecutive lanes).
#include "aa_common.h"
#include "aa_kernels.h"

namespace aa {

constexpr int kBN = 64;          // keys per LDS tile
constexpr int kKsStride = 136;   // bf16 per K row in LDS
constexpr int kVtStride = 72;    // bf16 per V^T row in LDS
constexpr int kOsStride = 136;   // bf16 per output-staging row in LDS

enum FlashMode : int { kAnchor = 0, kSparse = 1, kDense = 2 };

template <int QB>
struct FlashSmem {
  union {
    struct {
      __bf16 ks[2][kBN * kKsStride];
      __bf16 vt[2][128 * kVtStride];
    } t;
    __bf16 os[4][32 * QB * kOsStride];  // epilogue staging, reuses the tile space
  };
};

__device__ __forceinline__ void scale_q8(const uint4& raw, float sm_scale, int scale_mode, bf16x8& dst) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t o[4];
  if (scale_mode == 0) {  // bf16 chain: bf16(bf16(q * bf16(sm_scale)) * bf16(log2e))
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
  uint4 packed = {o[0], o[1], o[2], o[3]};
  dst = *reinterpret_cast<bf16x8*>(&packed);
}

template <int QB, int MODE>
__global__ void __launch_bounds__(256) flash_kernel(const FlashArgs p) {
  __shared__ __attribute__((aligned(16))) FlashSmem<QB> sm;
  constexpr int BM = 128 * QB;

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
  if (MODE != kSparse) qblk = n_qblk - 1 - qblk;  // longest rows first
  const int R0 = qblk * BM;
  const int S = p.big_block;
  const int bb = R0 / S;
  const int wr0 = R0 + wave * 32 * QB;
  const int64_t bh = (int64_t)b * p.n_q_heads + hq;

  const __bf16* qp = p.q + b * p.q_sb + hq * p.q_sh;
  const __bf16* kp = p.k + b * p.k_sb + kvh * p.k_sh;
  const __bf16* vp = p.v + b * p.v_sb + kvh * p.v_sh;

  // ---- queries: B operand, pre-scaled into the exp2 domain -----------------------------------
  bf16x8 qreg[QB][8];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const __bf16* row = qp + (int64_t)(wr0 + 32 * qb + c32) * p.q_sn + 8 * half;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const uint4 raw = *reinterpret_cast<const uint4*>(row + 16 * ks);
      scale_q8(raw, p.sm_scale, MODE == kAnchor ? p.scale_mode : 1, qreg[qb][ks]);
    }
  }

  // ---- running state -------------------------------------------------------------------------
  float m_run[QB], l_run[QB];
  floatx16 acc[4][QB];
  if (MODE == kSparse) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int row = wr0 + 32 * qb + c32;
      m_run[qb] = p.M[bh * p.n_ctx + row];
      l_run[qb] = half == 0 ? p.L[bh * p.n_ctx + row] : 0.f;  // halves are summed at the end
      const float* af = p.acc_frag + ((bh * (p.n_ctx / 32) + row / 32) * 16) * 256 + lane * 4;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const floatx4 t = *reinterpret_cast<const floatx4*>(af + (db * 4 + rg) * 256);
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[db][qb][rg * 4 + c] = t[c];
        }
    }
  } else {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      m_run[qb] = -INFINITY;
      l_run[qb] = 0.f;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[db][qb][r] = 0.f;
    }
  }

  // ---- tile schedule -------------------------------------------------------------------------
  int n_tiles, n_init = 0, cnt = 0;
  const int32_t* cbase = nullptr;
  if (MODE == kAnchor) {
    n_init = min(S, R0 + BM) / kBN;
    n_tiles = n_init + (bb >= 1 ? (R0 + BM - bb * S) / kBN : 0);
  } else if (MODE == kDense) {
    n_tiles = (R0 + BM) / kBN;
  } else {
    cnt = p.counts[bh * (p.n_ctx / S) + bb];
    cbase = p.coords + bh * p.coords_per_head + coords_tri(bb, S, p.block_size);
    n_tiles = (cnt + kBN - 1) / kBN;
  }
  auto tile_key0 = [&](int i) -> int {
    if (MODE == kAnchor) return i < n_init ? i * kBN : bb * S + (i - n_init) * kBN;
    return i * kBN;  // dense: key index; sparse: position in the index list
  };

  uint4 kreg[4];
  uint32_t vreg[4][4];
  auto issue_loads = [&](int i) {
    const int key0 = tile_key0(i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = tid + 256 * j, row = id >> 4, c = id & 15;
      int64_t key = key0 + row;
      if (MODE == kSparse) key = (key0 + row < cnt) ? cbase[key0 + row] : 0;
      kreg[j] = *reinterpret_cast<const uint4*>(kp + key * p.k_sn + 8 * c);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int g4 = 4 * (wave + 4 * j);  // first of the four keys this wave transposes
      int64_t keys[4];
      if (MODE == kSparse) {
        const int4 ids = *reinterpret_cast<const int4*>(cbase + key0 + g4);
        keys[0] = key0 + g4 + 0 < cnt ? ids.x : 0;
        keys[1] = key0 + g4 + 1 < cnt ? ids.y : 0;
        keys[2] = key0 + g4 + 2 < cnt ? ids.z : 0;
        keys[3] = key0 + g4 + 3 < cnt ? ids.w : 0;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) keys[e] = key0 + g4 + e;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) vreg[j][e] = *reinterpret_cast<const uint32_t*>(vp + keys[e] * p.v_sn + 2 * lane);
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = tid + 256 * j, row = id >> 4, c = id & 15;
      *reinterpret_cast<uint4*>(&sm.t.ks[buf][row * kKsStride + 8 * c]) = kreg[j];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gq = wave + 4 * j;                                        // key group (4 keys)
      const int slot0 = 4 * ((gq & ~3) | ((gq & 1) << 1) | ((gq >> 1) & 1));  // bits 2,3 of the key swapped
      const uint32_t* d = vreg[j];
      uint2 lo, hi;
      lo.x = (d[0] & 0xffffu) | (d[1] << 16);
      lo.y = (d[2] & 0xffffu) | (d[3] << 16);
      hi.x = (d[0] >> 16) | (d[1] & 0xffff0000u);
      hi.y = (d[2] >> 16) | (d[3] & 0xffff0000u);
      *reinterpret_cast<uint2*>(&sm.t.vt[buf][(2 * lane) * kVtStride + slot0]) = lo;
      *reinterpret_cast<uint2*>(&sm.t.vt[buf][(2 * lane + 1) * kVtStride + slot0]) = hi;
    }
  };

  if (n_tiles > 0) {
    issue_loads(0);
    store_tile(0);
  }
  __syncthreads();

  for (int i = 0; i < n_tiles; ++i) {
    const int buf = i & 1;
    const int key0 = tile_key0(i);
    if (i + 1 < n_tiles) issue_loads(i + 1);

    // a wave whose rows all lie above this tile (causal) has nothing to do
    const bool wave_active = (MODE == kSparse) || (key0 <= wr0 + 32 * QB - 1);
    if (wave_active) {
      // ---- S^T = K Q^T ------------------------------------------------------------------------
      floatx16 s[2][QB];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[kb][qb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(&sm.t.ks[buf][(32 * kb + c32) * kKsStride + 16 * ks + 8 * half]);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) s[kb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[qb][ks], s[kb][qb], 0, 0, 0);
        }

      // ---- masks ------------------------------------------------------------------------------
      if (MODE != kSparse) {
        if (key0 + kBN - 1 > wr0) {  // tile touches the diagonal of this wave
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int key = key0 + 32 * kb + 8 * (r >> 2) + 4 * half + (r & 3);
                if (key > wr0 + 32 * qb + c32) s[kb][qb][r] = -INFINITY;
              }
        }
      } else if (key0 + kBN > cnt) {  // last, partly filled chunk of the index list
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int pos = key0 + 32 * kb + 8 * (r >> 2) + 4 * half + (r & 3);
              if (pos >= cnt) s[kb][qb][r] = -INFINITY;
            }
      }

      // ---- online soft-max (exp2 domain) ------------------------------------------------------
      bf16x8 pfrag[2][QB][2];
      float alpha[QB];
      bool rescale = false;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        float mx = s[0][qb][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kb][qb][r]);
        mx = fmaxf(mx, xor32(mx));
        const float m_new = fmaxf(m_run[qb], mx);
        alpha[qb] = fast_exp2(m_run[qb] - m_new);
        rescale |= (m_new != m_run[qb]);
        m_run[qb] = m_new;
        float sum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          float pv[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            pv[r] = fast_exp2(s[kb][qb][r] - m_new);
            sum += pv[r];
          }
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            uint4 w;
            w.x = pack_bf16(pv[8 * st + 0], pv[8 * st + 1]);
            w.y = pack_bf16(pv[8 * st + 2], pv[8 * st + 3]);
            w.z = pack_bf16(pv[8 * st + 4], pv[8 * st + 5]);
            w.w = pack_bf16(pv[8 * st + 6], pv[8 * st + 7]);
            pfrag[kb][qb][st] = *reinterpret_cast<bf16x8*>(&w);
          }
        }
        l_run[qb] = l_run[qb] * alpha[qb] + sum;
      }
      // multiplying by alpha == 1 is exact, so the rescale is skipped when no lane's max moved
      if (__any(rescale)) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[db][qb][r] *= alpha[qb];
      }

      // ---- O^T += V^T P^T ---------------------------------------------------------------------
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            const bf16x8 a = *reinterpret_cast<const bf16x8*>(&sm.t.vt[buf][(32 * db + c32) * kVtStride + 32 * kb + 16 * st + 8 * half]);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) acc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pfrag[kb][qb][st], acc[db][qb], 0, 0, 0);
          }
    }

    if (i + 1 < n_tiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue --------------------------------------------------------------------------------
  if (MODE == kAnchor) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int row = wr0 + 32 * qb + c32;
      const float l_tot = l_run[qb] + xor32(l_run[qb]);
      if (half == 0) {
        p.M_out[bh * p.n_ctx + row] = m_run[qb];
        p.L_out[bh * p.n_ctx + row] = l_tot;
      }
      float* af = p.acc_out + ((bh * (p.n_ctx / 32) + row / 32) * 16) * 256 + lane * 4;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          floatx4 t;
#pragma unroll
          for (int c = 0; c < 4; ++c) t[c] = acc[db][qb][rg * 4 + c];
          *reinterpret_cast<floatx4*>(af + (db * 4 + rg) * 256) = t;
        }
    }
  } else {
    // out = bf16(acc / l): stage the wave's [32*QB][128] tile in LDS, then write whole rows
    __bf16* os = sm.os[wave];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float l_tot = l_run[qb] + xor32(l_run[qb]);
      const float inv = 1.0f / l_tot;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          uint2 w;
          w.x = pack_bf16(acc[db][qb][rg * 4 + 0] * inv, acc[db][qb][rg * 4 + 1] * inv);
          w.y = pack_bf16(acc[db][qb][rg * 4 + 2] * inv, acc[db][qb][rg * 4 + 3] * inv);
          *reinterpret_cast<uint2*>(&os[(32 * qb + c32) * kOsStride + 32 * db + 8 * rg + 4 * half]) = w;
        }
    }
    __syncthreads();
    __bf16* op = p.out + b * p.o_sb + hq * p.o_sh;
#pragma unroll
    for (int it = 0; it < 8 * QB; ++it) {
      const int r = it * 4 + (lane >> 4), c = lane & 15;
      const uint4 w = *reinterpret_cast<const uint4*>(&os[r * kOsStride + 8 * c]);
      *reinterpret_cast<uint4*>(op + (int64_t)(wr0 + r) * p.o_sn + 8 * c) = w;
    }
  }
}

template <int QB, int MODE>
static hipError_t launch(const FlashArgs& a, hipStream_t stream) {
  const int BM = 128 * QB;
  const uint32_t grid = (uint32_t)a.batch * a.n_q_heads * (a.n_ctx / BM);
  hipLaunchKernelGGL((flash_kernel<QB, MODE>), dim3(grid), dim3(256), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_flash(const FlashArgs& a, int mode, int qb, hipStream_t stream) {
  if (qb == 1) {
    if (mode == kAnchor) return launch<1, kAnchor>(a, stream);
    if (mode == kSparse) return launch<1, kSparse>(a, stream);
    return launch<1, kDense>(a, stream);
  }
  if (mode == kAnchor) return launch<2, kAnchor>(a, stream);
  if (mode == kSparse) return launch<2, kSparse>(a, stream);
  return launch<2, kDense>(a, stream);
}

}  // namespace aa
