// Internal launch interfaces between the C-ABI layer and the kernel translation units.
#pragma once
#include "aa_common.h"

namespace aa {

struct FlashArgs {
  const uint16_t* q; int64_t q_sb, q_sh, q_sn;
  const uint16_t* k; int64_t k_sb, k_sh, k_sn;
  const uint16_t* v; int64_t v_sb, v_sh, v_sn;
  uint16_t* out;     int64_t o_sb, o_sh, o_sn;   // sparse / dense modes
  float* M_out; float* L_out; float* acc_out;  // anchor mode
  // anchor mode, optional (both or neither; block_size <= 128): the work-group also mean-pools its 128 raw query rows
  // and anchors into qbar [B,Hq,N/block_size,head_dim] and abar [B,Hq,N/block_size], bit for bit what pool_kernel computes
  uint16_t* qbar_out; uint16_t* abar_out;
  const float* M; const float* L; const float* acc_frag;  // sparse mode (resume state)
  const int32_t* coords; const int32_t* counts; int64_t coords_per_head;  // sparse mode
  int batch, n_q_heads, n_kv_heads, n_ctx;
  int head_dim;  // 128 or 64
  int big_block, block_size;
  float sm_scale; int scale_mode;
  int q_blocks_per_wg;  // set by the launcher
  int dtype;            // AA_DTYPE_BF16 / AA_DTYPE_F16: what the 16-bit elements of q, k, v, out, qbar, abar are
};

// mode: 0 anchor (stage 1), 1 sparse (stage 3), 2 dense causal
hipError_t launch_flash(const FlashArgs& a, int mode, hipStream_t stream);

struct PoolArgs {
  const uint16_t* q; int64_t q_sb, q_sh, q_sn;
  const float* M;
  uint16_t* qbar; uint16_t* abar;
  int batch, n_q_heads, n_ctx, block_size;
  int head_dim;  // 128 or 64
  int dtype;
};
hipError_t launch_pool(const PoolArgs& a, hipStream_t stream);

struct SelectArgs {
  const uint16_t* qbar; const uint16_t* abar;
  const uint16_t* k; int64_t k_sb, k_sh, k_sn;
  float* thr;  // per pooled row: smallest raw dot product that passes the selection test
  uint32_t* mask; int32_t* coords; int32_t* counts; int64_t coords_per_head;
  int batch, n_q_heads, n_kv_heads, n_ctx;
  int big_block, block_size;
  float scale2, theta_log2;
  // candidate keys of big block bb: key_lo <= j < bb*S - key_slack (as run: block_size and block_size; intended: S and 0)
  int key_lo, key_slack;
  int head_dim;  // 128 or 64
  int dtype;
};
hipError_t launch_select_thresholds(const SelectArgs& a, hipStream_t stream);
hipError_t launch_select_scores(const SelectArgs& a, hipStream_t stream);
hipError_t launch_select_compact(const SelectArgs& a, hipStream_t stream);

}  // namespace aa
