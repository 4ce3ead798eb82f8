// C ABI of the AnchorAttention gfx950 kernels: argument validation, scratch carving, launches.
// Declarations and their reference counterparts: include/anchor_attn_hip.h.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/anchor_attn_hip.h"
#include "aa_common.h"
#include "aa_kernels.h"

// Device memory for aa_stage2_select_static(): the stage-2 bitmask and thresholds of callers that cannot
// allocate.  Every GPU the library's code object is loaded on holds its own copy until the process ends.  In host
// code this name only stands for the symbol; the memory's address on a device comes from hipGetSymbolAddress().
static __device__ __align__(256) unsigned char scratch[AA_STATIC_SCRATCH_BYTES];

namespace aa {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

namespace {

struct Dims {
  int batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step;
};

// Checks every entry point shares: head counts, head_dim, and the sizes one launch can address.
int check_common_dims(const Dims& d, const char* who) {
  if (d.batch <= 0 || d.n_q_heads <= 0 || d.n_kv_heads <= 0 || d.n_ctx <= 0) {
    set_error("%s: batch, head counts and n_ctx must be positive (got %d, %d, %d, %d)", who, d.batch, d.n_q_heads, d.n_kv_heads, d.n_ctx);
    return AA_EBADARG;
  }
  if (d.n_q_heads % d.n_kv_heads != 0) {
    set_error("%s: n_kv_heads (%d) must divide n_q_heads (%d)", who, d.n_kv_heads, d.n_q_heads);
    return AA_EBADARG;
  }
  if (d.head_dim != 128 && d.head_dim != 64) {
    set_error("%s: head_dim %d is not supported (128 or 64)", who, d.head_dim);
    return AA_EUNSUPPORTED;
  }
  if (d.n_ctx % 128 != 0) {
    set_error("%s: n_ctx %d must be a multiple of 128", who, d.n_ctx);
    return AA_EUNSUPPORTED;
  }
  if (d.n_ctx > (1 << 20)) {
    set_error("%s: n_ctx %d is larger than 1048576", who, d.n_ctx);
    return AA_EUNSUPPORTED;
  }
  if ((int64_t)d.batch * d.n_q_heads * (d.n_ctx / 128) > 0x7fffffffLL) {
    set_error("%s: problem too large for one launch", who);
    return AA_EUNSUPPORTED;
  }
  return AA_OK;
}

// The common checks plus the big-block geometry of the three AnchorAttention stages.
int check_dims(const Dims& d, const char* who) {
  if (int rc = check_common_dims(d, who)) return rc;
  if (d.block_size != 16 && d.block_size != 32 && d.block_size != 64 && d.block_size != 128 && d.block_size != 256) {
    set_error("%s: block_size %d is not supported (16, 32, 64, 128 or 256)", who, d.block_size);
    return AA_EUNSUPPORTED;
  }
  if (d.step != 16 && d.step != 32) {
    set_error("%s: step %d is not supported (16 or 32)", who, d.step);
    return AA_EUNSUPPORTED;
  }
  if (d.n_ctx % (d.block_size * d.step) != 0) {
    set_error("%s: n_ctx %d is not a multiple of block_size*step = %d", who, d.n_ctx, d.block_size * d.step);
    return AA_EUNSUPPORTED;
  }
  return AA_OK;
}

int check_tensor(const void* ptr, int64_t sb, int64_t sh, int64_t sn, int n_ctx, int head_dim, const char* who, const char* name) {
  if (ptr == nullptr) {
    set_error("%s: %s is NULL", who, name);
    return AA_EBADARG;
  }
  if ((reinterpret_cast<uintptr_t>(ptr) & 15u) != 0 || (sb % 8) != 0 || (sh % 8) != 0 || (sn % 8) != 0) {
    set_error("%s: %s must be 16-byte aligned with strides that are multiples of 8 elements (ptr=%p strides=%lld,%lld,%lld)", who, name, ptr, (long long)sb, (long long)sh, (long long)sn);
    return AA_EMISALIGNED;
  }
  if (sn < head_dim) {
    set_error("%s: %s row stride %lld is smaller than head_dim", who, name, (long long)sn);
    return AA_EBADARG;
  }
  if (sn > (int64_t)1 << 14) {  // the kernels address rows of one head with 32-bit byte offsets
    set_error("%s: %s row stride %lld is larger than 16384 elements", who, name, (long long)sn);
    return AA_EUNSUPPORTED;
  }
  if ((int64_t)n_ctx * sn * 2 > (int64_t)0xffffffffLL) {
    set_error("%s: %s spans %lld bytes per head (n_ctx %d x row stride %lld elements); the kernels address one head with 32-bit byte offsets",
              who, name, (long long)n_ctx * sn * 2, n_ctx, (long long)sn);
    return AA_EUNSUPPORTED;
  }
  return AA_OK;
}

int check_ptr(const void* ptr, const char* who, const char* name) {
  if (ptr == nullptr) {
    set_error("%s: %s is NULL", who, name);
    return AA_EBADARG;
  }
  if ((reinterpret_cast<uintptr_t>(ptr) & 15u) != 0) {
    set_error("%s: %s must be 16-byte aligned", who, name);
    return AA_EMISALIGNED;
  }
  return AA_OK;
}

int check_dtype(int dtype, const char* who) {
  if (dtype != AA_DTYPE_BF16 && dtype != AA_DTYPE_F16) {
    set_error("%s: dtype %d is neither AA_DTYPE_BF16 nor AA_DTYPE_F16", who, dtype);
    return AA_EBADARG;
  }
  return AA_OK;
}

int check_launch(hipError_t e, const char* who) {
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", who, hipGetErrorString(e));
    return AA_ELAUNCH;
  }
  return AA_OK;
}

hipError_t run_flash(const FlashArgs& a, int mode, hipStream_t stream) {
  return launch_flash(a, mode, stream);
}

size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

// Address of `scratch` on the current device, looked up once per device (with that device current) and kept.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** out, const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: cannot tell the current device (%s, device %d)", who, hipGetErrorString(e), dev);
    return AA_ELAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
      return AA_ELAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return AA_OK;
}

struct Workspace {
  size_t M, L, acc, qbar, abar, mask, coords, counts, total;
};

Workspace carve(int batch, int hq, int n_ctx, int head_dim, int block_size, int step) {
  Workspace w;
  const size_t bh = (size_t)batch * hq;
  size_t off = 0;
  w.M = off;      off += align256(bh * n_ctx * 4);
  w.L = off;      off += align256(bh * n_ctx * 4);
  w.acc = off;    off += align256(bh * n_ctx * head_dim * 4);
  w.qbar = off;   off += align256(bh * (n_ctx / block_size) * head_dim * 2);
  w.abar = off;   off += align256(bh * (n_ctx / block_size) * 2);
  w.mask = off;   off += align256((size_t)aa_mask_words(batch, hq, n_ctx, block_size, step) * 4);
  w.coords = off; off += align256(bh * (size_t)aa_coords_entries_per_head(n_ctx, block_size, step) * 4);
  w.counts = off; off += align256(bh * (n_ctx / (block_size * step)) * 4);
  w.total = off;
  return w;
}

}  // namespace
}  // namespace aa

using namespace aa;

extern "C" {

#ifndef AA_ABLATE
#define AA_ABLATE 0
#endif
// (1000 + n marks a timing-only build that leaves part of a kernel out, see aa_flash.hip; never a product)
int aa_version(void) { return AA_ABLATE ? 1000 + AA_ABLATE : 3; }

const char* aa_last_error(void) { return g_error; }

int64_t aa_coords_entries_per_head(int n_ctx, int block_size, int step) {
  const int64_t S = (int64_t)block_size * step;
  return coords_tri(n_ctx / S, S, block_size);
}

int64_t aa_coords_offset(int big_block, int block_size, int step) {
  return coords_tri(big_block, (int64_t)block_size * step, block_size);
}

static int64_t mask_bit_words(int batch, int n_q_heads, int n_ctx, int block_size, int step) {
  return (int64_t)batch * n_q_heads * (n_ctx / (block_size * step)) * (n_ctx / 128) * 4;
}

int64_t aa_mask_words(int batch, int n_q_heads, int n_ctx, int block_size, int step) {
  // key bitmask followed by one float32 threshold per pooled row
  return mask_bit_words(batch, n_q_heads, n_ctx, block_size, step) + (int64_t)batch * n_q_heads * (n_ctx / block_size);
}

size_t aa_workspace_bytes(int batch, int n_q_heads, int n_ctx, int head_dim, int block_size, int step) {
  if (batch <= 0 || n_q_heads <= 0 || n_ctx <= 0 || (head_dim != 128 && head_dim != 64) || block_size <= 0 || step <= 0) return 0;
  return carve(batch, n_q_heads, n_ctx, head_dim, block_size, step).total;
}

// Stage 1; with qbar/abar non-null (block_size <= 128) the kernel also emits the pooled queries and anchors.
static int stage1_impl(const char* who, const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                       const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                       const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                       float* M, float* L, float* acc_frag, void* qbar, void* abar,
                       int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                       int block_size, int step, float sm_scale, int scale_mode, int dtype, void* stream) {
  int rc;
  if ((rc = check_dims({batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step}, who))) return rc;
  if ((rc = check_dtype(dtype, who))) return rc;
  if ((rc = check_tensor(q, q_sb, q_sh, q_sn, n_ctx, head_dim, who, "q"))) return rc;
  if ((rc = check_tensor(k, k_sb, k_sh, k_sn, n_ctx, head_dim, who, "k"))) return rc;
  if ((rc = check_tensor(v, v_sb, v_sh, v_sn, n_ctx, head_dim, who, "v"))) return rc;
  if ((rc = check_ptr(M, who, "M")) || (rc = check_ptr(L, who, "L")) || (rc = check_ptr(acc_frag, who, "acc_frag"))) return rc;
  if (scale_mode != AA_SCALE_BF16_CHAIN && scale_mode != AA_SCALE_FP32) {
    set_error("%s: unknown scale_mode %d", who, scale_mode);
    return AA_EBADARG;
  }
  FlashArgs a = {};
  a.q = (const uint16_t*)q; a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn;
  a.k = (const uint16_t*)k; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.v = (const uint16_t*)v; a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn;
  a.M_out = M; a.L_out = L; a.acc_out = acc_frag;
  a.qbar_out = (uint16_t*)qbar; a.abar_out = (uint16_t*)abar;
  a.batch = batch; a.n_q_heads = n_q_heads; a.n_kv_heads = n_kv_heads; a.n_ctx = n_ctx; a.head_dim = head_dim;
  a.big_block = block_size * step; a.block_size = block_size;
  a.sm_scale = sm_scale; a.scale_mode = scale_mode; a.dtype = dtype;
  return check_launch(run_flash(a, 0, (hipStream_t)stream), who);
}

int aa_stage1_anchor_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         float* M, float* L, float* acc_frag,
                         int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                         int block_size, int step, float sm_scale, int scale_mode, int dtype, void* stream) {
  return stage1_impl("aa_stage1_anchor_fwd", q, q_sb, q_sh, q_sn, k, k_sb, k_sh, k_sn, v, v_sb, v_sh, v_sn, M, L, acc_frag, nullptr,
                     nullptr, batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step, sm_scale, scale_mode, dtype, stream);
}

int aa_pool_q_anchor(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn, const float* M,
                     void* qbar, void* abar,
                     int batch, int n_q_heads, int n_ctx, int head_dim, int block_size, int dtype, void* stream) {
  const char* who = "aa_pool_q_anchor";
  int rc;
  if ((rc = check_dtype(dtype, who))) return rc;
  if ((rc = check_dims({batch, n_q_heads, n_q_heads, n_ctx, head_dim, block_size, 16}, who))) return rc;
  if ((rc = check_tensor(q, q_sb, q_sh, q_sn, n_ctx, head_dim, who, "q"))) return rc;
  if ((rc = check_ptr(M, who, "M")) || (rc = check_ptr(qbar, who, "qbar")) || (rc = check_ptr(abar, who, "abar"))) return rc;
  PoolArgs a = {};
  a.q = (const uint16_t*)q; a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn;
  a.M = M; a.qbar = (uint16_t*)qbar; a.abar = (uint16_t*)abar;
  a.batch = batch; a.n_q_heads = n_q_heads; a.n_ctx = n_ctx; a.block_size = block_size; a.head_dim = head_dim; a.dtype = dtype;
  return check_launch(launch_pool(a, (hipStream_t)stream), who);
}

int aa_stage2_select(const void* qbar, const void* abar,
                     const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                     uint32_t* mask_ws, int32_t* coords, int32_t* counts,
                     int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                     int block_size, int step, double sm_scale, float theta_log2, int geometry, int dtype, void* stream) {
  const char* who = "aa_stage2_select";
  int rc;
  if ((rc = check_dtype(dtype, who))) return rc;
  if (geometry != AA_GEOMETRY_AS_RUN && geometry != AA_GEOMETRY_INTENDED) {
    set_error("%s: geometry %d is neither AA_GEOMETRY_AS_RUN nor AA_GEOMETRY_INTENDED", who, geometry);
    return AA_EBADARG;
  }
  if ((rc = check_dims({batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step}, who))) return rc;
  if ((rc = check_tensor(k, k_sb, k_sh, k_sn, n_ctx, head_dim, who, "k"))) return rc;
  if ((rc = check_ptr(qbar, who, "qbar")) || (rc = check_ptr(abar, who, "abar")) || (rc = check_ptr(mask_ws, who, "mask_ws")) ||
      (rc = check_ptr(coords, who, "coords")) || (rc = check_ptr(counts, who, "counts")))
    return rc;
  SelectArgs a = {};
  a.qbar = (const uint16_t*)qbar; a.abar = (const uint16_t*)abar;
  a.k = (const uint16_t*)k; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.mask = mask_ws; a.coords = coords; a.counts = counts;
  a.thr = reinterpret_cast<float*>(mask_ws + mask_bit_words(batch, n_q_heads, n_ctx, block_size, step));
  a.coords_per_head = aa_coords_entries_per_head(n_ctx, block_size, step);
  a.batch = batch; a.n_q_heads = n_q_heads; a.n_kv_heads = n_kv_heads; a.n_ctx = n_ctx; a.head_dim = head_dim;
  a.big_block = block_size * step; a.block_size = block_size;
  a.scale2 = (float)(sm_scale * 1.44269504);  // double product, then float32, as the definition does
  a.theta_log2 = theta_log2;
  a.dtype = dtype;
  a.key_lo = geometry == AA_GEOMETRY_AS_RUN ? block_size : block_size * step;
  a.key_slack = geometry == AA_GEOMETRY_AS_RUN ? block_size : 0;
  // the score kernel numbers (query head of the KV group, big block) pairs with 16 bits and addresses the pooled
  // queries with 32-bit byte offsets
  if ((int64_t)(n_q_heads / n_kv_heads) * (n_ctx / (block_size * step)) >= 65536 ||
      (int64_t)batch * n_q_heads * (n_ctx / block_size) * 2 * head_dim > 0xffffffffLL) {
    set_error("%s: too many (head, big block) pairs or pooled rows for one launch (heads per KV head %d, big blocks %d, pooled rows %lld)",
              who, n_q_heads / n_kv_heads, n_ctx / (block_size * step), (long long)batch * n_q_heads * (n_ctx / block_size));
    return AA_EUNSUPPORTED;
  }
  if ((rc = check_launch(launch_select_thresholds(a, (hipStream_t)stream), who))) return rc;
  if ((rc = check_launch(launch_select_scores(a, (hipStream_t)stream), who))) return rc;
  return check_launch(launch_select_compact(a, (hipStream_t)stream), who);
}

int aa_stage2_select_static(const void* qbar, const void* abar,
                            const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                            int32_t* coords, int32_t* counts,
                            int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                            int block_size, int step, double sm_scale, float theta_log2, int geometry, int dtype, void* stream) {
  const char* who = "aa_stage2_select_static";
  int rc;
  if ((rc = check_dims({batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step}, who))) return rc;
  const int64_t need = aa_mask_words(batch, n_q_heads, n_ctx, block_size, step) * 4;
  if (need > (int64_t)AA_STATIC_SCRATCH_BYTES) {
    set_error("%s: this problem needs %lld bytes of stage-2 scratch, the static scratch holds %lld (batch*n_q_heads*n_ctx^2 too "
              "large: use aa_stage2_select with a caller-provided buffer)", who, (long long)need, (long long)AA_STATIC_SCRATCH_BYTES);
    return AA_EUNSUPPORTED;
  }
  void* ws = nullptr;
  if ((rc = static_scratch(&ws, who))) return rc;
  // from here on exactly aa_stage2_select: same checks, same kernels, the scratch pointer as an ordinary argument
  return aa_stage2_select(qbar, abar, k, k_sb, k_sh, k_sn, static_cast<uint32_t*>(ws), coords, counts, batch, n_q_heads,
                          n_kv_heads, n_ctx, head_dim, block_size, step, sm_scale, theta_log2, geometry, dtype, stream);
}

int aa_stage3_sparse_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         const int32_t* coords, const int32_t* counts,
                         const float* M, const float* L, const float* acc_frag,
                         void* out, int64_t o_sb, int64_t o_sh, int64_t o_sn,
                         int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                         int block_size, int step, float sm_scale, int dtype, void* stream) {
  const char* who = "aa_stage3_sparse_fwd";
  int rc;
  if ((rc = check_dtype(dtype, who))) return rc;
  if ((rc = check_dims({batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step}, who))) return rc;
  if ((rc = check_tensor(q, q_sb, q_sh, q_sn, n_ctx, head_dim, who, "q"))) return rc;
  if ((rc = check_tensor(k, k_sb, k_sh, k_sn, n_ctx, head_dim, who, "k"))) return rc;
  if ((rc = check_tensor(v, v_sb, v_sh, v_sn, n_ctx, head_dim, who, "v"))) return rc;
  if ((rc = check_tensor(out, o_sb, o_sh, o_sn, n_ctx, head_dim, who, "out"))) return rc;
  if ((rc = check_ptr(coords, who, "coords")) || (rc = check_ptr(counts, who, "counts")) || (rc = check_ptr(M, who, "M")) ||
      (rc = check_ptr(L, who, "L")) || (rc = check_ptr(acc_frag, who, "acc_frag")))
    return rc;
  FlashArgs a = {};
  a.q = (const uint16_t*)q; a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn;
  a.k = (const uint16_t*)k; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.v = (const uint16_t*)v; a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn;
  a.out = (uint16_t*)out; a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.M = M; a.L = L; a.acc_frag = acc_frag;
  a.coords = coords; a.counts = counts;
  a.coords_per_head = aa_coords_entries_per_head(n_ctx, block_size, step);
  a.batch = batch; a.n_q_heads = n_q_heads; a.n_kv_heads = n_kv_heads; a.n_ctx = n_ctx; a.head_dim = head_dim;
  a.big_block = block_size * step; a.block_size = block_size;
  a.sm_scale = sm_scale; a.scale_mode = AA_SCALE_FP32; a.dtype = dtype;
  return check_launch(run_flash(a, 1, (hipStream_t)stream), who);
}

int aa_anchor_attn_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                       const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                       const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                       void* out, int64_t o_sb, int64_t o_sh, int64_t o_sn,
                       void* workspace, size_t workspace_bytes, int32_t* counts_out,
                       int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                       int block_size, int step, double sm_scale, float theta_log2, int scale_mode, int geometry,
                       int dtype, void* stream) {
  const char* who = "aa_anchor_attn_fwd";
  int rc;
  if ((rc = check_dims({batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step}, who))) return rc;
  if ((rc = check_ptr(workspace, who, "workspace"))) return rc;
  const Workspace w = carve(batch, n_q_heads, n_ctx, head_dim, block_size, step);
  if (workspace_bytes < w.total) {
    set_error("%s: workspace has %zu bytes, %zu needed", who, workspace_bytes, w.total);
    return AA_EBADARG;
  }
  char* ws = static_cast<char*>(workspace);
  float* M = (float*)(ws + w.M);
  float* L = (float*)(ws + w.L);
  float* acc = (float*)(ws + w.acc);
  void* qbar = ws + w.qbar;
  void* abar = ws + w.abar;
  uint32_t* mask = (uint32_t*)(ws + w.mask);
  int32_t* coords = (int32_t*)(ws + w.coords);
  int32_t* counts = (int32_t*)(ws + w.counts);
  // A stage-1 work-group holds 128 query rows: whole pooled rows when block_size <= 128, and then it pools them itself
  // (same arithmetic as aa_pool_q_anchor, bit for bit) instead of a separate pass over the queries.
  const bool fused_pool = block_size <= 128;
  if ((rc = stage1_impl(who, q, q_sb, q_sh, q_sn, k, k_sb, k_sh, k_sn, v, v_sb, v_sh, v_sn, M, L, acc, fused_pool ? qbar : nullptr,
                        fused_pool ? abar : nullptr, batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step,
                        (float)sm_scale, scale_mode, dtype, stream)))
    return rc;
  if (!fused_pool &&
      (rc = aa_pool_q_anchor(q, q_sb, q_sh, q_sn, M, qbar, abar, batch, n_q_heads, n_ctx, head_dim, block_size, dtype, stream)))
    return rc;
  if ((rc = aa_stage2_select(qbar, abar, k, k_sb, k_sh, k_sn, mask, coords, counts, batch, n_q_heads, n_kv_heads, n_ctx,
                             head_dim, block_size, step, sm_scale, theta_log2, geometry, dtype, stream)))
    return rc;
  if ((rc = aa_stage3_sparse_fwd(q, q_sb, q_sh, q_sn, k, k_sb, k_sh, k_sn, v, v_sb, v_sh, v_sn, coords, counts, M, L, acc, out,
                                 o_sb, o_sh, o_sn, batch, n_q_heads, n_kv_heads, n_ctx, head_dim, block_size, step, (float)sm_scale,
                                 dtype, stream)))
    return rc;
  if (counts_out != nullptr) {
    const size_t bytes = (size_t)batch * n_q_heads * (n_ctx / (block_size * step)) * 4;
    hipError_t e = hipMemcpyAsync(counts_out, counts, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream);
    if ((rc = check_launch(e, who))) return rc;
  }
  return AA_OK;
}

int aa_dense_causal_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                        const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                        const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                        void* out, int64_t o_sb, int64_t o_sh, int64_t o_sn,
                        int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                        float sm_scale, int dtype, void* stream) {
  const char* who = "aa_dense_causal_fwd";
  int rc;
  if ((rc = check_dtype(dtype, who))) return rc;
  if ((rc = check_common_dims({batch, n_q_heads, n_kv_heads, n_ctx, head_dim, 128, 16}, who))) return rc;
  if ((rc = check_tensor(q, q_sb, q_sh, q_sn, n_ctx, head_dim, who, "q"))) return rc;
  if ((rc = check_tensor(k, k_sb, k_sh, k_sn, n_ctx, head_dim, who, "k"))) return rc;
  if ((rc = check_tensor(v, v_sb, v_sh, v_sn, n_ctx, head_dim, who, "v"))) return rc;
  if ((rc = check_tensor(out, o_sb, o_sh, o_sn, n_ctx, head_dim, who, "out"))) return rc;
  FlashArgs a = {};
  a.q = (const uint16_t*)q; a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn;
  a.k = (const uint16_t*)k; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.v = (const uint16_t*)v; a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn;
  a.out = (uint16_t*)out; a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.batch = batch; a.n_q_heads = n_q_heads; a.n_kv_heads = n_kv_heads; a.n_ctx = n_ctx; a.head_dim = head_dim;
  a.big_block = n_ctx; a.block_size = 128;  // one "big block": bb is always 0
  a.sm_scale = sm_scale; a.scale_mode = AA_SCALE_FP32; a.dtype = dtype;
  return check_launch(run_flash(a, 2, (hipStream_t)stream), who);
}

}  // extern "C"
