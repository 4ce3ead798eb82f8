/*
 * anchor_attn_hip.h - C ABI of the gfx950 (MI355X) AnchorAttention prefill kernels.
 *
 * Every entry point takes plain device pointers, sizes, element strides and a HIP stream
 * (passed as void*; NULL is the default stream).  The library never allocates or frees device
 * memory: scratch is handed in by the caller.  All launches are asynchronous on the given
 * stream and nothing synchronises the device.  Return value: 0 on success, otherwise one of
 * the AA_E* codes; aa_last_error() then describes the failure (thread-local string).
 *
 * Tensors: q/out are [batch, n_q_heads, n_ctx, head_dim]; k/v are [batch, n_kv_heads, n_ctx,
 * head_dim] with n_kv_heads dividing n_q_heads (query head h reads KV head
 * h / (n_q_heads / n_kv_heads), the order repeat_kv produces; pass n_kv_heads == n_q_heads for
 * pre-repeated K/V as the reference's caller does).  Element type is bf16 or fp16 (the `dtype`
 * argument, AA_DTYPE_*, the same for every tensor of a call), head_dim must be
 * 128 or 64 with stride 1, every row must start on a 16-byte boundary; the other three dimensions
 * are addressed through the element strides (sb, sh, sn), so [B,N,H,D] storage works unchanged.
 * "S" below is the big block, block_size * step keys/queries.
 *
 * Reference citations are paths inside yuzhouzhang9/Anchor-Attention.
 */
#ifndef ANCHOR_ATTN_HIP_H_
#define ANCHOR_ATTN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AA_OK 0
#define AA_EBADARG 1      /* null pointer, non-positive size, head counts that do not divide, unknown dtype/mode */
#define AA_EUNSUPPORTED 2 /* head_dim not 128 or 64, block_size not in 16..256, step not 16/32, n_ctx % S != 0, n_ctx > 2^20 */
#define AA_EMISALIGNED 3  /* pointer or stride not a multiple of 16 bytes */
#define AA_ELAUNCH 4      /* HIP runtime error at launch */

/* Element type of q, k, v, out and of the pooled queries/anchors.  The reference takes bf16 and fp16 tensors
 * (dtype = tl.bfloat16 if Q.dtype == torch.bfloat16 else tl.float16: anchor_step_1_2_v2.py:193, anchor_attn_v4.py:265,
 * get_mask_test.py:157); every ".to(dtype)" of its kernels - scaled queries, probabilities, pooled queries and
 * anchors, stage-2 scores, output - then rounds to that type.  Accumulators and M, L, Acc are float32 either way. */
#define AA_DTYPE_BF16 0
#define AA_DTYPE_F16 1

/* How stage 1 pre-scales queries.  AA_SCALE_BF16_CHAIN reproduces the reference's stage-1
 * kernel, where sm_scale is a compile-time constant and q * sm_scale * 1.44269504 is therefore
 * evaluated in the tensors' 16-bit type with a rounding after each multiply (anchor_step_1_2_v2.py:19,115-116).
 * AA_SCALE_FP32 is the float32 product rounded once (what stage 3 does, anchor_attn_v4.py:66). */
#define AA_SCALE_BF16_CHAIN 0
#define AA_SCALE_FP32 1

/* Which keys stage 2 may select for big block bb.  AA_GEOMETRY_AS_RUN is what the reference's operator does
 * (get_mask_test.py:93-94): [block_size, bb*S - block_size) - keys below S are then attended twice (stage 1
 * already covers [0,S)) and the last block_size keys before the big block never.  AA_GEOMETRY_INTENDED is the
 * range the reference's fused variant walks (anchor_fuse_step_1_2_v2.py:152, init_limit .. local_start):
 * [S, bb*S), no overlap and no gap.  Never the default; it exists to measure what the as-run quirks cost. */
#define AA_GEOMETRY_AS_RUN 0
#define AA_GEOMETRY_INTENDED 1

/* 2 for this ABI.  1000 + n marks a timing-only build (`make ablations`, AA_ABLATE = n) that leaves part of a kernel out and
 * computes wrong results on purpose; such a build is for bench_ablations.py only and the Python loader refuses it. */
int aa_version(void);
const char* aa_last_error(void);

/* ---- scratch geometry ---------------------------------------------------------------------- */

/* Selected-key index lists are packed: per (batch, q head) one slab of
 * aa_coords_entries_per_head() int32; big block bb's ascending list starts at
 * aa_coords_offset(bb) inside the slab and holds counts[b,h,bb] entries (capacity
 * bb*S - 2*block_size, the number of candidate keys).  Replaces the reference's
 * true_coords [B,H,N/S,N] buffer (get_mask_test.py:138-141). */
int64_t aa_coords_entries_per_head(int n_ctx, int block_size, int step);
int64_t aa_coords_offset(int big_block, int block_size, int step);

/* Number of uint32 words of the stage-2 scratch: the key bitmask [batch, n_q_heads, n_ctx/S, n_ctx/128, 4]
 * followed by one float32 selection threshold per pooled query row [batch, n_q_heads, n_ctx/block_size]. */
int64_t aa_mask_words(int batch, int n_q_heads, int n_ctx, int block_size, int step);

/* Bytes of scratch aa_anchor_attn_fwd() needs (M, L, Acc, pooled q, pooled anchors, bitmask,
 * index lists, counts - in that order, each 256-byte aligned). */
size_t aa_workspace_bytes(int batch, int n_q_heads, int n_ctx, int head_dim, int block_size, int step);

/* ---- stage 1: pattern-based anchor computation ---------------------------------------------
 * Replaces anchor_attn_step_1 / get_mask_fused_anchor_triton with init_cnt = local_cnt = 1
 * (anchor_step_1_2_v2.py:8-196; call site anchor_attn_v4.py:237-241): flash attention of each
 * query row r over keys [0,S) U [bb*S, r] (bb = r / S), exp2 domain.
 * Outputs: M [B,Hq,N] float32 running max (the anchors), L [B,Hq,N] float32 row sums,
 * acc_frag float32 with B*Hq*N*head_dim elements: the unnormalised PV accumulator in MFMA fragment
 * order - element (b,h,row,d) lives at ((((b*Hq+h)*(N/32) + row/32)*(head_dim/32) + d/32)*4 + (d%32)/8)*256
 * + (((d%8)/4)*32 + row%32)*4 + d%4.  Stage 3 consumes exactly this order. */
int aa_stage1_anchor_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         float* M, float* L, float* acc_frag,
                         int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                         int block_size, int step, float sm_scale, int scale_mode, int dtype, void* stream);

/* ---- stage 2: difference-aware stripe identification -------------------------------------- */

/* Mean-pools raw queries and anchors over block_size rows, rounding to the 16-bit type
 * (get_mask_test.py:75-84): qbar [B,Hq,N/block_size,head_dim], abar [B,Hq,N/block_size], both of the tensors' 16-bit type.
 * Sums run in float32 in ascending row order. */
int aa_pool_q_anchor(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn, const float* M,
                     void* qbar, void* abar,
                     int batch, int n_q_heads, int n_ctx, int head_dim, int block_size, int dtype, void* stream);

/* Replaces anchor_attn_step_2 / get_q_mask / get_q_mask_triton (anchor_step_1_2_v2.py:199-210,
 * get_mask_test.py:7-159): key j in [block_size, bb*S - block_size) is selected for big block bb
 * iff for one of its pooled rows i  float(round16(dot(qbar_i,k_j) * sm_scale*1.44269504)) + theta_log2
 * >= float(abar_i).  theta_log2 is float32(theta * 1.44269504), the product formed in double precision as the
 * reference's entry does with Python floats (anchor_attn_v4.py:298) and handed to the kernel as a float32
 * argument.  sm_scale is a double because the score scale is a compile-time constant in the reference's kernel:
 * float32(double(sm_scale) * 1.44269504) (get_mask_test.py:86).  geometry: AA_GEOMETRY_* (the candidate range
 * above is the as-run one).
 * mask_ws: scratch of aa_mask_words() uint32.  Outputs: coords (packed, see above) and
 * counts [B,Hq,N/S] int32.  Deterministic: no atomics, lists are ascending. */
int aa_stage2_select(const void* qbar, const void* abar,
                     const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                     uint32_t* mask_ws, int32_t* coords, int32_t* counts,
                     int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                     int block_size, int step, double sm_scale, float theta_log2, int geometry, int dtype, void* stream);

/* Same operation, same kernels and same results as aa_stage2_select, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc) and therefore cannot provide
 * mask_ws: the bitmask and thresholds live in a static device array of AA_STATIC_SCRATCH_BYTES inside the library
 * (one copy per GPU, held until the process ends).  This entry point has no counterpart in the reference, whose
 * get_q_mask allocates its buffers with torch on every call (get_mask_test.py:138-145).
 * It calls no hipMalloc/hipFree or other allocating routine.  Problems whose aa_mask_words()*4 exceeds
 * AA_STATIC_SCRATCH_BYTES are refused with AA_EUNSUPPORTED (the Llama-3.1-8B layer at 131072 tokens, 32 query heads,
 * needs 32.1 MiB and fits).  The first call on a device looks the array's address up (hipGetSymbolAddress): make
 * that call outside any stream capture.  All calls on one GPU share the array: calls that overlap on one GPU (two
 * streams, two threads) race; calls ordered on one stream do not.  Nothing has to be cleared between calls: every
 * word stage 2 reads is written earlier in the same call. */
#define AA_STATIC_SCRATCH_BYTES (40 * 1024 * 1024)
int aa_stage2_select_static(const void* qbar, const void* abar,
                            const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                            int32_t* coords, int32_t* counts,
                            int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                            int block_size, int step, double sm_scale, float theta_log2, int geometry, int dtype, void* stream);

/* ---- stage 3: fine-grained sparse flash attention ------------------------------------------
 * Replaces _triton_stripe_sparse_attn_fwd_kernel_step3 (anchor_attn_v4.py:7-105; launch
 * :246-268): resumes the online softmax from (M, L, acc_frag) over the K/V rows gathered at the
 * big block's selected indices and writes out = round16(acc / l).  M, L, acc_frag are read-only.
 * coords and counts are read as they are found in device memory: a count below 0 or above the list's capacity is
 * clamped to it and an index outside [0, n_ctx) to the nearest valid row, so stale or corrupt lists give wrong
 * values but no access outside the tensors. */
int aa_stage3_sparse_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         const int32_t* coords, const int32_t* counts,
                         const float* M, const float* L, const float* acc_frag,
                         void* out, int64_t o_sb, int64_t o_sh, int64_t o_sn,
                         int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                         int block_size, int step, float sm_scale, int dtype, void* stream);

/* ---- whole operator -------------------------------------------------------------------------
 * Replaces _anchor_attn (anchor_attn_v4.py:226-273): stage 1 -> pooling -> stage 2 -> stage 3 on
 * one stream.  workspace: aa_workspace_bytes() bytes of device scratch (contents undefined
 * afterwards).  counts_out (optional, may be NULL): [B,Hq,N/S] int32 copy of the per-big-block
 * selection counts, from which the caller forms the sparsity ratio (anchor_attn_v4.py:270-272).
 * theta_log2 and the double sm_scale are those of aa_stage2_select (the caller forms theta * 1.44269504 in double
 * precision, as anchor_attn_v4.py:298 does, so that the one-call and the staged paths see the same float32);
 * stages 1 and 3 use float32(sm_scale), a run-time float32 argument of the reference's stage-3 kernel. */
int aa_anchor_attn_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                       const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                       const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                       void* out, int64_t o_sb, int64_t o_sh, int64_t o_sn,
                       void* workspace, size_t workspace_bytes, int32_t* counts_out,
                       int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                       int block_size, int step, double sm_scale, float theta_log2, int scale_mode, int geometry,
                       int dtype, void* stream);

/* ---- dense causal baseline on the same MFMA core --------------------------------------------
 * Counterpart of the reference's dense comparison path (flash_attn_triton.py:83-211, GQA mapping
 * :129-132): plain causal softmax attention, out = round16(softmax(q k^T * sm_scale) v).
 * n_ctx must be a multiple of 128. */
int aa_dense_causal_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sn,
                        const void* k, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                        const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                        void* out, int64_t o_sb, int64_t o_sh, int64_t o_sn,
                        int batch, int n_q_heads, int n_kv_heads, int n_ctx, int head_dim,
                        float sm_scale, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ANCHOR_ATTN_HIP_H_ */
