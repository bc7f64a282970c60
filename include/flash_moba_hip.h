/*
 * flash_moba_hip.h -- C ABI of the MI355X (gfx950) FlashMoBA kernels.
 *
 * One shared library, libflash_moba_hip.so, exports exactly the entry points declared
 * here.  Every pointer is a DEVICE pointer owned by the caller unless stated otherwise;
 * strides are in ELEMENTS; `stream` is a hipStream_t passed as void*.  No entry point
 * allocates, frees or synchronises: scratch memory comes in through `workspace`
 * arguments whose size the matching *_workspace_bytes() query returns.  All launches go
 * to `stream`.  Return value: 0 on success, non-zero on error (then fmoba_last_error()
 * returns a thread-local, NUL-terminated description).  Arguments are validated on the
 * host BEFORE anything is launched.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * mit-han-lab/flash-moba checkout).
 */
#ifndef FLASH_MOBA_HIP_H_
#define FLASH_MOBA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMOBA_DTYPE_F16 0
#define FMOBA_DTYPE_BF16 1

/* Library/ABI version (major*10000 + minor*100 + patch). */
int fmoba_version(void);
/* Last error message of the calling thread ("" if none). */
const char *fmoba_last_error(void);
/* 0 if the current HIP device is a gfx950 part the kernels were built for, else non-zero
 * (replaces the compute-capability check of csrc/flash_topk/flash_topk_api.cpp:147-151). */
int fmoba_check_device(void);

/* ------------------------------------------------------------------------------------
 * Per-chunk key mean-pool.
 * Replaces flash_moba/triton_mean_pool.py:41-109 (mean_pool_kernel) as launched by
 * flash_topk_mean_pool (:112-157):
 *   km[cu_km[b] + c, h, :] = cast(sum_fp32(k[cu_k[b] + c*chunk + r, h, :], r < n) / n),
 *   n = min(chunk, len_b - c*chunk).
 * Rows of km beyond cu_km[batch] are not touched.
 * ---------------------------------------------------------------------------------- */
typedef struct {
  const void *k;            /* (total_k, heads_k, head_dim) */
  void *km;                 /* (>= cu_km[batch], heads_k, head_dim) */
  const int32_t *cu_seqlens_k;  /* (batch + 1) */
  const int32_t *cu_seqlens_km; /* (batch + 1) */
  int32_t batch;
  int32_t max_chunks;       /* ceil(max_seqlen_k / chunk) */
  int32_t heads_k;
  int32_t head_dim;         /* multiple of 8 */
  int32_t chunk;
  int32_t dtype;            /* FMOBA_DTYPE_* */
  int64_t k_row_stride, k_head_stride;
  int64_t km_row_stride, km_head_stride;
} fmoba_mean_pool_args;
int fmoba_mean_pool(const fmoba_mean_pool_args *a, void *stream);
/* cu_seqlens_km[b] = sum over b' < b of ceil((cu_seqlens[b'+1] - cu_seqlens[b']) / chunk), b = 0 .. batch: the offsets of
 * the pooled sequences, in one launch.  Replaces the tensor expressions of flash_topk_mean_pool
 * (flash_moba/triton_mean_pool.py:132-139: lengths, ceil-division, cumulative sum, padding with a leading zero). */
int fmoba_chunk_offsets(const int32_t *cu_seqlens, int32_t *cu_seqlens_km, int32_t batch, int32_t chunk, void *stream);

/* ------------------------------------------------------------------------------------
 * Fused top-k block gating + CSC build.
 * Replaces moba_fused_topk (csrc/flash_topk/flash_topk_api.cpp:130-258), i.e. the three
 * kernels of csrc/flash_topk/src/flash_topk_launch_template.h:65-118, AND the segmented
 * sort the reference runs afterwards (flash_moba/flash_moba_interface.py:570-572): the
 * row lists written to `flat_indices` are already ascending.
 *
 *   col_offsets (batch, heads, max_cols) int64, col_nnz (batch, heads, max_cols) int32,
 *   flat_indices (total_q*heads*topk) int32  -- all fully written by the call
 *   (unused slots of flat_indices are 0), max_cols = ceil(max_seqlen_k / chunk).
 *   raw_indices / raw_values (total_q, heads, round_up(topk,16)) int32 / fp32 are the
 *   ordered per-row lists (descending score, ties -> higher chunk first, unfilled -1 /
 *   -inf); pass NULL for both to skip them.
 * ---------------------------------------------------------------------------------- */
typedef struct {
  const void *q;            /* (total_q, heads, head_dim) */
  const void *km;           /* (total_km, heads_k, head_dim) */
  const int32_t *cu_seqlens_q, *cu_seqlens_k, *cu_seqlens_km; /* (batch + 1) each */
  int64_t *col_offsets;
  int32_t *col_nnz;
  int32_t *flat_indices;
  int32_t *raw_indices;     /* optional */
  float *raw_values;        /* optional */
  void *workspace;          /* fmoba_fused_topk_workspace_bytes() bytes, 256-byte aligned */
  size_t workspace_bytes;
  int32_t batch, total_q, heads, heads_k, head_dim;
  int32_t max_seqlen_q, max_seqlen_k;
  int32_t topk, chunk, is_causal, dtype;
  int64_t q_row_stride, q_head_stride, km_row_stride, km_head_stride;
} fmoba_fused_topk_args;
size_t fmoba_fused_topk_workspace_bytes(int32_t batch, int32_t total_q, int32_t heads,
                                        int32_t max_seqlen_q, int32_t max_seqlen_k, int32_t chunk);
int fmoba_fused_topk(const fmoba_fused_topk_args *a, void *stream);
/* The same call without a workspace, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference, whose host code allocates on every call.  `workspace` / `workspace_bytes` of `a` are
 * ignored: selection bits and segment counts live in a fixed array inside the library's code object
 * (FMOBA_STATIC_SCRATCH_BYTES per device, held until the process ends).  The call fails with a clear
 * error, before anything is launched, when fmoba_fused_topk_workspace_bytes() of the same sizes exceeds
 * that limit (the headline shape -- 65536 tokens, 16 heads, 224 chunks -- needs 30.3 MB and fits).
 * It calls no hipMalloc / hipFree.  All calls on one device share the array: calls that overlap on one
 * device (different streams or threads) race; calls in stream order are safe, every call clears what
 * it needs zeroed with a fill kernel of its own.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress): make it outside any stream capture. */
#define FMOBA_STATIC_SCRATCH_BYTES (32u << 20)
int fmoba_fused_topk_static(const fmoba_fused_topk_args *a, void *stream);

/* ------------------------------------------------------------------------------------
 * Segmented ascending sort of signed int32 keys with 64-bit segment offsets.
 * Replaces varlen_sort (csrc/flash_topk/src/varlen_sort.cu:127-162, CUB
 * DeviceSegmentedSort).  dst[i] = 0 for positions outside every segment.  Segments must
 * not overlap.  `workspace`: fmoba_varlen_sort_workspace_bytes(total) bytes -- `total` int32
 * (marks of the segments, second buffer of segments too long for LDS) and 256 bytes of
 * notes the launches leave each other.  A workspace of `total` int32 alone is accepted as
 * well; the call then always clears dst first and every launch looks at every segment.
 * ---------------------------------------------------------------------------------- */
size_t fmoba_varlen_sort_workspace_bytes(int64_t total);
int fmoba_varlen_sort(const int64_t *seg_starts, const int64_t *seg_ends, int64_t num_segments,
                      const int32_t *src, int32_t *dst, int64_t total, void *workspace,
                      size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------
 * Sparse attention forward over a CSC pattern.
 * Replaces moba_varlen_fwd (csrc/flash_moba/flash_moba_api.cpp:375-596).
 *   out (total_q, heads, head_dim) dtype, softmax_lse (heads, total_q) fp32.
 * Rows that see no key get out = 0, lse = +inf.
 * Two forms.  Row blocks (patterns in which a row selects a good part of the chunks it may see):
 * one workgroup per 256 (or 128) query rows walks every chunk any of its rows selected, with the running
 * softmax state in registers; `workspace` then holds one selection bit per (row, head, chunk).
 * Columns (sparser patterns): every visit of a (query row, key block) pair leaves a
 * partial result in `workspace`, and a second launch merges the partials of each row.  A key
 * block is fmoba_attn_fwd_key_block(lg_block_n) keys (128 if lg_block_n is a multiple of 128,
 * else 64).  max_visits_per_row bounds the number of visits of any (row, head): for a pattern
 * from the gating, topk * lg_block_n / key_block; for an arbitrary pattern,
 * fmoba_csc_max_row_visits() computes it.  Visits beyond the bound are dropped (and reported: visits_overflow).
 * workspace: fmoba_attn_fwd_workspace_bytes() bytes, contents undefined on entry and return.
 * ---------------------------------------------------------------------------------- */
typedef struct {
  const void *q, *k, *v;
  void *out;
  float *softmax_lse;
  const int64_t *col_offsets;   /* (batch, heads, max_cols) */
  const int32_t *col_nnz;       /* (batch, heads, max_cols) */
  const int32_t *row_indices;   /* flat row lists */
  const int32_t *cu_seqlens_q, *cu_seqlens_k;
  /* optional (may be NULL): the same pattern as one bit per (row, head, chunk), word
   * [(h * ceil(max_cols/32) + c/32) * total_q + global row] bit c%32 -- what fmoba_fused_topk leaves
   * at the first 256-byte boundary of its workspace.  Only the row-block form reads it; without it
   * that form derives the bits from the lists first. */
  const uint32_t *selection_bits;
  void *workspace;
  size_t workspace_bytes;
  int32_t batch, total_q, total_k, heads, heads_k, head_dim;
  int32_t max_seqlen_q, max_seqlen_k, max_cols;
  int32_t lg_block_m, lg_block_n;
  int32_t is_causal, dtype;
  int32_t max_visits_per_row;
  int32_t fwd_mode;             /* 0 = the library chooses, 1 = column form, 2 = row-block form */
  float softmax_scale;
  int64_t q_row_stride, q_head_stride, k_row_stride, k_head_stride;
  int64_t v_row_stride, v_head_stride, o_row_stride, o_head_stride;
  /* optional (may be NULL): one int32 the caller has set to 0.  A form that stores per-visit partial results
   * raises it (atomic max) to the visit count of any (row, head) that exceeds max_visits_per_row -- such a
   * row's result is wrong, its surplus visits were dropped -- so that a caller who passed a bound of its own
   * can tell afterwards (a device-to-host read after the stream has passed the call).  Stays 0 otherwise. */
  int32_t *visits_overflow;
} fmoba_attn_fwd_args;
int32_t fmoba_attn_fwd_key_block(int32_t lg_block_n);
/* Bytes of workspace for the call described by `a` (sizes, max_visits_per_row and fwd_mode are read,
 * pointers are not), and which form it will run (1 = row blocks, 0 = columns). */
size_t fmoba_attn_fwd_workspace_bytes(const fmoba_attn_fwd_args *a);
int32_t fmoba_attn_fwd_uses_row_blocks(const fmoba_attn_fwd_args *a);
/* counts (total_q * heads) int32 and max_out (1) int32 are device outputs: visits per (row, head) and
 * their maximum for the pattern in `a` (q/k/v/out/workspace of `a` are not read).  No counterpart in the
 * reference, whose row-wise scratch needs no bound. */
int fmoba_csc_max_row_visits(const fmoba_attn_fwd_args *a, int32_t *counts, int32_t *max_out, void *stream);
int fmoba_attn_fwd(const fmoba_attn_fwd_args *a, void *stream);
/* The same call split into its two launches so that each can be timed on its own: phases is a bit
 * mask, 1 = the column pass (clears the visit counters first), 2 = the per-row combine; in the
 * row-block form 1 = building the selection bits, 2 = the attention pass.
 * fmoba_attn_fwd(a, s) == fmoba_attn_fwd_phases(a, 3, s). */
#define FMOBA_FWD_COLUMNS 1
#define FMOBA_FWD_COMBINE 2
int fmoba_attn_fwd_phases(const fmoba_attn_fwd_args *a, int32_t phases, void *stream);

/* ------------------------------------------------------------------------------------
 * Sparse attention backward.
 * Replaces moba_varlen_bwd (csrc/flash_moba/flash_moba_api.cpp:610-848).
 *   dq (total_q, heads, d), dk/dv (total_k, heads, d) -- dk/dv are PER QUERY HEAD; for
 *   GQA/MQA the caller sums groups of heads/heads_k (flash_moba_api.cpp:842-845).
 *   softmax_d (heads, total_q + 128*batch) fp32: row (b, r) of head h is stored at
 *   h*(total_q + 128*batch) + cu_q[b] + 128*b + r (flash_bwd_preprocess_kernel.h:86).
 *   dK/dV come from one column-stationary pass.  dQ has two forms (dq_mode: 0 = the library
 *   chooses, 1 = row blocks, 2 = partials; fmoba_attn_bwd_uses_partials() tells the choice):
 *     row blocks: the dK/dV pass leaves the dS tiles (16-bit, lg_block_n entries per entry of
 *       row_indices) in the workspace and a row-stationary pass (128 or 256 query rows per
 *       workgroup, accumulators in registers) multiplies them with K; the only form for
 *       head_dim > 128;
 *     partials: the dK/dV pass leaves one dQ partial row (16-bit) per visit of a (query row,
 *       key block) pair, a second launch adds the partials of each row in key order.  This is
 *       the form that scales when sequences have thousands of chunks.  (Key blocks have 128 keys
 *       when lg_block_n is a multiple of 128 and head_dim > 64, else 64.)
 *   workspace: fmoba_attn_bwd_workspace_bytes(args) bytes (only the sizes, dq_mode,
 *   num_row_indices and max_visits_per_row of args are read), contents undefined on entry and on
 *   return.  num_row_indices = number of int32 entries of row_indices (every col_offsets[i] +
 *   col_nnz[i] must be <= it).  max_visits_per_row bounds the visits of any (row, head): for a
 *   pattern from the gating topk * lg_block_n / 64; for an arbitrary pattern
 *   fmoba_csc_max_row_visits() counts them in forward key blocks, multiply by
 *   fmoba_attn_fwd_key_block(lg_block_n) / 64.  Visits beyond the bound are dropped (and reported: visits_overflow).
 *   No floating-point atomics: results are bitwise reproducible whatever `deterministic` says.
 * ---------------------------------------------------------------------------------- */
typedef struct {
  const void *dout, *q, *k, *v, *out;
  const float *softmax_lse;
  void *dq, *dk, *dv;
  float *softmax_d;
  const int64_t *col_offsets;
  const int32_t *col_nnz;
  const int32_t *row_indices;
  const int32_t *cu_seqlens_q, *cu_seqlens_k;
  void *workspace;
  size_t workspace_bytes;
  int64_t num_row_indices;
  int32_t batch, total_q, total_k, heads, heads_k, head_dim;
  int32_t max_seqlen_q, max_seqlen_k, max_cols;
  int32_t lg_block_m, lg_block_n;
  int32_t is_causal, dtype, deterministic;
  int32_t max_visits_per_row, dq_mode;
  float softmax_scale;
  int64_t q_row_stride, q_head_stride, k_row_stride, k_head_stride;
  int64_t v_row_stride, v_head_stride, o_row_stride, o_head_stride;
  int64_t do_row_stride, do_head_stride;
  int64_t dq_row_stride, dq_head_stride, dk_row_stride, dk_head_stride;
  int64_t dv_row_stride, dv_head_stride;
  int32_t *visits_overflow;  /* optional, as in fmoba_attn_fwd_args (counts are in the backward's key blocks) */
} fmoba_attn_bwd_args;
int32_t fmoba_attn_bwd_uses_partials(const fmoba_attn_bwd_args *a);
size_t fmoba_attn_bwd_workspace_bytes(const fmoba_attn_bwd_args *a);
int fmoba_attn_bwd(const fmoba_attn_bwd_args *a, void *stream);
/* The same call split into its three launches so that each can be timed on its own:
 * phases is a bit mask, 1 = dot(dO, O) (flash_bwd_launch_template.h:70-74), 2 = the
 * column-stationary dK/dV kernel, which also fills the workspace (:76-96), 4 = the dQ pass
 * in either form (stands where the reference converts its fp32 dQ accumulator, :98-104).  fmoba_attn_bwd(a, s) == fmoba_attn_bwd_phases(a, 7, s). */
#define FMOBA_BWD_PREP 1
#define FMOBA_BWD_DKDV 2
#define FMOBA_BWD_DQ 4
int fmoba_attn_bwd_phases(const fmoba_attn_bwd_args *a, int32_t phases, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_MOBA_HIP_H_ */
