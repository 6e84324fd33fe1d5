/*
 * topk_attn.h — C ABI of the MI355X (gfx950) sparse-decode path:
 *   stage 1  fused q·K^T GEMV + exact top-k selection (flat, centre-only, two-level cluster)
 *   stage 2  gather-based retrieval attention over the selected tokens
 *   stage 3  split-K flash-decoding with a separate log-sum-exp combine
 *
 * Conventions
 *   - Every pointer marked "device" is a HIP device pointer owned by the caller.
 *   - Every call is asynchronous on `stream` (a hipStream_t passed as void*; NULL = the null stream),
 *     allocates nothing, and keeps all temporaries in the caller-provided workspace whose size the
 *     matching *_workspace_bytes() query returns.  Two calls may share a workspace only if they are
 *     ordered on one stream.
 *   - Return value is a tka_status; nothing here prints or exits.  Argument validation happens before
 *     the first HIP call, so a bad call returns TKA_EINVAL / TKA_EUNSUPPORTED on a machine with no GPU.
 *   - Tensor element types are IEEE binary16 (TKA_F16) or bfloat16 (TKA_BF16); head_dim must be 128.
 *   - Fields named reserved* must be zero (a later version may give them a meaning, as version 2.0.0 did with
 *     score_mode); zero the argument block before filling it in.
 *   - Strides are in ELEMENTS.  Offsets are 64-bit everywhere (the reference's int32 offsets overflow
 *     beyond 524288 tokens at 32 heads, retrieval_attn/retrieval_attention.cu:323).
 *
 * Score definition (all stage-1 entry points).  For KV head h with `group` query heads g = 0..G-1:
 *     qf[d]   = ((f32(q[hG+0][d]) + f32(q[hG+1][d])) + ...) + f32(q[hG+G-1][d])        (fp32, ascending g)
 *     p_j     = fma chain over d = 8j..8j+7 of qf[d]*f32(K[t][h][d]) starting from +0.0f   (j = 0..15)
 *     dot     = butterfly sum of p_0..p_15 with partner distances 8, 4, 2, 1
 *     score   = dot * scale                                                            (one fp32 multiply)
 * which is the 16-lane reduction order of the reference GEMV (gemv_topk.cu:320-328).  The selection
 * order is (score descending, token index ascending); -0.0 compares equal to +0.0 and NaN sorts below
 * every number.  Selected indices are returned in that rank order.
 */
#ifndef TOPK_ATTN_H_
#define TOPK_ATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TKA_HEAD_DIM 128
#define TKA_MAX_TOPK 8192      /* largest k of one selection                                   */
#define TKA_MAX_GROUP 8        /* query heads sharing one KV head: 1, 2, 4 or 8               */
#define TKA_MAX_SPLITS 1024    /* largest split count of flash-decoding / retrieval attention */
#define TKA_NOALLOC_SCRATCH_BYTES (128u << 20) /* built-in scratch of tka_sparse_decode_step_noalloc, per GPU */

typedef enum tka_status {
  TKA_OK = 0,
  TKA_EINVAL = 1,        /* null pointer, non-positive size, k > seq_len, ...          */
  TKA_EUNSUPPORTED = 2,  /* head_dim != 128, unknown dtype, group too large, ...       */
  TKA_EHIP = 3,          /* a HIP runtime call failed (launch error, bad stream)       */
  TKA_EWORKSPACE = 4,    /* workspace missing or smaller than *_workspace_bytes()      */
  TKA_ESCRATCH = 5       /* tka_sparse_decode_step_noalloc: the call needs more than
                            TKA_NOALLOC_SCRATCH_BYTES of scratch memory                */
} tka_status;

typedef enum tka_dtype { TKA_F16 = 0, TKA_BF16 = 1 } tka_dtype;

typedef enum tka_softmax_mode {
  TKA_SOFTMAX_SCALED = 0, /* softmax(scale * q.k), max-subtracted (baseline_1.py:104-107)                 */
  TKA_SOFTMAX_RAW_EXP = 1 /* exp(s)/sum exp(s) on unscaled scores (retrieval_attention.cu:1277-1319);
                             evaluated max-subtracted in fp32, which is the same function               */
} tka_softmax_mode;

/* How stage 1 adds up the 128 products of a score.
 * TKA_SCORE_CANONICAL: the 16-lane order defined above; scores are bit-identical to the reference order on any route.
 * TKA_SCORE_MATRIX: where keys are shared by a batch of at least two entries (key_stride_b == 0, group == 1) the
 *   scores come from the matrix cores (v_mfma_f32_16x16x32, fp32 accumulation in the unit's own order): within a
 *   few units in the last place of the canonical ones (1e-5 of the exact dot product), not bit-identical to them.
 *   The selection is exact on the scores the call computed: out_idx / out_val are the first k of a stable
 *   descending sort of what out_scores would hold.  A call it does not apply to (grouped queries, keys not shared, a
 *   batch of one, a top-k over chunks of more than 16384 keys) returns TKA_EUNSUPPORTED: the scoring order that ran
 *   is always the one that was asked for.
 *   (The batch pipeline of retrieval_attention.cu:654-896 as a skinny GEMM; about 4x quicker at batch 32.) */
typedef enum tka_score_mode { TKA_SCORE_CANONICAL = 0, TKA_SCORE_MATRIX = 1 } tka_score_mode;

const char* tka_status_string(int status);
/* Library version as major*10000 + minor*100 + patch. */
int tka_version(void);

/* ------------------------------------------------------------------------------------------------
 * Stage 1a — flat fused GEMV + top-k.
 * Replaces the launch in main() of gemv_topk.cu:466-469 (grid 160 x 128, compile-time shapes) and the
 * standalone retrieval_topk_kernel launch (retrieval_attention.cu:1162-1238) with one runtime-shaped
 * call.  With num_chunks > 1 the sequence is cut into num_chunks equal ranges and a separate top-k is
 * taken inside each (the per-chunk selection of retrieval_attention.cu:1198-1237); out slot is
 * [b][h][c*k + r] and indices are global token ids.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_gemv_topk_args {
  const void* q;          /* device [batch][num_kv_heads*group][128]                         */
  const void* keys;       /* device; row (b,t,h) at keys + b*stride_b + t*stride_n + h*stride_h */
  int32_t dtype;          /* tka_dtype of q and keys                                          */
  int32_t batch;
  int32_t num_kv_heads;
  int32_t group;          /* query heads per KV head; their scores are summed (see header)    */
  int32_t head_dim;       /* must be 128                                                      */
  int32_t k;              /* selected per chunk                                               */
  int32_t num_chunks;     /* >= 1; seq_len must be a multiple                                 */
  int32_t score_mode;     /* tka_score_mode; 0 = the canonical order of the header            */
  int64_t seq_len;
  int64_t q_stride_b;     /* elements between batch entries of q                              */
  int64_t key_stride_b;   /* 0 = keys shared by all batch entries (retrieval_attention.cu:681-683) */
  int64_t key_stride_n;
  int64_t key_stride_h;
  float scale;            /* score multiplier, e.g. 1/sqrt(128); 1.0f = none                  */
  int32_t reserved1;
  int32_t* out_idx;       /* device [batch][num_kv_heads][num_chunks*k], rank order           */
  float* out_val;         /* device, same shape, fp32 scores of the selected; may be NULL     */
  float* out_scores;      /* device [batch][num_kv_heads][seq_len] all scores; may be NULL    */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_gemv_topk_args;

size_t tka_gemv_topk_workspace_bytes(const tka_gemv_topk_args* args);
int tka_gemv_topk(const tka_gemv_topk_args* args);

/* GEMV phase alone: writes out_scores only (k, out_idx, out_val, workspace ignored).
 * Counterpart of gemv_phase_kernel, gemv_profile_split.cu:69-252. */
int tka_gemv_scores(const tka_gemv_topk_args* args);

/* Diagnostic (no counterpart in the reference): after a tka_gemv_topk call with the same arguments, *count =
 * how many of its segments were redone from the keys by the selection kernel.  Long segments are selected from
 * candidates above a threshold sampled inside the GEMV launch; a segment whose candidates turn out fewer than k,
 * or more than fit, or one of whose streaming workgroups ran out of its bounded wait for the threshold, is
 * redone - exact; all CUs share that work in a launch behind the selection, and a call with EVERY segment redone
 * costs about 2.3 times the ordinary one (one workgroup redoes a segment on the routes of the shorter segments:
 * a quarter of a millisecond per 32768 tokens).  0 for calls that do not take that path.
 * Waits for the stream. */
int tka_gemv_topk_redone_segments(const tka_gemv_topk_args* args, int32_t* count);
/* Same protocol: *count = candidate slices of that call (512 tokens each; 256 on calls that announce the cut of a
 * segment of up to 65536 tokens inside the GEMV launch) whose workgroup gave up waiting. */
int tka_gemv_topk_gave_up_slices(const tka_gemv_topk_args* args, int32_t* count);

/* Testing hooks (no counterpart in the reference).  Process-wide; read once at the start of every call; they
 * change how the candidate route of stage 1 gets to its result, never the result (union_handoff_order shows a
 * list in the order in which it is otherwise only handed on).  NULL restores the defaults (all zero).  Every
 * kernel still runs to its end under any setting: the waits involved are bounded. */
typedef struct tka_test_hooks {
  int32_t force_segment_redo;  /* 1: the selection accepts no candidate count, every segment of the routes that
                                  store candidates above a sampled threshold is redone from the keys    */
  int32_t tau_spin_limit;      /* > 0: polls of a streaming workgroup for its segment's threshold before
                                  it gives up (default 65536)                                           */
  int32_t tau_withhold_mod;    /* > 0: the threshold of segments s with s % mod == rem is withheld ...   */
  int32_t tau_withhold_rem;
  int32_t tau_withhold_mode;   /* ... 0: for good (every slice of the segment gives up); 1: until the
                                  first slice of the segment has given up (the later ones see it).  On
                                  calls that announce the CUT of a segment of up to 65536 tokens inside
                                  the GEMV launch the same hooks withhold that word, always for good     */
  int32_t union_handoff_order; /* 1: tka_sparse_decode_step writes out_union_idx the way it hands the list to
                                  its attention when the caller does not ask for it: in the order of the
                                  route, which may list -1 (an id the attention skips) inside the count  */
  int32_t fused_tail;          /* the launch that selects and attends in one (tka_sparse_decode_step of a
                                  caller that asks for the output alone, long segments): 0 = where it is the
                                  form that is as quick (calls of 256 segments and more), 1 = wherever it fits, 2 = never */
} tka_test_hooks;
int tka_set_test_hooks(const tka_test_hooks* hooks);

/* ------------------------------------------------------------------------------------------------
 * Stage 1b — selection phase alone on caller-supplied fp32 scores.
 * Counterpart of the sort-only kernel of gemv_profile_split.cu:255-323 and of every
 * cub::BlockRadixSort::SortDescending call site of the reference (gemv_topk.cu:361).
 * Given the same fp32 vector, the indices are those of a stable sort by (score desc, index asc).
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_topk_args {
  const float* scores;    /* device [num_segments][seg_stride]                                */
  int32_t num_segments;
  int32_t k;
  int64_t seg_len;        /* elements per segment that take part                              */
  int64_t seg_stride;     /* elements between segments (>= seg_len)                           */
  int32_t* out_idx;       /* device [num_segments][k]; index inside the segment               */
  float* out_val;         /* device [num_segments][k]; may be NULL                            */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_topk_args;

size_t tka_topk_workspace_bytes(const tka_topk_args* args);
int tka_topk_f32(const tka_topk_args* args);

/* ------------------------------------------------------------------------------------------------
 * Stage 1c — centre-only selection with expansion.
 * Replaces both launches of center_only_topk/gemv_topk.cu:545-564 (single-block and 5-CTA cluster
 * kernels): score `num_centers` centroids per head, take the top `top_c`, and expand centroid c to
 * its `cluster_len` member tokens  out[h][j*cluster_len + i] = c_j*cluster_len + i  (:272-279).
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_center_topk_args {
  const void* q;          /* device [num_heads][128]                                          */
  const void* centers;    /* device [num_heads][num_centers][128] (gemv_topk.cu:93 layout)    */
  int32_t dtype;
  int32_t num_heads;
  int32_t num_centers;
  int32_t top_c;
  int32_t cluster_len;
  int32_t head_dim;
  float scale;
  int32_t reserved0;
  int32_t* out_idx;       /* device [num_heads][top_c*cluster_len] token ids                  */
  int32_t* out_centers;   /* device [num_heads][top_c] chosen centroids, rank order; may be NULL */
  float* out_center_val;  /* device [num_heads][top_c]; may be NULL                           */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_center_topk_args;

size_t tka_center_topk_expand_workspace_bytes(const tka_center_topk_args* args);
int tka_center_topk_expand(const tka_center_topk_args* args);

/* ------------------------------------------------------------------------------------------------
 * Stage 1d — two-level cluster selection.
 * Replaces gemv_topk_kernel as launched at gemv_topk.cu:466-469: top `top_c` centroids per head,
 * then top `k` tokens inside each chosen cluster of `cluster_len` consecutive tokens;
 * out[h][r*k + i] = c_r*cluster_len + local_i  (gemv_topk.cu:372-378).  No scaling in the reference;
 * `scale` multiplies both levels.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_cluster_topk_args {
  const void* q;          /* device [num_heads][128]                                          */
  const void* centers;    /* device [num_heads][num_centers][128]                             */
  const void* keys;       /* device [num_centers*cluster_len][num_heads][128] via strides     */
  int32_t dtype;
  int32_t num_heads;
  int32_t num_centers;
  int32_t top_c;
  int32_t cluster_len;
  int32_t k;
  int32_t head_dim;
  float scale;
  int64_t key_stride_n;
  int64_t key_stride_h;
  int32_t* out_idx;       /* device [num_heads][top_c*k]                                      */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_cluster_topk_args;

size_t tka_cluster_gemv_topk_workspace_bytes(const tka_cluster_topk_args* args);
int tka_cluster_gemv_topk(const tka_cluster_topk_args* args);

/* ------------------------------------------------------------------------------------------------
 * Index-set helper: per (batch, kv head) the ascending duplicate-free union of the selected ids with
 * the sink range [0, sink) and the local window [seq_len-local, seq_len).  No counterpart in the
 * reference (its selections never overlap); needed so a token is never weighted twice.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_index_union_args {
  const int32_t* idx;     /* device [num_segments][k]                                         */
  int32_t num_segments;
  int32_t k;
  int32_t sink;
  int32_t local;
  int64_t seq_len;
  int32_t* out_idx;       /* device [num_segments][k + sink + local], ascending, tail = -1    */
  int32_t* out_count;     /* device [num_segments]                                            */
  void* stream;
} tka_index_union_args;

int tka_index_union(const tka_index_union_args* args);

/* ------------------------------------------------------------------------------------------------
 * Stage 3 (and the attention half of stage 2) — split-K flash-decoding.
 * Replaces the MHAFlashDecodeKernel launch of baseline_1.cu:689-692 / flash_decoding.cu:462-466
 * (grid heads*cluster x 128, output pre-zeroed, half atomicAdd) with partial kernels that write fp32
 * (m, l, acc) per split and a combine kernel that writes the output once.
 * kv_idx == NULL: dense attention over [0, seq_len).
 * kv_idx != NULL: attention over the listed tokens only (gathered rows); list h of batch b has
 *                 kv_count ? kv_count[b*num_kv_heads+h] : idx_len  valid entries.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_flash_decode_args {
  const void* q;          /* device [batch][num_kv_heads*group][128]                          */
  const void* keys;       /* device; row (b,t,h) as in tka_gemv_topk_args                     */
  const void* values;     /* device; same strides as keys                                     */
  void* out;              /* device [batch][num_kv_heads*group][128], out_dtype               */
  int32_t dtype;          /* of q, keys, values                                               */
  int32_t out_dtype;
  int32_t batch;
  int32_t num_kv_heads;
  int32_t group;
  int32_t head_dim;
  int32_t num_splits;     /* workgroups per (batch, kv head); 0 = choose                      */
  int32_t softmax_mode;   /* tka_softmax_mode                                                 */
  int64_t seq_len;
  int64_t q_stride_b;
  int64_t out_stride_b;
  int64_t kv_stride_b;    /* 0 = shared by the batch                                          */
  int64_t kv_stride_n;
  int64_t kv_stride_h;
  float scale;
  int32_t idx_len;        /* row length of kv_idx                                             */
  const int32_t* kv_idx;  /* device [batch][num_kv_heads][idx_len] or NULL                    */
  const int32_t* kv_count;/* device [batch][num_kv_heads] or NULL                             */
  const float* kv_logit;  /* device [batch][num_kv_heads][idx_len] or NULL: logits supplied by
                             the caller instead of q.k (requires group == 1 and kv_idx);
                             the hand-off of retrieval_attention.cu:1232-1237                 */
  float* out_lse;         /* device [batch][num_kv_heads*group] natural-log LSE; may be NULL  */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_flash_decode_args;

size_t tka_flash_decode_workspace_bytes(const tka_flash_decode_args* args);
int tka_flash_decode(const tka_flash_decode_args* args);

/* Combine alone: out[r][d] = sum_s acc[r][s][d]*2^(m[r][s]-M) / sum_s l[r][s]*2^(m[r][s]-M),
 * M = max_s m[r][s]; m is in the base-2 domain, a split with l == 0 contributes nothing.
 * Replaces the DSM ring max/sum and half atomicAdd of flash_decoding.cu:325-387. */
typedef struct tka_lse_combine_args {
  const float* part_m;    /* device [rows][num_splits]                                        */
  const float* part_l;    /* device [rows][num_splits]                                        */
  const float* part_acc;  /* device [rows][num_splits][128]                                   */
  int32_t rows;           /* batch * query heads                                              */
  int32_t num_splits;
  int32_t out_dtype;
  int32_t reserved0;
  void* out;              /* device [rows][128]                                               */
  float* out_lse;         /* device [rows] natural-log LSE; may be NULL                       */
  void* stream;
} tka_lse_combine_args;

int tka_lse_combine(const tka_lse_combine_args* args);

/* ------------------------------------------------------------------------------------------------
 * Stage 2 — the retrieval_attention op, general form.
 * One call = chunked GEMV + per-chunk top-k + softmax over the num_chunks*k survivors + gathered
 * P.V, i.e. retrieval_topk_kernel + retrieval_reduce_kernel (retrieval_attention.cu:1162-1339).
 * The reference's six hand-off variants compute the same function and map onto this one path.
 * The caches are shared by the batch (retrieval_attention.cu:681-683); where the reference pipelines the batch
 * entries through one cluster (retrieval_attention.cu:654-896), this call reads the keys once per tile of up to
 * eight entries.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_ra_args {
  const void* q;          /* device [batch][num_heads][128]                                   */
  const void* keys;       /* device [seq_len][num_heads][128] shared by the batch             */
  const void* values;     /* device [seq_len][num_heads][128]                                 */
  void* out;              /* device [batch][num_heads][128], same dtype                       */
  int32_t dtype;
  int32_t batch;
  int32_t num_heads;
  int32_t head_dim;
  int32_t topk_per_chunk; /* reference: 32, 128, 256, 512, 1024                               */
  int32_t num_chunks;     /* reference: 4                                                     */
  int32_t softmax_mode;   /* reference: TKA_SOFTMAX_RAW_EXP                                   */
  int32_t bench_print;    /* 1: print the reference's "Avg time ... Throughput" line
                             (retrieval_attention.cu:1610) after a blocking timed rerun       */
  int64_t seq_len;        /* reference: 8192                                                  */
  float scale;            /* reference: 1.0f                                                  */
  int32_t score_mode;     /* tka_score_mode of the scoring stage; 0 = canonical               */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_ra_args;

size_t tka_retrieval_attention_workspace_bytes(const tka_ra_args* args);
int tka_retrieval_attention(const tka_ra_args* args);

/* ------------------------------------------------------------------------------------------------
 * End-to-end sparse decode step: GEMV + top-k per KV head (scores summed over the query group),
 * union with `sink` first and `local` last tokens, gathered attention with online softmax for every
 * query head.  The composition the reference runs as two launches in baseline_1.cu:689-699.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tka_sparse_decode_args {
  const void* q;          /* device [batch][num_kv_heads*group][128]                          */
  const void* keys;       /* device [batch][seq_len][num_kv_heads][128] via strides           */
  const void* values;
  void* out;              /* device [batch][num_kv_heads*group][128], out_dtype               */
  int32_t dtype;
  int32_t out_dtype;
  int32_t batch;
  int32_t num_kv_heads;
  int32_t group;
  int32_t head_dim;
  int32_t k;
  int32_t sink;
  int32_t local;
  int32_t num_splits;     /* of the sparse attention; 0 = choose                              */
  int64_t seq_len;
  int64_t q_stride_b;
  int64_t out_stride_b;
  int64_t kv_stride_b;
  int64_t kv_stride_n;
  int64_t kv_stride_h;
  float scale;
  int32_t reserved0;
  int32_t* out_topk_idx;  /* device [batch][num_kv_heads][k] rank order; may be NULL (saves a sort) */
  float* out_topk_val;    /* device, same shape; may be NULL; needs out_topk_idx              */
  int32_t* out_union_idx; /* device [batch][num_kv_heads][k+sink+local], ascending, -1 behind the count; may be NULL
                             (the step then hands the tokens to the attention in whatever form its route selects them) */
  int32_t* out_union_count;/* device [batch][num_kv_heads]; may be NULL; needs out_union_idx (TKA_EINVAL otherwise) */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
} tka_sparse_decode_args;

size_t tka_sparse_decode_workspace_bytes(const tka_sparse_decode_args* args);
int tka_sparse_decode_step(const tka_sparse_decode_args* args);
/* The same step for callers that cannot allocate device memory and bring no workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * launchers allocate and free their scratch inside every call (retrieval_attention.cu:1658-1659,1978-1979).
 * `workspace` and `workspace_bytes` are ignored: the temporaries live in a buffer of TKA_NOALLOC_SCRATCH_BYTES
 * (128 MiB) that is part of the library's device code - every GPU the library runs on holds one from load to
 * process exit - and the call itself allocates nothing.  A call whose tka_sparse_decode_workspace_bytes() is
 * larger returns TKA_ESCRATCH before anything is launched (batch 8 x 8 KV heads x 131072 tokens, k = 2048 needs
 * 102 MiB; 8 heads x 1048576 tokens, k = 4096 needs 98 MiB).  Outputs are identical to tka_sparse_decode_step's.
 * All calls on one GPU share that one buffer: two calls may only overlap in time if they run on different
 * GPUs; on one GPU they must be ordered (one stream, or events between streams), otherwise they race.
 * The buffer's address on a GPU is looked up by the first call made with that GPU current (which must also be the
 * GPU of args->stream): make that first call outside any stream capture; later calls may be captured and replayed. */
int tka_sparse_decode_step_noalloc(const tka_sparse_decode_args* args);

/* Diagnostic, as tka_gemv_topk_redone_segments: segments of the last step with these arguments (same workspace)
 * that the selection kernel redid from the keys.  Waits for the stream. */
int tka_sparse_decode_redone_segments(const tka_sparse_decode_args* args, int32_t* count);

/* ------------------------------------------------------------------------------------------------
 * Read probes (measurement; no counterpart in the reference): launch a kernel that only READS a KV cache in the
 * access pattern of one of the two kernels that carry the bytes of the decode step, so that their achieved
 * bandwidth can be set against what the memory system gives to that pattern on the same machine.
 *   TKA_PROBE_STREAM  every row of every (batch entry, head), one head per workgroup, `threads` (256 or 512) threads,
 *                     `rounds` rounds of eight 16-byte loads per lane (512 x 2 is the shape of the long-segment GEMV);
 *   TKA_PROBE_GATHER  the K and V rows of the token lists idx[batch][num_heads][idx_len] (ids outside the cache read
 *                     row 0), `tokens_per_wg` ids per workgroup: the pattern of the gathered attention.
 * Nothing is written but, never in practice, the word `sink`.  Asynchronous on `stream`; time it with events.
 * ---------------------------------------------------------------------------------------------- */
typedef enum tka_probe_kind { TKA_PROBE_STREAM = 0, TKA_PROBE_GATHER = 1 } tka_probe_kind;
typedef struct tka_probe_args {
  const void* keys;       /* device; row (b,t,h) at keys + b*kv_stride_b + t*kv_stride_n + h*kv_stride_h (elements of 2 bytes) */
  const void* values;     /* device; gather only, same strides                                 */
  const int32_t* idx;     /* device; gather only                                               */
  uint32_t* sink;         /* device; one word                                                  */
  int32_t kind;           /* tka_probe_kind                                                    */
  int32_t batch;
  int32_t num_kv_heads;
  int32_t idx_len;        /* gather: ids per list                                              */
  int32_t threads;        /* stream: 256 or 512                                                */
  int32_t rounds;         /* stream: 1 .. 64                                                   */
  int32_t nontemporal;    /* stream: 1 = loads with the streaming hint (what the GEMV uses)    */
  int32_t tokens_per_wg;  /* gather: ids per workgroup (a multiple of 128)                     */
  int64_t seq_len;
  int64_t kv_stride_b;
  int64_t kv_stride_n;
  int64_t kv_stride_h;
  void* stream;
} tka_probe_args;
int tka_probe_read(const tka_probe_args* args);

/* ------------------------------------------------------------------------------------------------
 * Per-kernel timing.  When enabled, every kernel launch made by this library is bracketed by a pair
 * of HIP events recorded on the launch stream; tka_profile_read() synchronises those events and
 * accumulates elapsed time per kernel name.  Process-wide, not thread-safe; off by default.
 * ---------------------------------------------------------------------------------------------- */
int tka_profile_enable(int on);
int tka_profile_reset(void);
/* Returns the number of distinct kernels seen (<= cap); fills names[i] (static strings),
 * total_ms[i], launches[i]. */
int tka_profile_read(const char** names, double* total_ms, int64_t* launches, int cap);

#ifdef __cplusplus
}
#endif

/* The thirty reference-named launchers of the retrieval_attention op (bind.cpp:5-243) are declared in
 * topk_attn_ra_launchers.h. */

#endif /* TOPK_ATTN_H_ */
