// Parameter blocks and launch functions of the device kernels (internal to the library).
#pragma once
#include "common.hpp"

namespace tka {

// ---- stage 1: GEMV ----------------------------------------------------------------------------
struct GemvParams {
  const void* q;        // [batch][num_kv_heads*group][128]
  const void* keys;
  float* scores;        // [batch][num_kv_heads][num_chunks][chunk_len]; selection kernels also read them
  const int32_t* cluster_ids;  // [batch*num_kv_heads*num_chunks] or nullptr: chunk c covers the tokens of that cluster
  // two-level selection with the centre stage inside the GEMV launch (gemv_scores_kernel only): chunk c of head h
  // covers the cluster whose centroid has rank c among centers[h], and the id is also written to cluster_ids_out
  const void* centers;         // [num_kv_heads][num_centers][128] or nullptr
  int32_t* cluster_ids_out;    // [num_kv_heads*num_chunks]
  int num_centers;             // <= kGemvInlineCentres
  uint32_t* hist;       // [batch*num_kv_heads*num_chunks][kHistBins] or nullptr; must be zero on entry
  // candidate mode: only tokens whose key reaches the segment's sampled threshold are stored
  uint64_t* tau_words;        // [segments][2] (epoch << 32) | threshold key, and the token cut among keys equal to it
  uint32_t* sample_flags;     // [segments][64] epoch of the call in which that sampling workgroup last arrived
  uint32_t* sample_pool;      // [segments][num_samples] keys of the sampled tokens
  uint32_t epoch;             // tells this call's words from older contents of the workspace (never 0)
  uint32_t* seg_flags;        // [segments] a streaming workgroup whose wait for the threshold expired stores the epoch here
  int tau_spin_limit;         // polls of a streaming workgroup for its threshold before it gives up
  // testing (tka_test_hooks): the threshold of segments with seg % withhold_mod == withhold_rem is never published
  // (mode 0) or published only once a slice of the segment has given up, after a bounded wait (mode 1); 0 = off
  int withhold_mod, withhold_rem, withhold_mode;
  int num_samples, sample_rank;   // per segment
  int interleave_segs;        // the same kernel: consecutive scoring workgroups take the same tokens of consecutive segments
  int samplers_score;         // gemv_cut_slices_kernel with front sampling: the sampling workgroups go on to score tokens like the others
  uint64_t split_ranks;       // common-cut route: byte g - 1 holds the 1-based rank of the sample that ends part g of the candidates
                              // (ascending; byte kCutParts - 1 equals sample_rank), see gemv_cut_split_ranks
  int sample_wgs;             // sampling workgroups at the front of the candidate grid (set by the launcher)
  int early_wgs;              // streaming workgroups behind them that take several slices each (set by the launcher)
  uint64_t* cand;             // [segments][wgs_per_chunk][tokens_per_wg] one slice per workgroup, ascending index:
                              // key << 32 | count << 9 | token offset in the slice (count in entry 0 only)
  int64_t cand_seg_stride;    // entries between the slice arrays of consecutive segments
  uint64_t* cand_head;        // [segments][wgs_per_chunk][kCandHead] entries 0 .. kCandHead-1 of every slice, densely packed:
                              // an ordinary slice (about 18 candidates) lies here whole, two full lines that stay in the
                              // L2 until the kernel ends; `cand` only takes what goes beyond (heavy ties)
  uint32_t* cand_count;       // common-cut route: [segments][wgs_per_chunk] candidates of every slice
  uint64_t* cut_splits;       // common-cut route: [segments][kCutParts] composites of the samples that end the parts of the
                              // candidates in rank order; the last one is the cut itself
  int64_t chunk_len;    // tokens per chunk
  int64_t q_stride_b, key_stride_b, key_stride_n, key_stride_h;
  int batch, num_kv_heads, group, num_chunks;
  int wgs_per_chunk, tokens_per_wg;
  float scale;
};
int launch_gemv_scores(const GemvParams& p, int dtype, hipStream_t stream);
// Keys shared by the batch (key_stride_b == 0): one pass over the keys scores several batch entries; plain scores only.
int launch_gemv_scores_shared(const GemvParams& p, int dtype, hipStream_t stream);
// The same on the matrix cores (one query head per KV head): scores to a few units in the last place of the canonical ones.
int launch_gemv_scores_mfma(const GemvParams& p, int dtype, hipStream_t stream);
int launch_gemv_candidates(const GemvParams& p, int dtype, hipStream_t stream);   // thresholds + candidate slices
// The same over keys shared by the batch (key_stride_b == 0, batch >= 2): one pass over the keys scores a tile of batch entries.
int launch_gemv_candidates_shared(const GemvParams& p, int dtype, hipStream_t stream);
void gemv_candidate_plan(int64_t chunk_len, int64_t total_rows, int k, int max_candidates, int* num_samples, int* sample_rank);
int gemv_tokens_per_wg(int64_t total_rows, int64_t chunk_len);
// Common-cut route: every workgroup derives the segment's cut from the same sample rows and stores its slice's candidates
// (p.cand_head: the first kCutHead of a slice as composites, zeros behind; p.cand: the rest; p.cand_count; p.num_samples /
// p.sample_rank and the slice length p.tokens_per_wg from gemv_cut_plan; p.wgs_per_chunk: the slices of a segment).
int launch_gemv_cut(const GemvParams& p, int dtype, hipStream_t stream);
// The same for calls that fill the GPU: the first workgroups of the launch, one per segment, find the cut and the part ends and
// announce them; the GEMV workgroups (512 tokens each) score nothing twice.
int launch_gemv_cut_slices(const GemvParams& p, int dtype, hipStream_t stream);
// sampled_once: the plan for launch_gemv_cut_slices (kCutSamplesOnce samples) instead of launch_gemv_cut (256).
void gemv_cut_plan(int64_t chunk_len, int k, bool sampled_once, int* num_samples, int* sample_rank, int* slice_len);
uint64_t gemv_cut_split_ranks(int64_t chunk_len, int k, int num_samples, int sample_rank);

// ---- stage 1: selection -----------------------------------------------------------------------
struct SelectParams {
  const float* scores;    // segment s starts at scores + s*seg_stride
  int64_t seg_len;
  int64_t seg_stride;
  uint32_t* hist;         // [num_segments][kHistBins]; nullptr: the lists hold candidates above a sampled threshold
  uint64_t* tau_words;    // [num_segments][2] candidate thresholds (workspace); the candidate selection kernel clears them
  uint32_t* sample_flags; // [num_segments][64] arrival flags of the sampling workgroups (workspace)
  uint32_t* sample_pool;  // [num_segments][kGemvMaxSamples] sampled keys (workspace)
  uint32_t* seg_flags;    // [num_segments] candidate mode: bit 0 = the segment was redone from the keys, bits 8.. = how many
                          // of its slices came from workgroups whose wait for the threshold had expired
  uint32_t* redo_queue;   // candidate route: the item counters of launch_redo_segments (drawn, done per phase)
  uint32_t* redo_rec;     // ... its record per segment: 16 words, then four per chunk of 4096 tokens
  int64_t redo_rec_stride;
  uint32_t* redo_hist;    // candidate route: [num_segments][kHistBins]; set = a flagged segment is left to launch_redo_segments
  int max_entries;        // candidate mode: a segment with more candidates than this is also redone from the keys
  int from_keys;          // candidate selection kernel: no slices, the workgroup scores its (short) segment itself
  int from_scores;        // candidate selection kernel: no slices, the entries are all scores of the segment (<= 16384)
  uint32_t* list_cnt;     // [num_segments][parts] entries in each slice list (finalize turns them into offsets)
  uint64_t* list;         // [num_segments][list_stride] composites with bin >= threshold bin, slice p at p*part_len
  const uint64_t* cand_head;  // candidate mode: [num_segments][parts][kCandHead] the first entries of every slice
  const uint64_t* cut_splits; // common-cut route: [num_segments][kCutParts], see GemvParams
  int64_t list_stride;
  int32_t* out_idx;       // [num_segments][out_stride] rank order, or nullptr (no sort)
  float* out_val;         // same shape or nullptr
  int32_t* out_expand;    // [num_segments][k*expand] or nullptr (centre-only expansion)
  int32_t* union_idx;     // [num_segments][k+sink+local] ascending union with sink/local ranges, or nullptr
  int32_t* union_count;   // [num_segments]
  const int32_t* seg_base_ids;  // nullptr, or per segment a cluster id: index base = id * seg_len
  int64_t out_stride;
  int num_segments;
  int k;
  int parts;              // workgroups (slices) per segment
  int part_len;           // scores per slice: 4096 or 16384
  int segs_per_row;       // chunks per (batch, head): index base = (s % segs_per_row) * seg_len
  int expand;             // cluster_len of the expansion, 0 = none
  int sink, local;        // union mode
  int union_handoff;      // the union list only goes to the attention kernels: any order, and -1 (an id they skip) may stand
                          // inside the count (select_wave_kernel, select_rank_kernel)
  int unordered;          // select_wave kernel: out_idx / out_val need not be in rank order
};
size_t select_workspace_bytes(int num_segments, int64_t seg_len);
// Carves the workspace; returns how many leading 32-bit words (the histograms) need clearing.
size_t select_carve(void* ws, int num_segments, int64_t seg_len, SelectParams* p);
size_t select_epoch_words(void* ws, int num_segments, int64_t seg_len, uint32_t** words);
void select_plan(int64_t seg_len, int num_segments, SelectParams* p);
int launch_zero_u32(uint32_t* ptr, size_t count, hipStream_t stream);
// Raises a kernel's dynamic-LDS limit once per (kernel, device); safe to call from several host threads.
int allow_dynamic_lds(const void* kernel, int bytes);
int launch_select_hist(const SelectParams& p, hipStream_t stream);
int launch_select(const SelectParams& p, hipStream_t stream);   // filter + finalize
int launch_select_filter(const SelectParams& p, hipStream_t stream);
int launch_select_finalize(const SelectParams& p, hipStream_t stream);
// Candidate slices -> outputs; a segment whose slices cannot be used is redone from the keys by its workgroup.
int launch_select_finalize_cand(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream);
bool redo_segments_fits(const GemvParams& g, int num_segments);   // chunks of key rows addressed with 32-bit offsets, flagged segments listed in LDS
int launch_redo_segments(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream);
int select_cand_max_parts();   // most candidate slices per segment
// Common-cut route: ranks the candidates of a segment by counting and writes the top k in rank order (and the expansion);
// p.list / p.list_stride / p.parts describe the slices written by launch_gemv_cut.
int launch_select_rank(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream);
int select_cand_capacity();    // most candidates per segment
// One workgroup per segment, keys in registers: rank-ordered top-k of fp32 scores, segments of up to
// select_wave_max_len() scores, k up to select_wave_max_k(segment length).
int launch_select_wave(const SelectParams& p, hipStream_t stream);
int select_wave_max_len();
int select_wave_max_k(int64_t seg_len);

// One workgroup per segment of up to select_small_max_len() scores, k up to select_small_max_k(), rank order: a short
// program for calls of a few segments.
int launch_select_small(const SelectParams& p, hipStream_t stream);
int launch_gemv_select_small(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream);   // scores its segments itself
int select_small_max_len();
int select_small_max_k();

struct UnionParams {
  const int32_t* idx;     // [num_segments][k]
  int32_t* out_idx;       // [num_segments][k+sink+local]
  int32_t* out_count;     // [num_segments]
  int64_t seq_len;
  int num_segments, k, sink, local;
};
int launch_index_union(const UnionParams& p, hipStream_t stream);

// ---- stages 2/3: attention --------------------------------------------------------------------
struct AttnParams {
  const void* q;
  const void* keys;
  const void* values;
  const int32_t* kv_idx;    // [batch][num_kv_heads][idx_len] or nullptr (dense)
  const int32_t* kv_count;  // [batch][num_kv_heads] or nullptr
  const float* kv_logit;    // [batch][num_kv_heads][idx_len] or nullptr
  float* part_m;            // [rows][num_splits]
  float* part_l;            // [rows][num_splits]
  float* part_acc;          // [rows][num_splits][128]
  int64_t seq_len;
  int64_t q_stride_b, kv_stride_b, kv_stride_n, kv_stride_h;
  int batch, num_kv_heads, group, num_splits;
  int idx_len;
  int tokens_per_split;     // positions per workgroup
  int head_fastest;         // matrix-core kernel: the grid's x counts the KV heads and its y the splits (set by its launcher)
  float scale_log2e;        // scale * log2(e)
  // One split per row: the VALU kernel normalises and writes the result itself (no combine launch) when out is set.
  void* out;                // [batch][query heads][128] or nullptr
  float* out_lse;           // [rows] or nullptr
  int64_t out_stride_b;
  int out_dtype;
};
int launch_attn_partial(const AttnParams& p, int dtype, hipStream_t stream);       // VALU path (any group, logits)
int launch_attn_partial_mfma(const AttnParams& p, int dtype, hipStream_t stream);  // matrix-core path, group >= 2

// Selection and attention of the candidate route in one launch (attention_select.hip): every attention workgroup
// derives its segment's k-th largest composite from the candidate slices of the GEMV launch and keeps its split's
// share of the token list in LDS.  A segment whose candidates cannot be used gets empty partials and bit 0 of its
// seg_flags word; launch_lse_combine_redo then redoes it from the keys.
struct FusedSelectParams {
  const uint64_t* cand_head;  // [segments][parts][kCandHead], see GemvParams
  const uint64_t* cand;       // [segments][cand_seg_stride]
  int64_t cand_seg_stride;
  uint64_t* tau_words;        // [segments][2]  cleared by split 0 of every segment, like the selection kernel does
  uint32_t* sample_flags;     // [segments][64]
  uint32_t* seg_flags;        // [segments] bit 0: to be redone from the keys; bits 8..: slices that gave up
  int parts, part_len;        // slices per segment, tokens per slice
  int k, sink, local;
  int max_entries;            // a segment with more candidates is redone (0: every segment, the testing hook)
  int lds_entries;            // candidates of a segment that a workgroup keeps in LDS (set by the launcher)
};
bool attn_select_fits(int parts, int group);
int launch_attn_select_mfma(const AttnParams& p, const FusedSelectParams& f, int dtype, hipStream_t stream);

struct CombineParams {
  const float* part_m;
  const float* part_l;
  const float* part_acc;
  void* out;
  float* out_lse;
  int64_t out_stride_b;     // elements between batch entries of out
  int rows_per_batch;       // query heads
  int rows, num_splits, out_dtype;
};
int launch_lse_combine(const CombineParams& p, hipStream_t stream);
// The combine launch behind launch_attn_select_mfma: rows of unflagged segments are combined as usual; behind them in
// the grid one workgroup per segment looks at the segment's flag and, when it is set, redoes the segment from the keys
// (selection by fallback_segment into s.union_idx / s.union_count, attention over that list, output written directly).
// g, s: the stage-1 parameters of the step (s.out_idx must be null: no rank order); a: q, values, strides, scale.
int launch_lse_combine_redo(const CombineParams& c, const GemvParams& g, const SelectParams& s, const AttnParams& a, int dtype,
                            hipStream_t stream);

// ---- read probes (probes.hip) ------------------------------------------------------------------
struct ProbeParams {
  const void* base;     // rows of 256 bytes: row (b, t, h) at base + 2 * (b * stride_b + t * stride_n + h * stride_h)
  const void* base2;    // gather: the second cache (values)
  const int32_t* idx;   // gather: [batch][num_heads][idx_len] token ids
  uint32_t* sink;       // one word that no run writes (it keeps the loads alive)
  int64_t seq_len, stride_b, stride_n, stride_h;
  int batch, num_heads, idx_len;
};
int launch_probe_stream(const ProbeParams& p, int threads, int rounds, bool nontemporal, hipStream_t stream);
int launch_probe_gather(const ProbeParams& p, int tokens_per_wg, hipStream_t stream);

}  // namespace tka
