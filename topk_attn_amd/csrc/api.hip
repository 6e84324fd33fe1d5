// C ABI of the library: argument validation (before any HIP call), workspace carving, launch sequence.
#include <atomic>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <string>
#include <vector>

#include "kernels.hpp"

// Scratch of tka_sparse_decode_step_noalloc: device memory that belongs to the loaded code object, one copy per
// GPU, there from the moment the library is loaded on that GPU until the process ends.  In host code this name is
// only a handle for hipGetSymbolAddress (noalloc_scratch below); kernels get the address it returns.
static __device__ __align__(256) unsigned char scratch[TKA_NOALLOC_SCRATCH_BYTES];

namespace tka {

// ---- per-kernel timing ------------------------------------------------------------------------

namespace {
struct TimedLaunch {
  const char* name;
  hipEvent_t start, stop;
};
bool g_profile_on = false;
std::vector<TimedLaunch> g_pending;
std::vector<hipEvent_t> g_event_pool;
struct KernelTotal {
  const char* name;
  double ms;
  int64_t launches;
};
std::vector<KernelTotal> g_totals;
std::mutex g_profile_mutex;

hipEvent_t take_event() {
  if (!g_event_pool.empty()) {
    hipEvent_t e = g_event_pool.back();
    g_event_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}

void drain_pending() {
  for (TimedLaunch& t : g_pending) {
    float ms = 0.0f;
    if (hipEventSynchronize(t.stop) == hipSuccess && hipEventElapsedTime(&ms, t.start, t.stop) == hipSuccess) {
      KernelTotal* slot = nullptr;
      for (KernelTotal& k : g_totals)
        if (strcmp(k.name, t.name) == 0) slot = &k;
      if (!slot) {
        g_totals.push_back({t.name, 0.0, 0});
        slot = &g_totals.back();
      }
      slot->ms += ms;
      slot->launches += 1;
    }
    g_event_pool.push_back(t.start);
    g_event_pool.push_back(t.stop);
  }
  g_pending.clear();
}
}  // namespace

LaunchTimer::LaunchTimer(const char* name, hipStream_t stream) : name_(name), stream_(stream), slot_(nullptr) {
  if (!g_profile_on) return;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  hipEvent_t s = take_event(), e = take_event();
  if (!s || !e) return;
  g_pending.push_back({name, s, e});
  slot_ = (void*)e;
  (void)hipEventRecord(s, stream);
}

LaunchTimer::~LaunchTimer() {
  if (slot_) (void)hipEventRecord((hipEvent_t)slot_, stream_);
}

// ---- validation helpers -----------------------------------------------------------------------

namespace {

// Testing hooks (tka_set_test_hooks): process-wide, read once per call.
std::mutex g_hooks_mutex;
tka_test_hooks g_hooks = {0, 0, 0, 0, 0, 0, 0};
tka_test_hooks current_hooks() {
  std::lock_guard<std::mutex> lock(g_hooks_mutex);
  return g_hooks;
}

bool dtype_ok(int d) { return d == TKA_F16 || d == TKA_BF16; }
bool group_ok(int g) { return g == 1 || g == 2 || g == 4 || g == 8; }
bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

int check_gemv(const tka_gemv_topk_args* a, bool need_topk) {
  if (!a) return TKA_EINVAL;
  if (!a->q || !a->keys) return TKA_EINVAL;
  if (a->head_dim != TKA_HEAD_DIM || !dtype_ok(a->dtype) || !group_ok(a->group)) return TKA_EUNSUPPORTED;
  if (a->batch < 1 || a->num_kv_heads < 1 || a->seq_len < 1 || a->num_chunks < 1) return TKA_EINVAL;
  if (a->score_mode != TKA_SCORE_CANONICAL && a->score_mode != TKA_SCORE_MATRIX) return TKA_EUNSUPPORTED;
  if (a->reserved1 != 0) return TKA_EINVAL;   // reserved fields must be zero
  if (a->batch > 65535 || a->num_kv_heads > 65535) return TKA_EUNSUPPORTED;
  if (a->seq_len > 0x7fffffffLL) return TKA_EUNSUPPORTED;  // token ids are int32
  if (a->seq_len % a->num_chunks != 0) return TKA_EINVAL;
  if (a->key_stride_n < TKA_HEAD_DIM || a->key_stride_h < 0 || a->key_stride_b < 0 || a->q_stride_b < 0) return TKA_EINVAL;
  if ((a->key_stride_n | a->key_stride_h | a->key_stride_b | a->q_stride_b) & 7) return TKA_EINVAL;  // 16-byte rows
  if (!aligned16(a->q) || !aligned16(a->keys)) return TKA_EINVAL;
  if (a->batch > 1 && a->q_stride_b < (int64_t)a->num_kv_heads * a->group * TKA_HEAD_DIM) return TKA_EINVAL;
  if (need_topk) {
    if (!a->out_idx) return TKA_EINVAL;
    if (a->k < 1 || a->k > a->seq_len / a->num_chunks) return TKA_EINVAL;
    if (a->k > TKA_MAX_TOPK) return TKA_EUNSUPPORTED;
  } else if (!a->out_scores) {
    return TKA_EINVAL;
  }
  if (a->score_mode == TKA_SCORE_MATRIX && (a->batch >= 1 && a->num_kv_heads >= 1) &&
      !(a->group == 1 && a->key_stride_b == 0 && a->batch >= 2 && (!need_topk || a->seq_len / a->num_chunks <= 16384)))
    return TKA_EUNSUPPORTED;
  return TKA_OK;
}

// TKA_SCORE_MATRIX is served where keys are shared by a batch of at least two entries, one query head per KV head, and the
// scores are written out whole (the GEMV alone, or chunks of up to 16384 keys); a call that asks for it elsewhere is refused
// rather than silently scored in the canonical order.
bool matrix_scores_apply(const tka_gemv_topk_args* a) {
  return a->group == 1 && a->key_stride_b == 0 && a->batch >= 2;
}

size_t gemv_scores_bytes(const tka_gemv_topk_args* a) {
  return a->out_scores ? 0 : align_up((size_t)a->batch * a->num_kv_heads * (size_t)a->seq_len * sizeof(float), 256);
}

void fill_gemv_params(const tka_gemv_topk_args* a, float* scores, uint32_t* hist, GemvParams* g) {
  g->q = a->q;
  g->keys = a->keys;
  g->scores = scores;
  g->hist = hist;
  g->cluster_ids = nullptr;
  g->centers = nullptr;
  g->cluster_ids_out = nullptr;
  g->num_centers = 0;
  g->chunk_len = a->seq_len / a->num_chunks;
  g->q_stride_b = a->q_stride_b;
  g->key_stride_b = a->key_stride_b;
  g->key_stride_n = a->key_stride_n;
  g->key_stride_h = a->key_stride_h;
  g->batch = a->batch;
  g->num_kv_heads = a->num_kv_heads;
  g->group = a->group;
  g->num_chunks = a->num_chunks;
  g->scale = a->scale;
  g->tau_words = nullptr;
  g->sample_flags = nullptr;
  g->sample_pool = nullptr;
  g->epoch = 0;
  g->seg_flags = nullptr;
  g->tau_spin_limit = kTauSpinLimit;
  g->withhold_mod = g->withhold_rem = g->withhold_mode = 0;
  g->num_samples = g->sample_rank = g->sample_wgs = g->early_wgs = 0;
  g->split_ranks = 0;
  g->samplers_score = g->interleave_segs = 0;
  g->cand = nullptr;
  g->cand_seg_stride = 0;
  g->cand_head = nullptr;
  g->cand_count = nullptr;
  g->cut_splits = nullptr;
  const int64_t rows = (int64_t)a->batch * a->num_kv_heads * a->seq_len;
  g->tokens_per_wg = gemv_tokens_per_wg(rows, g->chunk_len);
  g->wgs_per_chunk = (int)((g->chunk_len + g->tokens_per_wg - 1) / g->tokens_per_wg);
}

// Segments of up to 16384 scores (k up to 1024, 2048 beyond 4096 scores): one workgroup per segment selects from
// plain scores with the keys in its registers.  Segments of up to 2048 rows that still have to be scored take this
// route only in numbers: a few are quicker scored and selected by one workgroup each in one launch.
constexpr int kWaveSelectMinSegments = 128;
// A small k out of a few thousand scores: one big workgroup per segment with a short program, up to this many segments.
constexpr int kSmallSelectMaxSegments = 64;
bool small_select_fits(int64_t seg_len, int k, int segs) {
  return seg_len > kFusedMaxSegLen && seg_len <= select_small_max_len() && k <= select_small_max_k() && segs <= kSmallSelectMaxSegments;
}
bool wave_select_fits(int64_t seg_len, int k) { return seg_len <= select_wave_max_len() && k <= select_wave_max_k(seg_len); }

// Samples per segment and rank of the threshold statistic when the call takes the candidate route (long segments,
// k a small share of them), else 0.
void candidate_plan(const tka_gemv_topk_args* a, int* num_samples, int* sample_rank) {
  *num_samples = *sample_rank = 0;
  const int64_t chunk_len = a->seq_len / a->num_chunks;
  const int64_t cand_slices = (chunk_len + kGemvCandTokensPerWg - 1) / kGemvCandTokensPerWg;
  // (the candidate kernel addresses the rows of a slice with 32-bit byte offsets)
  if (!a->out_scores && cand_slices <= select_cand_max_parts() && a->key_stride_n < (int64_t)1 << 21)
    gemv_candidate_plan(chunk_len, (int64_t)a->batch * a->num_kv_heads * a->seq_len, a->k, select_cand_capacity(), num_samples, sample_rank);
}

struct UnionOut {
  int32_t* idx;
  int32_t* count;
  int sink, local;
  bool handoff;     // the list only goes to the attention kernels: the selected tokens may come in any order, and -1 (an
                    // id those kernels skip) may stand inside the count
};

// Samples per segment and rank of the cut when the call takes the common-cut route (segments of middling length on
// calls of up to 1572864 rows; rank-ordered output, and the union list for a caller that only hands it to the
// attention), else 0.  Shorter segments are selected from the registers of one workgroup, longer ones (or many of
// them) by the sampling workgroups of the candidate route.
int64_t cut_route_min_len() { return (int64_t)select_cand_capacity() / 2 + 1; }
// Rows of a call beyond which the cut is found once per segment (by the first workgroups of the GEMV launch) instead of in every
// GEMV workgroup: scoring the 256 sample rows beside every 256 tokens is free only while the launch does not fill the
// GPU.  Decode steps, k = 2048, us per step in two / three launches: 1 x 32768 tokens 23.5 / 26.5, 2 x 32768 28.1 / 30.0,
// 1 x 65536 26.3 / 29.5, 3 x 32768 29.3 / 26.8, 4 x 32768 31.3 / 27.7, 8 x 32768 43.0 / 36.2.
constexpr int64_t kCutSplitMinRows = 65536;
// Tells this call's words in a workspace from older contents: never 0, the cleared state; bit 30 stays free for the
// "has a cut" mark of the candidate route's threshold words.
uint32_t next_epoch() {
  static std::atomic<uint32_t> call_counter{0};
  return (call_counter.fetch_add(1, std::memory_order_relaxed) & ~kTauHasCut) | 0x80000000u;
}
void cut_plan(const tka_gemv_topk_args* a, const UnionOut* u, int* num_samples, int* sample_rank, int* slice_len = nullptr) {
  *num_samples = *sample_rank = 0;
  const int64_t chunk_len = a->seq_len / a->num_chunks;
  if ((!a->out_idx && !u) || (u && !u->handoff) || a->out_scores || chunk_len < cut_route_min_len()) return;
  if (a->score_mode == TKA_SCORE_MATRIX) return;   // (the matrix cores score into a plain score array: the routes that select from one)
  const int64_t rows = (int64_t)a->batch * a->num_kv_heads * a->seq_len;
  int s = 0, r = 0, len = 0;
  gemv_cut_plan(chunk_len, a->k, rows > kCutSplitMinRows, &s, &r, &len);
  if (s == 0) return;
  if (slice_len) *slice_len = len;
  // Measured, decode steps with k = 2048 unless said (us per step, this route against the others): 1 x 32768 tokens
  // 21.1 / 32.2, 8 x 32768 30.7 / 43.4, 24 x 32768 54.6 / 68.8, 32 x 32768 67.6 / 73.2, 48 x 32768 94.4 / 95.9,
  // 64 x 32768 118.9 / 118.7, 16 x 49152 55.3 / 70.0, 32 x 49152 89.7 / 92.1, 40 x 20000 (k = 1000) 58.7 / 64.6,
  // 64 x 20000 81.3 / 88.5; segments that would also fit the registers of one workgroup (8193 .. 16384 tokens):
  // 1 x 16384 (k = 1024) 20.8 / 22.0, 8 x 16384 23.8 / 25.6, 8 x 12000 22.0 / 25.6, 16 x 16384 32.1 / 35.2, 32 x 16384
  // 46.1 / 48.3, 48 x 16384 58.8 / 58.9, 96 x 16384 100.4 / 102.2; rank-ordered top-k per call: 8 x 16384 (k = 1024)
  // 14.2 / 20.2, 16 x 16384 (k = 2048) 17.9 / 29.1, 32 x 16384 32.7 / 42.3, 8 x 9000 (k = 512) 13.7 / 15.9.  Up to 8192
  // tokens the registers of one workgroup win (8 x 8192, k = 512: 21.1 / 20.1 per step, 8 x 4096: 20.1 / 17.6).
  if (rows > kCutMaxRows) return;
  // Segments that the candidate route takes as well (65536 tokens): that route beyond sixteen segments
  // (decode steps: 1 x 65536 22.2 / 34.5, 2 x 65536 23.3 / 33.9, 4 x 65536 33.6 / 40.6, 8 x 65536 45.8 / 49.1,
  // 16 x 65536 68.0 / 68.5, 32 x 65536 113.8 / 111.6, 64 x 65536 208.6 / 198.6).
  if (rows > (int64_t)1 << 20 && chunk_len >= 65536) {
    int cs = 0, cr = 0;
    candidate_plan(a, &cs, &cr);
    if (cs != 0) return;
  }
  *num_samples = s;
  *sample_rank = r;
}

// Runs clear + GEMV (+histogram) + select.  `ws` holds [scores][select workspace].
// a->out_idx == nullptr skips the rank-order sort (then `u` must ask for the union list).
// `any_order`: the caller does not need out_idx / out_val in rank order (a route may still deliver it).
// Centre stage of a two-level selection done inside the GEMV launch of the token stage (see wave_route).
struct InlineCentres {
  const void* centers;   // [num_kv_heads][num_centers][128]
  int num_centers;
  int32_t* ids_out;      // [num_kv_heads*num_chunks] chosen cluster per (head, rank)
};

// Plain scores of a batch over one key cache: the matrix cores when the caller opted in, else the canonical order.
int launch_shared_scores(const tka_gemv_topk_args* a, const GemvParams& gp, hipStream_t stream) {
  if (a->score_mode == TKA_SCORE_MATRIX && a->group == 1) return launch_gemv_scores_mfma(gp, a->dtype, stream);
  return launch_gemv_scores_shared(gp, a->dtype, stream);
}

// Segments that fit in the registers of a workgroup: plain scores, then one workgroup per segment selects.
bool wave_route(const tka_gemv_topk_args* a, bool want_union) {
  const int segs = a->batch * a->num_kv_heads * a->num_chunks;
  const int64_t chunk_len = a->seq_len / a->num_chunks;
  return (a->out_idx || want_union) && wave_select_fits(chunk_len, a->k) &&
         (chunk_len > kFusedMaxSegLen || a->out_scores || segs >= kWaveSelectMinSegments);
}

struct FusedTail;
bool fused_tail_take(FusedTail* ft, const GemvParams& g, const SelectParams& s);

// `ft`: the caller can run selection and attention of the candidate route in one launch (launch_attn_select_mfma);
// when the call takes that route and the launch fits, only the GEMV is launched here and *ft is filled.
int run_gemv_topk(const tka_gemv_topk_args* a, int32_t* out_expand, int expand, const int32_t* cluster_ids = nullptr,
                  const UnionOut* u = nullptr, bool any_order = false, const InlineCentres* ic = nullptr, FusedTail* ft = nullptr) {
  hipStream_t stream = (hipStream_t)a->stream;
  const int segs = a->batch * a->num_kv_heads * a->num_chunks;
  const int64_t chunk_len = a->seq_len / a->num_chunks;
  unsigned char* ws = (unsigned char*)a->workspace;
  float* scores = a->out_scores ? a->out_scores : (float*)ws;
  ws += gemv_scores_bytes(a);

  SelectParams sp;
  memset(&sp, 0, sizeof sp);
  const size_t zero_words = select_carve(ws, segs, chunk_len, &sp);
  select_plan(chunk_len, segs, &sp);
  sp.scores = scores;
  sp.seg_len = chunk_len;
  sp.seg_stride = chunk_len;
  sp.out_idx = a->out_idx;
  sp.out_val = a->out_val;
  sp.out_expand = out_expand;
  sp.out_stride = a->k;
  sp.num_segments = segs;
  sp.k = a->k;
  sp.segs_per_row = a->num_chunks;
  sp.expand = expand;
  sp.seg_base_ids = cluster_ids;
  if (u) {
    sp.union_idx = u->idx;
    sp.union_count = u->count;
    sp.sink = u->sink;
    sp.local = u->local;
    sp.union_handoff = u->handoff ? 1 : 0;
  }

  GemvParams gp;
  fill_gemv_params(a, scores, sp.hist, &gp);
  gp.cluster_ids = cluster_ids;

  // Keys shared by the batch are read once for several batch entries.
  const bool shared_keys = a->key_stride_b == 0 && a->batch >= 2 && !cluster_ids;

  // A few segments of middling length: every GEMV workgroup derives the segment's cut from common sample rows and
  // stores its candidates, one workgroup per segment ranks them.
  int cut_samples = 0, cut_rank = 0, cut_slice_len = 0;
  cut_plan(a, u, &cut_samples, &cut_rank, &cut_slice_len);
  if (cut_samples != 0 && !ic) {
    GemvParams cp = gp;
    cp.hist = nullptr;
    cp.tokens_per_wg = cut_slice_len;
    cp.wgs_per_chunk = (int)((chunk_len + cut_slice_len - 1) / cut_slice_len);
    cp.num_samples = cut_samples;
    cp.sample_rank = cut_rank;
    cp.split_ranks = gemv_cut_split_ranks(chunk_len, a->k, cut_samples, cut_rank);
    cp.cand = sp.list;
    cp.cand_seg_stride = sp.list_stride;
    cp.cand_head = const_cast<uint64_t*>(sp.cand_head);
    cp.cand_count = sp.list_cnt;
    cp.cut_splits = (uint64_t*)sp.hist;   // (the histograms of the dense path: 8 KB per segment, free on this route)
    // a call that fills the GPU finds the cut in a launch of its own instead of in every GEMV workgroup
    const int64_t rows = (int64_t)segs * chunk_len;
    int rc;
    if (rows > kCutSplitMinRows) {
      {
        const tka_test_hooks hooks = current_hooks();
        cp.tau_words = sp.tau_words;
        cp.epoch = next_epoch();
        if (hooks.tau_spin_limit > 0) cp.tau_spin_limit = hooks.tau_spin_limit;
        cp.withhold_mod = hooks.tau_withhold_mod > 0 ? hooks.tau_withhold_mod : 0;
        cp.withhold_rem = hooks.tau_withhold_rem;
        // With more scoring workgroups than run at once (two per CU) the sampling ones take tokens of their own
        // afterwards instead of standing in front of the grid as extra workgroups: 0.2-0.4 us off the launch (16 x 16384
        // tokens 34.05 -> 33.8 us per decode step, 8 x 65536 46.7 -> 46.35).  Where all run at once the samplers would then
        // be the last to finish (2 x 65536: 23.35 -> 25.0).
        cp.samplers_score = (int64_t)segs * ((chunk_len + 2 * kCutTokensPerWg - 1) / (2 * kCutTokensPerWg)) > 512 ? 1 : 0;
        // Consecutive scoring workgroups take the same tokens of consecutive segments when the number of segments is a power
        // of two, instead of consecutive tokens of one segment: with sixteen or thirty-two heads a token's rows of one head
        // lie 4 or 8 KB apart, and the workgroups that run together, all on the same few heads, crowd the same memory
        // channels (per decode step, 16 x 32768 tokens 49.3 -> 43.8 us, 32 x 32768 78.8 -> 69.8, 2 x 8 x 32768 44.3 -> 43.0,
        // 16 x 16384 33.9 -> 32.9, 8 x 32768 30.35 -> 30.1; 12 and 24 x 32768 would lose 0.6-0.7 and keep the other order).
        // Also for any number of segments where a head's rows lie a multiple of 4 KB apart (3 x 16 x 32768 tokens 106 -> 95.5).
        cp.interleave_segs = (segs & (segs - 1)) == 0 || (a->key_stride_n * 2) % 4096 == 0 ? 1 : 0;
        rc = launch_gemv_cut_slices(cp, a->dtype, stream);
      }
    } else {
      rc = launch_gemv_cut(cp, a->dtype, stream);
    }
    if (rc != TKA_OK) return rc;
    SelectParams sc = sp;
    sc.hist = nullptr;
    sc.tau_words = cp.tau_words;   // (set when the GEMV launch announced the cuts itself)
    sc.parts = cp.wgs_per_chunk;
    sc.part_len = cut_slice_len;
    sc.max_entries = current_hooks().force_segment_redo ? 0 : kCutMaxSlices * kCutTokensPerWg;   // (no limit of its own)
    sc.scores = scores;
    sc.cut_splits = cp.cut_splits;
    return launch_select_rank(gp, sc, a->dtype, stream);
  }

  if (wave_route(a, u != nullptr)) {
    gp.hist = nullptr;
    SelectParams sw = sp;
    sw.unordered = any_order ? 1 : 0;
    if (ic) {   // the GEMV launch ranks the centroids itself and leaves the chosen ids for the selection
      gp.centers = ic->centers;
      gp.num_centers = ic->num_centers;
      gp.cluster_ids_out = ic->ids_out;
      sw.seg_base_ids = ic->ids_out;
    }
    int rc = shared_keys ? launch_shared_scores(a, gp, stream) : launch_gemv_scores(gp, a->dtype, stream);
    if (rc != TKA_OK) return rc;
    // a small k out of a few thousand scores on a call of a few segments: the short program of one big workgroup
    if (small_select_fits(chunk_len, a->k, segs) && a->out_idx && !u) return launch_select_small(sw, stream);
    return launch_select_wave(sw, stream);
  }
  if (ic) return TKA_EINVAL;   // (callers ask wave_route first)

  // Short segments: one launch, each workgroup scores and selects its own segment.  One CU pulls about
  // 55 GB/s, so beyond 2048 rows (0.5 MB) the separate GEMV launch with many workgroups per segment wins.
  if (!a->out_scores && chunk_len <= kFusedMaxSegLen) {
    // a small k in rank order: the short program (histogram, candidates ranked by counting) instead of a sort of the segment
    // (32 x 1024 centroids, top 64: 10.5 instead of 11.7 us; one workgroup per 4096 rows would take 21.5 against 13.2 in two launches)
    if (a->out_idx && !u && a->k <= select_small_max_k()) return launch_gemv_select_small(gp, sp, a->dtype, stream);
    SelectParams sf = sp;
    sf.from_keys = 1;
    return launch_select_finalize_cand(gp, sf, a->dtype, stream);
  }

  // Segments that fit in LDS whole: GEMV that stores plain scores (no histogram), then one selection launch.
  if (chunk_len <= select_cand_capacity()) {
    gp.hist = nullptr;
    int rc = shared_keys ? launch_shared_scores(a, gp, stream) : launch_gemv_scores(gp, a->dtype, stream);
    if (rc != TKA_OK) return rc;
    SelectParams sw = sp;
    sw.from_scores = 1;
    return launch_select_finalize_cand(gp, sw, a->dtype, stream);
  }

  int num_samples = 0, sample_rank = 0;
  const int64_t cand_slices = (chunk_len + kGemvCandTokensPerWg - 1) / kGemvCandTokensPerWg;
  candidate_plan(a, &num_samples, &sample_rank);
  if (num_samples == 0) {
    // dense: clear histograms, GEMV with histogram, filter, finalize
    int rc = launch_zero_u32(sp.hist, zero_words, stream);
    if (rc != TKA_OK) return rc;
    rc = launch_gemv_scores(gp, a->dtype, stream);
    if (rc != TKA_OK) return rc;
    return launch_select(sp, stream);
  }

  // Long segments: sampled threshold, GEMV that stores candidates only, selection straight from the
  // candidate slices.  A segment whose candidates turn out too few (or too many) is redone from the keys by
  // its selection workgroup.
  GemvParams cp = gp;
  cp.hist = nullptr;
  cp.tokens_per_wg = kGemvCandTokensPerWg;
  cp.wgs_per_chunk = (int)cand_slices;
  cp.tau_words = sp.tau_words;
  cp.sample_flags = sp.sample_flags;
  cp.sample_pool = sp.sample_pool;
  cp.epoch = next_epoch();
  const tka_test_hooks hooks = current_hooks();
  cp.seg_flags = sp.seg_flags;
  if (hooks.tau_spin_limit > 0) cp.tau_spin_limit = hooks.tau_spin_limit;
  cp.withhold_mod = hooks.tau_withhold_mod > 0 ? hooks.tau_withhold_mod : 0;
  cp.withhold_rem = hooks.tau_withhold_rem;
  cp.withhold_mode = hooks.tau_withhold_mode;
  cp.num_samples = num_samples;
  cp.sample_rank = sample_rank;
  cp.cand = sp.list;
  cp.cand_seg_stride = sp.list_stride;
  cp.cand_head = const_cast<uint64_t*>(sp.cand_head);
  // (keys shared by the batch: one pass over them scores a tile of batch entries)
  int rc = shared_keys && a->num_chunks == 1 ? launch_gemv_candidates_shared(cp, a->dtype, stream) : launch_gemv_candidates(cp, a->dtype, stream);
  if (rc != TKA_OK) return rc;
  SelectParams sc = sp;
  sc.hist = nullptr;
  sc.parts = cp.wgs_per_chunk;
  sc.part_len = cp.tokens_per_wg;
  sc.list_stride = sp.list_stride;
  // testing hook: no candidate count is acceptable, every segment is redone from the keys
  sc.max_entries = hooks.force_segment_redo ? 0 : select_cand_capacity();
  sc.scores = scores;
  if (ft && !sc.out_idx && sc.union_idx && a->num_chunks == 1 && !cluster_ids && attn_select_fits(sc.parts, a->group) &&
      fused_tail_take(ft, gp, sc))
    return TKA_OK;
  // A segment that the selection cannot take from its candidates is flagged and redone by the launch behind it, whose
  // workgroups share the work (they leave at once when no segment is flagged: 2 us per step).
  // (Key rows more than half a megabyte apart, or more than 2048 segments: the selection launch redoes its flagged segment itself, as it does on the other routes.)
  const bool shared_redo = redo_segments_fits(gp, sc.num_segments);
  if (shared_redo) sc.redo_hist = sp.hist;
  rc = launch_select_finalize_cand(gp, sc, a->dtype, stream);
  if (rc != TKA_OK || !shared_redo) return rc;
  return launch_redo_segments(gp, sc, a->dtype, stream);
}

int check_flash(const tka_flash_decode_args* a) {
  if (!a) return TKA_EINVAL;
  if (!a->values || !a->out) return TKA_EINVAL;
  if (!a->kv_logit && (!a->q || !a->keys)) return TKA_EINVAL;
  if (a->head_dim != TKA_HEAD_DIM || !dtype_ok(a->dtype) || !dtype_ok(a->out_dtype) || !group_ok(a->group)) return TKA_EUNSUPPORTED;
  if (a->softmax_mode != TKA_SOFTMAX_SCALED && a->softmax_mode != TKA_SOFTMAX_RAW_EXP) return TKA_EUNSUPPORTED;
  if (a->batch < 1 || a->num_kv_heads < 1 || a->seq_len < 1) return TKA_EINVAL;
  if (a->batch > 65535 || a->num_kv_heads > 65535 || a->seq_len > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  if (a->num_splits < 0 || a->num_splits > TKA_MAX_SPLITS) return TKA_EINVAL;
  if (a->kv_stride_n < TKA_HEAD_DIM || a->kv_stride_h < 0 || a->kv_stride_b < 0) return TKA_EINVAL;
  if ((a->kv_stride_n | a->kv_stride_h | a->kv_stride_b | a->q_stride_b | a->out_stride_b) & 7) return TKA_EINVAL;
  if (!aligned16(a->q) || !aligned16(a->keys) || !aligned16(a->values)) return TKA_EINVAL;
  if (a->kv_idx) {
    if (a->idx_len < 1) return TKA_EINVAL;
  } else if (a->kv_count || a->kv_logit) {
    return TKA_EINVAL;
  }
  if (a->kv_logit && a->group != 1) return TKA_EUNSUPPORTED;
  const int64_t hq = (int64_t)a->num_kv_heads * a->group * TKA_HEAD_DIM;
  if (a->batch > 1 && (a->out_stride_b < hq || (!a->kv_logit && a->q_stride_b < hq))) return TKA_EINVAL;
  return TKA_OK;
}

// Positions per workgroup (multiple of 128, one or more kernel steps) and the split count that follows.
void flash_plan(const tka_flash_decode_args* a, int* splits, int* tokens_per_split) {
  const int64_t len = a->kv_idx ? a->idx_len : a->seq_len;
  int64_t want = a->num_splits;
  if (want <= 0) {
    // measured: the dense scan likes about 2048 workgroups, the gathered form about one resident set (3 per CU)
    const int64_t rows = (int64_t)a->batch * a->num_kv_heads;
    want = (a->kv_idx ? 1024 : 2048) / rows;
    if (want < 1) want = 1;
    // id lists on the VALU kernel: from 512 rows on (256 with up to 2048 ids per row), or up to 512 ids per row, one
    // workgroup per row, which writes the result itself and saves the combine launch; below that about 512
    // workgroups (measured on the operator: 16 x 32 rows of 4096 ids 54 instead of 69 us, 4 x 32 rows 24.6 instead
    // of 25.4)
    const bool valu = a->group == 1 || a->kv_logit;
    if (valu && a->kv_idx) want = (rows >= 512 || len <= 512 || (rows >= 256 && len <= 2048)) ? 1 : 512 / rows;
    if (want < 1) want = 1;
  }
  int64_t tps = (len + want - 1) / want;
  tps = (tps + 127) / 128 * 128;
  if (tps < 128) tps = 128;
  int64_t s = (len + tps - 1) / tps;
  if (s > TKA_MAX_SPLITS) {
    s = TKA_MAX_SPLITS;
    tps = ((len + s - 1) / s + 127) / 128 * 128;
    s = (len + tps - 1) / tps;
  }
  *splits = (int)s;
  *tokens_per_split = (int)tps;
}

size_t flash_bytes(const tka_flash_decode_args* a) {
  int splits, tps;
  flash_plan(a, &splits, &tps);
  const size_t rows = (size_t)a->batch * a->num_kv_heads * a->group;
  return align_up(rows * splits * sizeof(float), 256) * 2 + align_up(rows * splits * TKA_HEAD_DIM * sizeof(float), 256);
}

// Parameter block of the attention kernels for a call and its plan; the partials lie at the head of `workspace`.
void fill_attn_params(const tka_flash_decode_args* a, void* workspace, int splits, int tps, AttnParams* out) {
  const size_t rows = (size_t)a->batch * a->num_kv_heads * a->group;
  unsigned char* ws = (unsigned char*)workspace;
  AttnParams ap;
  memset(&ap, 0, sizeof ap);
  ap.part_m = (float*)ws;
  ws += align_up(rows * splits * sizeof(float), 256);
  ap.part_l = (float*)ws;
  ws += align_up(rows * splits * sizeof(float), 256);
  ap.part_acc = (float*)ws;
  ap.q = a->q;
  ap.keys = a->keys;
  ap.values = a->values;
  ap.kv_idx = a->kv_idx;
  ap.kv_count = a->kv_count;
  ap.kv_logit = a->kv_logit;
  ap.seq_len = a->seq_len;
  ap.q_stride_b = a->q_stride_b;
  ap.kv_stride_b = a->kv_stride_b;
  ap.kv_stride_n = a->kv_stride_n;
  ap.kv_stride_h = a->kv_stride_h;
  ap.batch = a->batch;
  ap.num_kv_heads = a->num_kv_heads;
  ap.group = a->group;
  ap.num_splits = splits;
  ap.idx_len = a->idx_len;
  ap.tokens_per_split = tps;
  ap.scale_log2e = a->scale * 1.44269504088896340736f;
  *out = ap;
}

void fill_combine_params(const tka_flash_decode_args* a, const AttnParams& ap, CombineParams* out) {
  CombineParams cp;
  memset(&cp, 0, sizeof cp);
  cp.part_m = ap.part_m;
  cp.part_l = ap.part_l;
  cp.part_acc = ap.part_acc;
  cp.out = a->out;
  cp.out_lse = a->out_lse;
  cp.out_stride_b = a->out_stride_b;
  cp.rows_per_batch = a->num_kv_heads * a->group;
  cp.rows = a->batch * a->num_kv_heads * a->group;
  cp.num_splits = ap.num_splits;
  cp.out_dtype = a->out_dtype;
  *out = cp;
}

int run_flash(const tka_flash_decode_args* a, void* workspace) {
  hipStream_t stream = (hipStream_t)a->stream;
  int splits, tps;
  flash_plan(a, &splits, &tps);
  AttnParams ap;
  fill_attn_params(a, workspace, splits, tps, &ap);
  // grouped queries go to the matrix cores; one query head per KV head (and supplied logits) stay on VALU
  const bool mfma = a->group >= 2 && !a->kv_logit;
  if (!mfma && splits == 1) {   // nothing to combine: the kernel writes the result itself
    ap.out = a->out;
    ap.out_lse = a->out_lse;
    ap.out_stride_b = a->out_stride_b;
    ap.out_dtype = a->out_dtype;
    return launch_attn_partial(ap, a->dtype, stream);
  }
  int rc = mfma ? launch_attn_partial_mfma(ap, a->dtype, stream) : launch_attn_partial(ap, a->dtype, stream);
  if (rc != TKA_OK) return rc;
  CombineParams cp;
  fill_combine_params(a, ap, &cp);
  return launch_lse_combine(cp, stream);
}

// Filled by run_gemv_topk when it leaves the selection of the candidate route to the attention launch
// (launch_attn_select_mfma): the stage-1 parameters that launch and the redo of flagged segments need.
struct FusedTail {
  bool taken;
  GemvParams g;
  SelectParams s;
};

bool fused_tail_take(FusedTail* ft, const GemvParams& g, const SelectParams& s) {
  ft->taken = true;
  ft->g = g;
  ft->s = s;
  return true;
}

// Selection + attention in one launch, then the combine launch that also redoes flagged segments.  f.kv_idx / f.kv_count:
// the list and count arrays of the step's workspace (only a redone segment writes and reads them).
int run_fused_tail(const tka_flash_decode_args* f, const FusedTail& ft, void* workspace) {
  hipStream_t stream = (hipStream_t)f->stream;
  // Every split of a segment finds the segment's threshold again, and a workgroup holds the candidates in LDS (two per
  // CU): about 512 workgroups, not the thousand of the attention that reads its list from memory.  (The workspace is
  // sized for that plan, which has at least as many splits.)
  tka_flash_decode_args fa = *f;
  int splits, tps;
  flash_plan(&fa, &splits, &tps);
  if (fa.num_splits <= 0) {
    int64_t want = 512 / ((int64_t)fa.batch * fa.num_kv_heads);
    if (want < 1) want = 1;
    if (want < splits) {
      fa.num_splits = (int)want;
      flash_plan(&fa, &splits, &tps);
    }
  }
  AttnParams ap;
  fill_attn_params(f, workspace, splits, tps, &ap);
  FusedSelectParams fs;
  memset(&fs, 0, sizeof fs);
  fs.cand_head = ft.s.cand_head;
  fs.cand = ft.s.list;
  fs.cand_seg_stride = ft.s.list_stride;
  fs.tau_words = ft.s.tau_words;
  fs.sample_flags = ft.s.sample_flags;
  fs.seg_flags = ft.s.seg_flags;
  fs.parts = ft.s.parts;
  fs.part_len = ft.s.part_len;
  fs.k = ft.s.k;
  fs.sink = ft.s.sink;
  fs.local = ft.s.local;
  fs.max_entries = ft.s.max_entries;
  int rc = launch_attn_select_mfma(ap, fs, f->dtype, stream);
  if (rc != TKA_OK) return rc;
  CombineParams cp;
  fill_combine_params(f, ap, &cp);
  return launch_lse_combine_redo(cp, ft.g, ft.s, ap, f->dtype, stream);
}

}  // namespace
}  // namespace tka

using namespace tka;

extern "C" {

const char* tka_status_string(int status) {
  switch (status) {
    case TKA_OK: return "ok";
    case TKA_EINVAL: return "invalid argument";
    case TKA_EUNSUPPORTED: return "unsupported configuration";
    case TKA_EHIP: return "HIP runtime error";
    case TKA_EWORKSPACE: return "workspace missing or too small";
    case TKA_ESCRATCH: return "the call needs more scratch memory than the library's built-in buffer holds";
    default: return "unknown status";
  }
}

int tka_version(void) { return 200; }

// ---- stage 1 ----------------------------------------------------------------------------------

size_t tka_gemv_topk_workspace_bytes(const tka_gemv_topk_args* a) {
  if (check_gemv(a, true) != TKA_OK) return 0;
  const int segs = a->batch * a->num_kv_heads * a->num_chunks;
  return gemv_scores_bytes(a) + select_workspace_bytes(segs, a->seq_len / a->num_chunks);
}

int tka_gemv_topk(const tka_gemv_topk_args* a) {
  int rc = check_gemv(a, true);
  if (rc != TKA_OK) return rc;
  if (!a->workspace || a->workspace_bytes < tka_gemv_topk_workspace_bytes(a)) return TKA_EWORKSPACE;
  return run_gemv_topk(a, nullptr, 0);
}

// Per-segment flag words of the last candidate-route call with these arguments (bit 0: redone from the keys,
// bits 8..: slices whose workgroup gave up waiting for the threshold); empty for calls that take another route.
// `u`: the union list that the call asked for (nullptr: none), which decides the route with the other arguments.
static int read_segment_flags(const tka_gemv_topk_args* a, const UnionOut* u, std::vector<uint32_t>* flags) {
  flags->clear();
  int rc = check_gemv(a, true);
  if (rc != TKA_OK) return rc;
  if (!a->workspace || a->workspace_bytes < tka_gemv_topk_workspace_bytes(a)) return TKA_EWORKSPACE;
  int num_samples = 0, sample_rank = 0;
  cut_plan(a, u, &num_samples, &sample_rank);   // (no route between the two writes the flags: those segments are too short for the second)
  if (num_samples == 0) candidate_plan(a, &num_samples, &sample_rank);
  if (num_samples == 0) return TKA_OK;
  const int segs = a->batch * a->num_kv_heads * a->num_chunks;
  SelectParams sp;
  memset(&sp, 0, sizeof sp);
  select_carve((unsigned char*)a->workspace + gemv_scores_bytes(a), segs, a->seq_len / a->num_chunks, &sp);
  flags->resize((size_t)segs);
  if (hipStreamSynchronize((hipStream_t)a->stream) != hipSuccess) return TKA_EHIP;
  if (hipMemcpy(flags->data(), sp.seg_flags, flags->size() * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) return TKA_EHIP;
  return TKA_OK;
}

static int redone_segments(const tka_gemv_topk_args* a, const UnionOut* u, int32_t* count) {
  if (!count) return TKA_EINVAL;
  *count = 0;
  std::vector<uint32_t> flags;
  const int rc = read_segment_flags(a, u, &flags);
  for (uint32_t f : flags) *count += (int32_t)(f & 1u);
  return rc;
}

int tka_gemv_topk_redone_segments(const tka_gemv_topk_args* a, int32_t* count) { return redone_segments(a, nullptr, count); }

int tka_gemv_topk_gave_up_slices(const tka_gemv_topk_args* a, int32_t* count) {
  if (!count) return TKA_EINVAL;
  *count = 0;
  std::vector<uint32_t> flags;
  const int rc = read_segment_flags(a, nullptr, &flags);
  for (uint32_t f : flags) *count += (int32_t)(f >> 8);
  return rc;
}

int tka_set_test_hooks(const tka_test_hooks* hooks) {
  if (hooks && (hooks->tau_spin_limit < 0 || hooks->tau_withhold_mod < 0 || hooks->tau_withhold_rem < 0 ||
                (hooks->tau_withhold_mode != 0 && hooks->tau_withhold_mode != 1) || hooks->fused_tail < 0 || hooks->fused_tail > 2))
    return TKA_EINVAL;
  std::lock_guard<std::mutex> lock(g_hooks_mutex);
  if (hooks) g_hooks = *hooks;
  else g_hooks = tka_test_hooks{0, 0, 0, 0, 0, 0, 0};
  return TKA_OK;
}

int tka_gemv_scores(const tka_gemv_topk_args* a) {
  int rc = check_gemv(a, false);
  if (rc != TKA_OK) return rc;
  GemvParams gp;
  fill_gemv_params(a, a->out_scores, nullptr, &gp);
  if (a->key_stride_b == 0 && a->batch >= 2) return launch_shared_scores(a, gp, (hipStream_t)a->stream);
  return launch_gemv_scores(gp, a->dtype, (hipStream_t)a->stream);
}

static int check_topk(const tka_topk_args* a) {
  if (!a || !a->scores || !a->out_idx) return TKA_EINVAL;
  if (a->num_segments < 1 || a->seg_len < 1 || a->seg_stride < a->seg_len) return TKA_EINVAL;
  if (a->k < 1 || a->k > a->seg_len) return TKA_EINVAL;
  if (a->k > TKA_MAX_TOPK || a->num_segments > 65535 || a->seg_len > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  return TKA_OK;
}

size_t tka_topk_workspace_bytes(const tka_topk_args* a) {
  if (check_topk(a) != TKA_OK) return 0;
  return select_workspace_bytes(a->num_segments, a->seg_len);
}

int tka_topk_f32(const tka_topk_args* a) {
  int rc = check_topk(a);
  if (rc != TKA_OK) return rc;
  if (!a->workspace || a->workspace_bytes < tka_topk_workspace_bytes(a)) return TKA_EWORKSPACE;
  hipStream_t stream = (hipStream_t)a->stream;
  SelectParams sp;
  memset(&sp, 0, sizeof sp);
  const size_t zero_words = select_carve(a->workspace, a->num_segments, a->seg_len, &sp);
  select_plan(a->seg_len, a->num_segments, &sp);
  sp.scores = a->scores;
  sp.seg_len = a->seg_len;
  sp.seg_stride = a->seg_stride;
  sp.out_idx = a->out_idx;
  sp.out_val = a->out_val;
  sp.out_stride = a->k;
  sp.num_segments = a->num_segments;
  sp.k = a->k;
  sp.segs_per_row = 1;
  if (wave_select_fits(a->seg_len, a->k)) return launch_select_wave(sp, stream);
  if (a->seg_len <= select_cand_capacity()) {   // the segment fits in LDS whole: one launch
    GemvParams none;
    memset(&none, 0, sizeof none);
    sp.from_scores = 1;
    return launch_select_finalize_cand(none, sp, TKA_F16, stream);
  }
  rc = launch_zero_u32(sp.hist, zero_words, stream);
  if (rc != TKA_OK) return rc;
  rc = launch_select_hist(sp, stream);
  if (rc != TKA_OK) return rc;
  return launch_select(sp, stream);
}

static int center_as_gemv(const tka_center_topk_args* a, tka_gemv_topk_args* g) {
  if (!a || !a->q || !a->centers || !a->out_idx) return TKA_EINVAL;
  if (a->num_heads < 1 || a->num_centers < 1 || a->top_c < 1 || a->cluster_len < 1) return TKA_EINVAL;
  if ((int64_t)a->top_c * a->cluster_len > 0x7fffffffLL || (int64_t)a->num_centers * a->cluster_len > 0x7fffffffLL)
    return TKA_EUNSUPPORTED;
  memset(g, 0, sizeof *g);
  g->q = a->q;
  g->keys = a->centers;
  g->dtype = a->dtype;
  g->batch = 1;
  g->num_kv_heads = a->num_heads;
  g->group = 1;
  g->head_dim = a->head_dim;
  g->k = a->top_c;
  g->num_chunks = 1;
  g->seq_len = a->num_centers;
  g->q_stride_b = 0;
  g->key_stride_b = 0;
  g->key_stride_n = TKA_HEAD_DIM;
  g->key_stride_h = (int64_t)a->num_centers * TKA_HEAD_DIM;
  g->scale = a->scale;
  g->out_idx = a->out_centers;
  g->out_val = a->out_center_val;
  g->workspace = a->workspace;
  g->workspace_bytes = a->workspace_bytes;
  g->stream = a->stream;
  return TKA_OK;
}

size_t tka_center_topk_expand_workspace_bytes(const tka_center_topk_args* a) {
  tka_gemv_topk_args g;
  if (center_as_gemv(a, &g) != TKA_OK) return 0;
  int32_t dummy;
  if (!g.out_idx) g.out_idx = &dummy;
  size_t inner = tka_gemv_topk_workspace_bytes(&g);
  if (inner == 0) return 0;
  // room for the chosen centroid ids when the caller does not want them
  return inner + align_up((size_t)a->num_heads * a->top_c * sizeof(int32_t), 256);
}

int tka_center_topk_expand(const tka_center_topk_args* a) {
  tka_gemv_topk_args g;
  int rc = center_as_gemv(a, &g);
  if (rc != TKA_OK) return rc;
  const size_t tail = align_up((size_t)a->num_heads * a->top_c * sizeof(int32_t), 256);
  int32_t dummy;
  const bool own_centers = g.out_idx == nullptr;
  if (own_centers) g.out_idx = &dummy;  // placeholder for validation
  rc = check_gemv(&g, true);
  if (rc != TKA_OK) return rc;
  const size_t need = tka_center_topk_expand_workspace_bytes(a);
  if (!a->workspace || a->workspace_bytes < need) return TKA_EWORKSPACE;
  if (own_centers) g.out_idx = (int32_t*)((unsigned char*)a->workspace + (need - tail));
  return run_gemv_topk(&g, a->out_idx, a->cluster_len);
}

// ---- stage 1d: two-level cluster selection ---------------------------------------------------

static int cluster_parts(const tka_cluster_topk_args* a, tka_gemv_topk_args* c, tka_gemv_topk_args* t) {
  if (!a || !a->q || !a->centers || !a->keys || !a->out_idx) return TKA_EINVAL;
  if (a->num_heads < 1 || a->num_centers < 1 || a->top_c < 1 || a->cluster_len < 1 || a->k < 1) return TKA_EINVAL;
  if (a->top_c > a->num_centers || a->k > a->cluster_len) return TKA_EINVAL;
  if ((int64_t)a->num_centers * a->cluster_len > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  // level 1: centroids, [num_heads][num_centers][128]
  memset(c, 0, sizeof *c);
  c->q = a->q;
  c->keys = a->centers;
  c->dtype = a->dtype;
  c->batch = 1;
  c->num_kv_heads = a->num_heads;
  c->group = 1;
  c->head_dim = a->head_dim;
  c->k = a->top_c;
  c->num_chunks = 1;
  c->seq_len = a->num_centers;
  c->key_stride_n = TKA_HEAD_DIM;
  c->key_stride_h = (int64_t)a->num_centers * TKA_HEAD_DIM;
  c->scale = a->scale;
  c->stream = a->stream;
  // level 2: top_c chunks of cluster_len tokens per head, chunk start taken from level 1
  memset(t, 0, sizeof *t);
  t->q = a->q;
  t->keys = a->keys;
  t->dtype = a->dtype;
  t->batch = 1;
  t->num_kv_heads = a->num_heads;
  t->group = 1;
  t->head_dim = a->head_dim;
  t->k = a->k;
  t->num_chunks = a->top_c;
  t->seq_len = (int64_t)a->top_c * a->cluster_len;
  t->key_stride_n = a->key_stride_n;
  t->key_stride_h = a->key_stride_h;
  t->scale = a->scale;
  t->out_idx = a->out_idx;
  t->stream = a->stream;
  return TKA_OK;
}

size_t tka_cluster_gemv_topk_workspace_bytes(const tka_cluster_topk_args* a) {
  tka_gemv_topk_args c, t;
  if (cluster_parts(a, &c, &t) != TKA_OK) return 0;
  int32_t dummy;
  c.out_idx = &dummy;
  if (check_gemv(&c, true) != TKA_OK || check_gemv(&t, true) != TKA_OK) return 0;
  return align_up((size_t)a->num_heads * a->top_c * sizeof(int32_t), 256) + tka_gemv_topk_workspace_bytes(&c) +
         tka_gemv_topk_workspace_bytes(&t);
}

int tka_cluster_gemv_topk(const tka_cluster_topk_args* a) {
  tka_gemv_topk_args c, t;
  int rc = cluster_parts(a, &c, &t);
  if (rc != TKA_OK) return rc;
  int32_t dummy;
  c.out_idx = &dummy;
  if ((rc = check_gemv(&c, true)) != TKA_OK) return rc;
  if ((rc = check_gemv(&t, true)) != TKA_OK) return rc;
  const size_t need = tka_cluster_gemv_topk_workspace_bytes(a);
  if (!a->workspace || a->workspace_bytes < need) return TKA_EWORKSPACE;
  unsigned char* ws = (unsigned char*)a->workspace;
  int32_t* centre_ids = (int32_t*)ws;
  ws += align_up((size_t)a->num_heads * a->top_c * sizeof(int32_t), 256);
  if (a->num_centers <= kGemvInlineCentres && wave_route(&t, false)) {
    // few centroids, clusters that a workgroup selects from registers: two launches instead of three
    const InlineCentres ic = {a->centers, a->num_centers, centre_ids};
    t.workspace = ws + tka_gemv_topk_workspace_bytes(&c);
    t.workspace_bytes = tka_gemv_topk_workspace_bytes(&t);
    return run_gemv_topk(&t, nullptr, 0, nullptr, nullptr, false, &ic);
  }
  c.out_idx = centre_ids;
  c.workspace = ws;
  c.workspace_bytes = tka_gemv_topk_workspace_bytes(&c);
  rc = run_gemv_topk(&c, nullptr, 0);
  if (rc != TKA_OK) return rc;
  t.workspace = ws + c.workspace_bytes;
  t.workspace_bytes = tka_gemv_topk_workspace_bytes(&t);
  return run_gemv_topk(&t, nullptr, 0, centre_ids);
}

// ---- index union ------------------------------------------------------------------------------

int tka_index_union(const tka_index_union_args* a) {
  if (!a || !a->idx || !a->out_idx || !a->out_count) return TKA_EINVAL;
  if (a->num_segments < 1 || a->k < 1 || a->sink < 0 || a->local < 0 || a->seq_len < 1) return TKA_EINVAL;
  if (a->k > TKA_MAX_TOPK || a->seq_len > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  if (a->sink > a->seq_len || a->local > a->seq_len) return TKA_EINVAL;
  UnionParams up;
  up.idx = a->idx;
  up.out_idx = a->out_idx;
  up.out_count = a->out_count;
  up.seq_len = a->seq_len;
  up.num_segments = a->num_segments;
  up.k = a->k;
  up.sink = a->sink;
  up.local = a->local;
  return launch_index_union(up, (hipStream_t)a->stream);
}

// ---- stage 3 ----------------------------------------------------------------------------------

size_t tka_flash_decode_workspace_bytes(const tka_flash_decode_args* a) {
  if (check_flash(a) != TKA_OK) return 0;
  return flash_bytes(a);
}

int tka_flash_decode(const tka_flash_decode_args* a) {
  int rc = check_flash(a);
  if (rc != TKA_OK) return rc;
  if (!a->workspace || a->workspace_bytes < flash_bytes(a)) return TKA_EWORKSPACE;
  return run_flash(a, a->workspace);
}

int tka_lse_combine(const tka_lse_combine_args* a) {
  if (!a || !a->part_m || !a->part_l || !a->part_acc || !a->out) return TKA_EINVAL;
  if (a->rows < 1 || a->num_splits < 1) return TKA_EINVAL;
  if (!dtype_ok(a->out_dtype)) return TKA_EUNSUPPORTED;
  // the kernel keeps one weight per split in LDS; one workgroup per row on a 1-D grid
  if (a->num_splits > TKA_MAX_SPLITS || (int64_t)a->rows * a->num_splits > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  CombineParams cp;
  memset(&cp, 0, sizeof cp);
  cp.part_m = a->part_m;
  cp.part_l = a->part_l;
  cp.part_acc = a->part_acc;
  cp.out = a->out;
  cp.out_lse = a->out_lse;
  cp.out_stride_b = (int64_t)a->rows * TKA_HEAD_DIM;
  cp.rows_per_batch = a->rows;
  cp.rows = a->rows;
  cp.num_splits = a->num_splits;
  cp.out_dtype = a->out_dtype;
  return launch_lse_combine(cp, (hipStream_t)a->stream);
}

// ---- stage 2: the retrieval_attention op ------------------------------------------------------

static int ra_parts(const tka_ra_args* a, tka_gemv_topk_args* g, tka_flash_decode_args* f) {
  if (!a || !a->q || !a->keys || !a->values || !a->out) return TKA_EINVAL;
  if (a->batch < 1 || a->num_heads < 1 || a->seq_len < 1 || a->num_chunks < 1 || a->topk_per_chunk < 1) return TKA_EINVAL;
  if ((int64_t)a->topk_per_chunk * a->num_chunks > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  memset(g, 0, sizeof *g);
  g->q = a->q;
  g->keys = a->keys;
  g->dtype = a->dtype;
  g->batch = a->batch;
  g->num_kv_heads = a->num_heads;
  g->group = 1;
  g->head_dim = a->head_dim;
  g->k = a->topk_per_chunk;
  g->num_chunks = a->num_chunks;
  g->seq_len = a->seq_len;
  g->q_stride_b = (int64_t)a->num_heads * TKA_HEAD_DIM;
  g->key_stride_b = 0;
  g->key_stride_n = (int64_t)a->num_heads * TKA_HEAD_DIM;
  g->key_stride_h = TKA_HEAD_DIM;
  g->scale = a->scale;
  g->score_mode = a->score_mode;
  g->stream = a->stream;
  memset(f, 0, sizeof *f);
  f->q = a->q;
  f->keys = a->keys;
  f->values = a->values;
  f->out = a->out;
  f->dtype = a->dtype;
  f->out_dtype = a->dtype;
  f->batch = a->batch;
  f->num_kv_heads = a->num_heads;
  f->group = 1;
  f->head_dim = a->head_dim;
  f->num_splits = 0;
  f->softmax_mode = a->softmax_mode;
  f->seq_len = a->seq_len;
  f->q_stride_b = g->q_stride_b;
  f->out_stride_b = g->q_stride_b;
  f->kv_stride_b = 0;
  f->kv_stride_n = g->key_stride_n;
  f->kv_stride_h = TKA_HEAD_DIM;
  f->scale = 1.0f;  // the handed-off scores are already scaled
  f->idx_len = a->topk_per_chunk * a->num_chunks;
  f->stream = a->stream;
  return TKA_OK;
}

size_t tka_retrieval_attention_workspace_bytes(const tka_ra_args* a) {
  tka_gemv_topk_args g;
  tka_flash_decode_args f;
  if (ra_parts(a, &g, &f) != TKA_OK) return 0;
  const size_t sel = (size_t)a->batch * a->num_heads * a->topk_per_chunk * a->num_chunks;
  int32_t dummy_i;
  float dummy_f;
  g.out_idx = &dummy_i;
  f.kv_idx = &dummy_i;
  f.kv_logit = &dummy_f;
  if (check_gemv(&g, true) != TKA_OK || check_flash(&f) != TKA_OK) return 0;
  return tka_gemv_topk_workspace_bytes(&g) + align_up(sel * sizeof(int32_t), 256) + align_up(sel * sizeof(float), 256) +
         flash_bytes(&f);
}

static int ra_launch(const tka_ra_args* a) {
  tka_gemv_topk_args g;
  tka_flash_decode_args f;
  int rc = ra_parts(a, &g, &f);
  if (rc != TKA_OK) return rc;
  const size_t sel = (size_t)a->batch * a->num_heads * a->topk_per_chunk * a->num_chunks;
  unsigned char* ws = (unsigned char*)a->workspace;
  int32_t* idx = (int32_t*)ws;
  ws += align_up(sel * sizeof(int32_t), 256);
  float* val = (float*)ws;
  ws += align_up(sel * sizeof(float), 256);
  g.out_idx = idx;
  g.out_val = val;
  f.kv_idx = idx;
  f.kv_logit = val;
  rc = check_gemv(&g, true);
  if (rc != TKA_OK) return rc;
  rc = check_flash(&f);
  if (rc != TKA_OK) return rc;
  const size_t gemv_ws = tka_gemv_topk_workspace_bytes(&g);
  g.workspace = ws;
  g.workspace_bytes = gemv_ws;
  rc = run_gemv_topk(&g, nullptr, 0, nullptr, nullptr, true);   // (softmax and the weighted sum take any order)
  if (rc != TKA_OK) return rc;
  return run_flash(&f, ws + gemv_ws);
}

int tka_retrieval_attention(const tka_ra_args* a) {
  const size_t need = tka_retrieval_attention_workspace_bytes(a);
  if (need == 0) {
    tka_gemv_topk_args g;
    tka_flash_decode_args f;
    int rc = ra_parts(a, &g, &f);
    if (rc != TKA_OK) return rc;
    int32_t di;
    float df;
    g.out_idx = &di;
    f.kv_idx = &di;
    f.kv_logit = &df;
    rc = check_gemv(&g, true);
    if (rc != TKA_OK) return rc;
    rc = check_flash(&f);
    return rc != TKA_OK ? rc : TKA_EINVAL;
  }
  if (!a->workspace || a->workspace_bytes < need) return TKA_EWORKSPACE;
  int rc = ra_launch(a);
  if (rc != TKA_OK || !a->bench_print) return rc;
  // Harness compatibility: the reference op warms up 10 times, times its launch and prints one line
  // that test_ra.py:63-75 parses.  Blocking, like the reference (retrieval_attention.cu:1586-1612).
  hipStream_t stream = (hipStream_t)a->stream;
  for (int i = 0; i < 10; ++i)
    if ((rc = ra_launch(a)) != TKA_OK) return rc;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return TKA_EHIP;
  (void)hipEventRecord(e0, stream);
  rc = ra_launch(a);
  (void)hipEventRecord(e1, stream);
  float ms = 0.0f;
  if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = TKA_EHIP;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc == TKA_OK) {
    printf("Retrieval Attention Config: TOPK=%d, TOTAL_TOPK=%d, BLOCK_SIZE=%d\n", a->topk_per_chunk,
           a->topk_per_chunk * a->num_chunks, 1024);
    printf("Retrieval Attention - Avg time: %.3f ms, Throughput: %.2f iter/s\n", ms, 1000.0f / ms);
    fflush(stdout);
  }
  return rc;
}

// ---- end-to-end sparse decode step ------------------------------------------------------------

static int sd_parts(const tka_sparse_decode_args* a, tka_gemv_topk_args* g, tka_flash_decode_args* f) {
  if (!a || !a->q || !a->keys || !a->values || !a->out) return TKA_EINVAL;
  if (a->sink < 0 || a->local < 0 || a->k < 1) return TKA_EINVAL;
  if (a->sink > a->seq_len || a->local > a->seq_len) return TKA_EINVAL;
  memset(g, 0, sizeof *g);
  g->q = a->q;
  g->keys = a->keys;
  g->dtype = a->dtype;
  g->batch = a->batch;
  g->num_kv_heads = a->num_kv_heads;
  g->group = a->group;
  g->head_dim = a->head_dim;
  g->k = a->k;
  g->num_chunks = 1;
  g->seq_len = a->seq_len;
  g->q_stride_b = a->q_stride_b;
  g->key_stride_b = a->kv_stride_b;
  g->key_stride_n = a->kv_stride_n;
  g->key_stride_h = a->kv_stride_h;
  g->scale = a->scale;
  g->stream = a->stream;
  memset(f, 0, sizeof *f);
  f->q = a->q;
  f->keys = a->keys;
  f->values = a->values;
  f->out = a->out;
  f->dtype = a->dtype;
  f->out_dtype = a->out_dtype;
  f->batch = a->batch;
  f->num_kv_heads = a->num_kv_heads;
  f->group = a->group;
  f->head_dim = a->head_dim;
  f->num_splits = a->num_splits;
  f->softmax_mode = TKA_SOFTMAX_SCALED;
  f->seq_len = a->seq_len;
  f->q_stride_b = a->q_stride_b;
  f->out_stride_b = a->out_stride_b;
  f->kv_stride_b = a->kv_stride_b;
  f->kv_stride_n = a->kv_stride_n;
  f->kv_stride_h = a->kv_stride_h;
  f->scale = a->scale;
  f->idx_len = a->k + a->sink + a->local;
  f->stream = a->stream;
  return TKA_OK;
}

// The attention takes the selected tokens in any order and skips -1; a caller that asks for the list gets it ascending and dense.
static bool sd_union_handoff(const tka_sparse_decode_args* a) { return !a->out_union_idx || current_hooks().union_handoff_order != 0; }

// A caller that asks for the ascending list on a step whose segments the common-cut route would take (beyond what the
// registers of one workgroup hold, where the list-making routes need four launches): the step runs on that route with a
// hand-off list of its own in the workspace, and the caller's list is made from the rank-ordered ids by one more launch
// behind the attention (8 x 32768 tokens: 36 instead of 43 us per step).  `g`: the stage-1 arguments of the step.
static bool sd_list_behind(const tka_sparse_decode_args* a, const tka_gemv_topk_args& g) {
  // (beyond a million rows the routes that make the list themselves are as quick: 48 x 32768 tokens 98.2 / 95.9 us)
  if (sd_union_handoff(a) || a->seq_len <= select_cand_capacity() || (int64_t)a->batch * a->num_kv_heads * a->seq_len > (int64_t)1 << 20) return false;
  tka_gemv_topk_args probe = g;
  int32_t di;
  probe.out_idx = &di;
  const UnionOut uo = {nullptr, nullptr, a->sink, a->local, true};
  int num_samples = 0, sample_rank = 0;
  cut_plan(&probe, &uo, &num_samples, &sample_rank);
  return num_samples != 0;
}

static int sd_check(const tka_sparse_decode_args* a, tka_gemv_topk_args* g, tka_flash_decode_args* f) {
  int rc = sd_parts(a, g, f);
  if (rc != TKA_OK) return rc;
  int32_t di;
  g->out_idx = &di;
  f->kv_idx = &di;
  f->kv_count = &di;
  rc = check_gemv(g, true);
  if (rc != TKA_OK) return rc;
  return check_flash(f);
}

size_t tka_sparse_decode_workspace_bytes(const tka_sparse_decode_args* a) {
  tka_gemv_topk_args g;
  tka_flash_decode_args f;
  if (sd_check(a, &g, &f) != TKA_OK) return 0;
  const size_t segs = (size_t)a->batch * a->num_kv_heads;
  return align_up(segs * a->k * sizeof(int32_t), 256) + align_up(segs * a->k * sizeof(float), 256) +
         align_up(segs * (size_t)f.idx_len * sizeof(int32_t), 256) + align_up(segs * sizeof(int32_t), 256) +
         tka_gemv_topk_workspace_bytes(&g) + flash_bytes(&f);
}

// Offset of the stage-1 workspace inside the workspace of the step.
static size_t sd_gemv_ws_offset(const tka_sparse_decode_args* a, const tka_flash_decode_args& f) {
  const size_t segs = (size_t)a->batch * a->num_kv_heads;
  return align_up(segs * a->k * sizeof(int32_t), 256) + align_up(segs * a->k * sizeof(float), 256) +
         align_up(segs * (size_t)f.idx_len * sizeof(int32_t), 256) + align_up(segs * sizeof(int32_t), 256);
}

int tka_sparse_decode_redone_segments(const tka_sparse_decode_args* a, int32_t* count) {
  if (!count) return TKA_EINVAL;
  *count = 0;
  tka_gemv_topk_args g;
  tka_flash_decode_args f;
  int rc = sd_check(a, &g, &f);
  if (rc != TKA_OK) return rc;
  if (!a->workspace || a->workspace_bytes < tka_sparse_decode_workspace_bytes(a)) return TKA_EWORKSPACE;
  g.workspace = (unsigned char*)a->workspace + sd_gemv_ws_offset(a, f);
  g.workspace_bytes = tka_gemv_topk_workspace_bytes(&g);
  const bool behind = sd_list_behind(a, g);
  int32_t di;
  if (behind) g.out_idx = &di;   // (as the step runs it)
  const UnionOut uo = {nullptr, nullptr, a->sink, a->local, sd_union_handoff(a) || behind};
  return redone_segments(&g, &uo, count);
}

int tka_sparse_decode_step(const tka_sparse_decode_args* a) {
  tka_gemv_topk_args g;
  tka_flash_decode_args f;
  int rc = sd_check(a, &g, &f);
  if (rc != TKA_OK) return rc;
  if (a->out_topk_val && !a->out_topk_idx) return TKA_EINVAL;   // values come with the rank-ordered ids only
  if (a->out_union_count && !a->out_union_idx) return TKA_EINVAL;   // the count belongs to the list (without the list the step
                                                                     // hands its tokens on in a form whose count is not the union's)
  const size_t need = tka_sparse_decode_workspace_bytes(a);
  if (!a->workspace || a->workspace_bytes < need) return TKA_EWORKSPACE;
  const size_t segs = (size_t)a->batch * a->num_kv_heads;
  unsigned char* ws = (unsigned char*)a->workspace;
  int32_t* tidx = (int32_t*)ws;
  ws += align_up(segs * a->k * sizeof(int32_t), 256);
  float* tval = (float*)ws;
  ws += align_up(segs * a->k * sizeof(float), 256);
  int32_t* uidx = (int32_t*)ws;
  ws += align_up(segs * (size_t)f.idx_len * sizeof(int32_t), 256);
  int32_t* ucnt = (int32_t*)ws;
  ws += align_up(segs * sizeof(int32_t), 256);
  const bool behind = sd_list_behind(a, g);   // (the list for the attention then stays in the workspace)
  int32_t* const hand_cnt = ucnt;
  if (a->out_topk_idx) tidx = a->out_topk_idx;
  if (a->out_topk_val) tval = a->out_topk_val;
  if (a->out_union_idx && !behind) uidx = a->out_union_idx;
  if (a->out_union_count && !behind) ucnt = a->out_union_count;
  const size_t gemv_ws = tka_gemv_topk_workspace_bytes(&g);
  // rank-ordered top-k only if the caller asked for it (or the list is made from it); the attention needs the union list alone
  g.out_idx = a->out_topk_idx || behind ? tidx : nullptr;
  g.out_val = a->out_topk_idx ? tval : nullptr;
  g.workspace = ws;
  g.workspace_bytes = gemv_ws;
  UnionOut uo = {uidx, ucnt, a->sink, a->local, sd_union_handoff(a) || behind};
  // A caller that asks for neither list (the output alone): on long segments the attention launch can select the tokens
  // itself from the candidates of the GEMV launch, and the ids never leave the chip.  Every split of a segment then finds
  // the segment's threshold again, and that costs what the saved launch gives: us per step, one launch / two, k = 2048:
  // 64 segments of 131072 tokens 344.5 / 342.8, 96 segments 507.0 / 503.2, 128 segments 667.1 / 665.5, 128 segments of 65536
  // tokens 366.5 / 366.4, 192 segments 524.4 / 519.8, 256 segments 724.1 / 725.2.  (A form in which one split per segment
  // selects and the others wait for its list - a bounded wait - was 2 us slower still: the selection is a chain of
  // dependent steps that takes its 8-10 us whether or not the other splits keep out of its way.)  So the two launches
  // stay the rule and the one launch is taken from 256 segments on.
  FusedTail ft;
  ft.taken = false;
  const tka_test_hooks hooks = current_hooks();
  const bool output_only = !a->out_topk_idx && !a->out_union_idx && hooks.union_handoff_order == 0 && a->group >= 2 &&
                           (hooks.fused_tail == 1 || (hooks.fused_tail == 0 && segs >= 256));
  rc = run_gemv_topk(&g, nullptr, 0, nullptr, &uo, false, nullptr, output_only ? &ft : nullptr);
  if (rc != TKA_OK) return rc;
  f.kv_idx = uidx;
  f.kv_count = ucnt;
  if (ft.taken) return run_fused_tail(&f, ft, ws + gemv_ws);
  rc = run_flash(&f, ws + gemv_ws);
  if (rc != TKA_OK || !behind) return rc;
  UnionParams up;
  up.idx = tidx;
  up.out_idx = a->out_union_idx;
  up.out_count = a->out_union_count ? a->out_union_count : hand_cnt;   // (the attention has read its counts by then: one stream)
  up.seq_len = a->seq_len;
  up.num_segments = (int)segs;
  up.k = a->k;
  up.sink = a->sink;
  up.local = a->local;
  return launch_index_union(up, (hipStream_t)a->stream);
}

// ---- the step for callers that cannot allocate ------------------------------------------------

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};   // address of `scratch` on each device, looked up once with that device current
std::mutex g_scratch_mutex;

// Device address of the built-in scratch array on the current device.
int noalloc_scratch(void** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TKA_EHIP;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return TKA_EHIP;
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return TKA_OK;
}
}  // namespace

int tka_sparse_decode_step_noalloc(const tka_sparse_decode_args* a) {
  tka_gemv_topk_args g;
  tka_flash_decode_args f;
  int rc = sd_check(a, &g, &f);
  if (rc != TKA_OK) return rc;
  const size_t need = tka_sparse_decode_workspace_bytes(a);
  if (need == 0) return TKA_EINVAL;
  if (need > (size_t)TKA_NOALLOC_SCRATCH_BYTES) return TKA_ESCRATCH;
  void* ptr = nullptr;
  if ((rc = noalloc_scratch(&ptr)) != TKA_OK) return rc;
  // The array keeps what the last call left, laid out for that call's shapes.  The words by which the
  // candidate route tells this call's sampling state from older contents (thresholds, arrival flags, segment
  // flags) are cleared for this call's layout, with a fill kernel; the histograms are cleared by the route
  // that uses them; everything else is written before it is read.
  uint32_t* words = nullptr;
  const size_t n_words = select_epoch_words((unsigned char*)ptr + sd_gemv_ws_offset(a, f) + gemv_scores_bytes(&g),
                                            a->batch * a->num_kv_heads, a->seq_len, &words);
  if ((rc = launch_zero_u32(words, n_words, (hipStream_t)a->stream)) != TKA_OK) return rc;
  tka_sparse_decode_args b = *a;
  b.workspace = ptr;
  b.workspace_bytes = (size_t)TKA_NOALLOC_SCRATCH_BYTES;
  return tka_sparse_decode_step(&b);
}

// ---- read probes --------------------------------------------------------------------------------

int tka_probe_read(const tka_probe_args* a) {
  if (!a || !a->keys || !a->sink) return TKA_EINVAL;
  if (a->batch < 1 || a->num_kv_heads < 1 || a->seq_len < 1 || a->seq_len > 0x7fffffffLL) return TKA_EINVAL;
  if (a->kv_stride_n < TKA_HEAD_DIM || a->kv_stride_h < 0 || a->kv_stride_b < 0 || ((a->kv_stride_n | a->kv_stride_h | a->kv_stride_b) & 7)) return TKA_EINVAL;
  if (!aligned16(a->keys)) return TKA_EINVAL;
  ProbeParams p;
  memset(&p, 0, sizeof p);
  p.base = a->keys;
  p.base2 = a->values;
  p.idx = a->idx;
  p.sink = a->sink;
  p.seq_len = a->seq_len;
  p.stride_b = a->kv_stride_b;
  p.stride_n = a->kv_stride_n;
  p.stride_h = a->kv_stride_h;
  p.batch = a->batch;
  p.num_heads = a->num_kv_heads;
  p.idx_len = a->idx_len;
  if (a->kind == TKA_PROBE_STREAM) return launch_probe_stream(p, a->threads, a->rounds, a->nontemporal != 0, (hipStream_t)a->stream);
  if (a->kind == TKA_PROBE_GATHER) {
    if (!a->values || !a->idx || !aligned16(a->values) || a->idx_len < 1 || a->tokens_per_wg < 128 || a->tokens_per_wg % 128) return TKA_EINVAL;
    return launch_probe_gather(p, a->tokens_per_wg, (hipStream_t)a->stream);
  }
  return TKA_EUNSUPPORTED;
}

// ---- per-kernel timing ------------------------------------------------------------------------

int tka_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  g_profile_on = on != 0;
  return TKA_OK;
}

int tka_profile_reset(void) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  drain_pending();
  g_totals.clear();
  return TKA_OK;
}

int tka_profile_read(const char** names, double* total_ms, int64_t* launches, int cap) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  drain_pending();
  int n = 0;
  for (const KernelTotal& k : g_totals) {
    if (n >= cap) break;
    if (names) names[n] = k.name;
    if (total_ms) total_ms[n] = k.ms;
    if (launches) launches[n] = k.launches;
    ++n;
  }
  return n;
}

}  // extern "C"
