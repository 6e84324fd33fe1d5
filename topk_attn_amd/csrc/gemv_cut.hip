// Stage 1, GEMV phase for a FEW segments of middling length (a single head of 32768 keys): problems that no launch
// fills for long, so that what counts is the number of launches and of dependent round trips to memory, not bytes.
//
// Every workgroup scores its own slice of 256 tokens AND the same 256 sample tokens of its segment (spread evenly
// over the segment, at hashed offsets; after the first workgroup they come from the L2), all loads in flight
// together.  From the sample it takes the R-th largest element in the full order (score descending, token
// ascending): the segment's cut.  All workgroups of a segment compute the same cut from the same rows, so nobody
// waits for anybody.  Tokens at or above the cut are stored as the slice's candidates, as composites in token
// order.  The candidates are an upper set of the order, so whenever at least k of them exist they contain the top
// k; the ranking kernel (select_rank_kernel) checks that and otherwise redoes the segment from the keys.  About
// n R / 256 candidates per segment, see gemv_cut_plan.
//
// On calls that do fill the GPU (more than 65536 rows) the sample is scored once per segment instead: by the first
// workgroups of the GEMV launch, whose cut the others wait for (gemv_cut_slices_kernel), or by a launch before it
// (cut_sample_kernel).  Same cut, same slices, same ranking kernel.
//
// The scores are the canonical ones (gemv_topk.cu:303-332 of the reference: fma chain over the lane's 8 dims,
// xor butterfly over 16 lanes, one multiply).
#include <math.h>

#include "kernels.hpp"

namespace tka {

namespace {

constexpr int kCutThreads = 1024;
constexpr int kCutUnroll = 8;                                        // rows per lane

// Ranks of the S samples of a segment by counting, on the workgroup's 1024 threads (sh_rank must be zero and the keys in
// place behind a barrier): thread (s, q) counts the samples of block q (a quarter or a half of them, broadcast reads)
// that come before sample s, the threads of a sample add up in LDS.  The order is that of the ranking keys (the key
// with its last bits replaced by S - 1 - sample number, see ranking_key): all different, so one compare decides, exactly
// one sample holds rank R - 1, and samples that share a key (heavy ties) come in token order, as in the full order (key
// descending, token ascending).  Keys that differ in their last 8 bits only may change places; any sample will do as
// the cut, it is its rank among the samples that makes the number of candidates what was planned.
// The sample of rank R is the cut (sh_cut: its key and token); the samples whose ranks the bytes of `ranks` name (the last
// one is R, see gemv_cut_split_ranks) split the candidates into eight parts for the ranking kernel's eight workgroups
// per segment, and go to `splits` as composites when that is not null (the last one is the cut).  No barrier behind
// the last write.
// ANNOUNCED: other workgroups of the same launch are going to read `splits` (see gemv_cut_slices_kernel): the stores go
// to where every CU sees them and have got there when this function returns.
template <int S>
__device__ __forceinline__ uint32_t ranking_key(uint32_t key, int i) {
  return (key & ~(uint32_t)(S - 1)) | (uint32_t)(S - 1 - i);
}

template <int S, bool ANNOUNCED = false>
__device__ __forceinline__ void rank_samples(const uint32_t* sh_skey, const uint32_t* sh_rkey, uint32_t* sh_rank, uint32_t* sh_cut, int seg,
                                             int64_t stride, uint64_t ranks, uint64_t* splits) {
  const int tid = threadIdx.x;
  constexpr int kShare = kCutThreads / S;   // threads per sample: 4 (S = 256) or 2 (S = 512), each with 1 / kShare of the samples
  static_assert(kShare * S == kCutThreads && (S / kShare) % 4 == 0, "all threads count");
  {
    const int s = tid & (S - 1), q = tid / S;   // q is the same for a whole wave
    const uint32_t ks = sh_rkey[s];
    const u32x4* blk = (const u32x4*)(sh_rkey + q * (S / kShare));
    uint32_t ahead = 0;
#pragma unroll 16
    for (int i = 0; i < S / kShare / 4; ++i) {
      const u32x4 kj = blk[i];
      ahead += (kj[0] > ks ? 1u : 0u) + (kj[1] > ks ? 1u : 0u) + (kj[2] > ks ? 1u : 0u) + (kj[3] > ks ? 1u : 0u);
    }
    atomicAdd(&sh_rank[s], ahead);
  }
  __syncthreads();
  if (tid < S) {
    const uint32_t r = sh_rank[tid] + 1u;   // 1-based
    uint32_t part = 0;   // 1 .. 8 when this sample ends part `part` of the candidates (8: the cut itself)
#pragma unroll
    for (uint32_t gq = 1; gq <= (uint32_t)kCutParts; ++gq) part = r == ((uint32_t)(ranks >> (8 * (gq - 1))) & 0xffu) ? gq : part;
    if (part != 0) {   // (the ranks are all different: every part has a sample of its own)
      const uint32_t token = (uint32_t)cut_sample_token(seg, tid, stride);
      if (part == (uint32_t)kCutParts) { sh_cut[0] = sh_skey[tid]; sh_cut[1] = token; }
      if (ANNOUNCED) {
        __hip_atomic_store(splits + (int64_t)seg * kCutParts + (part - 1), composite(sh_skey[tid], token), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      } else if (splits) {
        splits[(int64_t)seg * kCutParts + (part - 1)] = composite(sh_skey[tid], token);
      }
    }
  }
}

// The group's query heads summed per dim, for a kernel that is short of registers (eight rows in flight per lane and two
// workgroups of 1024 threads per CU leave 64; with the heads of a group in registers beside the rows the kernel took
// 107 and ran one workgroup per CU): the first 16 G threads load one 16-byte piece of one head each, the
// converted values go through LDS (sh_q: 8 x 128 floats), and behind a barrier of the whole workgroup every thread adds up
// its 8 dims head after head - the order of load_group_query, so the sums are the same bit for bit.
// The piece of the query that this thread brings (one of the first 16 G threads: 16 bytes of head tid / 16), asked for
// here and used in group_query_through_lds.
__device__ __forceinline__ u32x4 group_query_piece(const GemvParams& p, int b, int h, int j) {
  const int tid = threadIdx.x;
  u32x4 w = (u32x4){0u, 0u, 0u, 0u};
  if (tid < 16 * p.group)
    w = *(const u32x4*)((const uint16_t*)p.q + (int64_t)b * p.q_stride_b + ((int64_t)h * p.group + (tid >> 4)) * kHeadDim + 8 * j);
  return w;
}
template <int DT>
__device__ __forceinline__ void group_query_through_lds(const GemvParams& p, const u32x4& w, int j, float* sh_q, float (&qf)[8]) {
  const int tid = threadIdx.x;
  if (tid < 16 * p.group) {
    float* dst = sh_q + (tid >> 4) * kHeadDim + 8 * j;
    *(f32x4*)dst = (f32x4){Elem<DT>::get(w, 0), Elem<DT>::get(w, 1), Elem<DT>::get(w, 2), Elem<DT>::get(w, 3)};
    *(f32x4*)(dst + 4) = (f32x4){Elem<DT>::get(w, 4), Elem<DT>::get(w, 5), Elem<DT>::get(w, 6), Elem<DT>::get(w, 7)};
  }
  __syncthreads();
  const float* src = sh_q + 8 * j;
  f32x4 lo = *(const f32x4*)src, hi = *(const f32x4*)(src + 4);
#pragma unroll 1
  for (int g = 1; g < p.group; ++g) {
    lo += *(const f32x4*)(src + g * kHeadDim);
    hi += *(const f32x4*)(src + g * kHeadDim + 4);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    qf[i] = lo[i];
    qf[4 + i] = hi[i];
  }
}

// Where a workgroup of these kernels works.  Their grids have y = KV head and chunk and z = batch entry (x: the place
// inside the segment), so that no division by a run-time value stands in front of the first load - the hardware has
// none: each costs some twenty-five instructions, and the five of a flat grid were 0.8 us of c1's 13.5.
struct SegPos {
  int b, h, chunk, seg;
};
__device__ __forceinline__ SegPos seg_position(const GemvParams& p) {
  SegPos s;
  s.b = (int)blockIdx.z;
  s.h = (int)blockIdx.y;
  s.chunk = 0;
  if (p.num_chunks != 1) {
    s.h = (int)(blockIdx.y / (uint32_t)p.num_chunks);
    s.chunk = (int)blockIdx.y - s.h * p.num_chunks;
  }
  s.seg = s.b * (int)gridDim.y + (int)blockIdx.y;
  return s;
}
// The same from a segment number (a flat grid): divisions only where a call has several chunks per head, or several
// batch entries.
__device__ __forceinline__ SegPos seg_position_flat(const GemvParams& p, int seg) {
  SegPos s;
  s.seg = seg;
  int bh = seg;
  s.chunk = 0;
  if (p.num_chunks != 1) {
    bh = (int)((uint32_t)seg / (uint32_t)p.num_chunks);
    s.chunk = seg - bh * p.num_chunks;
  }
  s.b = 0;
  s.h = bh;
  if (p.batch != 1) {
    s.b = (int)((uint32_t)bh / (uint32_t)p.num_kv_heads);
    s.h = bh - s.b * p.num_kv_heads;
  }
  return s;
}
static bool grid_ok(const GemvParams& p) { return (int64_t)p.num_kv_heads * p.num_chunks <= 65535 && p.batch <= 65535; }

// The candidates of a workgroup's TOKENS tokens (keys in sh_key, thread t owns token t_begin + t; the threads beyond
// TOKENS have left) to the slices of L tokens that they belong to: tokens at or above `cut` in the order, as composites
// (key << 32 | ~token, token counted inside the segment) ascending in token; the first kCutHead of a slice go to its
// place in the dense head array, which is always written whole (zeros behind the last candidate: no composite is
// zero), the rest to the slice's place in the wide array; the slice's count goes to its own word (kCutGaveUp without a
// cut).  L: 256, or 128 where k is a larger share of the segment and a slice of 256 would overflow its head entries.
template <int TOKENS, int L>
__device__ __forceinline__ void store_slices(const GemvParams& p, int seg, int t_begin, int n_local, const uint32_t* sh_key, uint32_t* sh_wcnt,
                                             uint64_t cut, bool have_cut) {
  static_assert(L % kWave == 0 && L >= kCutHead && TOKENS % L == 0, "whole waves per slice, a thread per head entry");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = tid / L, t_in = tid % L;
  const uint32_t token = (uint32_t)(t_begin + tid);
  const uint64_t mine = composite(sh_key[tid], token);
  const bool pass = have_cut && tid < n_local && mine >= cut;
  const unsigned long long mask = __ballot(pass);
  if (lane == 0) sh_wcnt[wave] = (uint32_t)__popcll(mask);
  __syncthreads();   // (the waves that have ended no longer count)
  uint32_t ahead = 0, total = 0;
#pragma unroll
  for (int v = 0; v < L / kWave; ++v) {
    const int w = sub * (L / kWave) + v;
    const uint32_t c = sh_wcnt[w];
    ahead += w < wave ? c : 0u;
    total += c;
  }
  const int slice = t_begin / L + sub;
  if (slice >= p.wgs_per_chunk) return;   // (p.wgs_per_chunk counts the slices of a segment: its last workgroup may have fewer)
  const int64_t slice_id = (int64_t)seg * p.wgs_per_chunk + slice;
  uint64_t* head = p.cand_head + slice_id * kCutHead;
  uint64_t* wide = p.cand + (int64_t)seg * p.cand_seg_stride + (int64_t)slice * L;
  if (pass) {
    const uint32_t pos = ahead + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
    (pos < (uint32_t)kCutHead ? head : wide)[pos] = mine;
  }
  if ((uint32_t)t_in >= total && t_in < kCutHead) head[t_in] = 0ull;
  if (t_in == 0) p.cand_count[slice_id] = have_cut ? total : kCutGaveUp;
}

// Row groups 0 .. 31 score the 256 tokens of the slice, the row groups behind them the S sample tokens (S = 256:
// sixteen waves), one round of eight loads per lane.
// Many waves and a short program: few workgroups run at a time on these problems, so a wave pays the first fetch
// of every line of code itself (the same rows on four waves with four rounds each: 9.6 instead of 8.1 us).
template <int DT, int S, int L>
__global__ __launch_bounds__(kCutThreads) void gemv_cut_kernel(GemvParams p) {
  constexpr int kCutSamples = S;
  constexpr int kCutRows = kCutTokensPerWg + S;
  static_assert(S == 64 || S == 256, "samples per segment (a power of two, 4 S threads rank them)");
  __shared__ __attribute__((aligned(16))) uint32_t sh_key[kCutRows];   // [0, 256) the slice, then the sample
  __shared__ uint32_t sh_wcnt[kCutTokensPerWg / kWave];
  __shared__ uint32_t sh_cut[2];
  __shared__ uint32_t sh_rank[kCutSamples];
  __shared__ __attribute__((aligned(16))) uint32_t sh_rkey[kCutSamples];   // ranking keys of the samples

  const int tid = threadIdx.x;
  const int j = tid & 15, rg = tid >> 4;
  const int slice = (int)blockIdx.x;   // this workgroup's 256 tokens inside the segment
  const SegPos at = seg_position(p);
  const int b = at.b, h = at.h, chunk = at.chunk, seg = at.seg;
  const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
  const int n = (int)p.chunk_len;
  const int t_begin = slice * kCutTokensPerWg;
  const int n_local = n - t_begin < kCutTokensPerWg ? n - t_begin : kCutTokensPerWg;
  const int64_t stride = n / kCutSamples;

  // the rows are asked for first and the query behind them: its conversion waits for it, and that wait would
  // otherwise stand in front of the row loads (one more round trip to memory in a kernel made of a few)
  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  const bool sampler = rg >= kCutTokensPerWg / kCutUnroll;   // (whole waves: each runs one side of the branch only)
  u32x4 kv[kCutUnroll];
  if (sampler) {
#pragma unroll
    for (int u = 0; u < kCutUnroll; ++u)
      kv[u] = *(const u32x4*)(kbase + cut_sample_token(seg, (rg * kCutUnroll + u) & (kCutSamples - 1), stride) * p.key_stride_n);
  } else {
#pragma unroll
    for (int u = 0; u < kCutUnroll; ++u) {
      const int row = rg * kCutUnroll + u;
      kv[u] = *(const u32x4*)(kbase + (int64_t)(t_begin + (row < n_local ? row : n_local - 1)) * p.key_stride_n);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  float qf[8];
  load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf);
  __builtin_amdgcn_sched_barrier(0);
  float mine = 0.0f;
#pragma unroll
  for (int u = 0; u < kCutUnroll; ++u) {
    const float sc = row_score<DT>(qf, kv[u], p.scale);
    if (j == u) mine = sc;
  }
  if (j < kCutUnroll) {
    const int row = rg * kCutUnroll + j;
    const uint32_t key = score_key(mine);
    sh_key[row] = key;
    if (sampler) sh_rkey[row - kCutTokensPerWg] = ranking_key<S>(key, row - kCutTokensPerWg);
  }
  if (tid < kCutSamples) sh_rank[tid] = 0;
  __syncthreads();

  rank_samples<S>(sh_key + kCutTokensPerWg, sh_rkey, sh_rank, sh_cut, seg, stride, p.split_ranks, slice == 0 ? p.cut_splits : nullptr);
  __syncthreads();
  if (tid >= kCutTokensPerWg) return;

  store_slices<kCutTokensPerWg, L>(p, seg, t_begin, n_local, sh_key, sh_wcnt, composite(sh_cut[0], sh_cut[1]), true);
}


// ---- the same route for calls that fill the GPU -----------------------------------------------------------------
// When a call has more rows than a few CUs' worth, scoring the sample again in every workgroup doubles the work of the
// launch.  Then one workgroup per segment finds the cut and the part ends (sample_segment), and the GEMV workgroups
// read them (gemv_cut_slices_kernel: 512 tokens, two slices, per workgroup, nothing scored twice).

// The work of one workgroup for one segment's cut: the kCutSamplesOnce sample rows (64 row groups, four rows per lane),
// their ranks, cut and part ends (to p.cut_splits).  Every thread of the 1024 calls it.  (With 512 samples the cut sits
// tighter - a fifth fewer candidates - and the part ends are steadier, eight samples per part instead of five; but the
// scoring workgroups wait for this one, and its longer counting cost them more than the ranking kernel gained: 8 x 32768
// tokens 37.8 instead of 33.9 us per decode step.)
// QLDS: the query through LDS (sh_q, see group_query_through_lds) instead of through registers.
template <int DT, bool ANNOUNCED, bool QLDS = false>
__device__ __forceinline__ void sample_segment(const GemvParams& p, const SegPos& at, float* sh_q = nullptr) {
  constexpr int S = kCutSamplesOnce, kRows = S / (kCutThreads / 16);
  __shared__ uint32_t sh_skey[S];
  __shared__ __attribute__((aligned(16))) uint32_t sh_rkey[S];
  __shared__ uint32_t sh_rank[S];
  __shared__ uint32_t sh_cut[2];
  const int tid = threadIdx.x;
  const int j = tid & 15, rg = tid >> 4;
  const int b = at.b, h = at.h, chunk = at.chunk, seg = at.seg;
  const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
  const int64_t stride = p.chunk_len / S;
  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  u32x4 kv[kRows];
#pragma unroll
  for (int u = 0; u < kRows; ++u) kv[u] = *(const u32x4*)(kbase + cut_sample_token(seg, rg * kRows + u, stride) * p.key_stride_n);
  __builtin_amdgcn_sched_barrier(0);
  float qf[8];
  if (QLDS) group_query_through_lds<DT>(p, group_query_piece(p, b, h, j), j, sh_q, qf);
  else load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf);
  __builtin_amdgcn_sched_barrier(0);
  float mine = 0.0f;
#pragma unroll
  for (int u = 0; u < kRows; ++u) {
    const float sc = row_score<DT>(qf, kv[u], p.scale);
    if (j == u) mine = sc;
  }
  if (j < kRows) {
    const int i = rg * kRows + j;
    const uint32_t key = score_key(mine);
    sh_skey[i] = key;
    sh_rkey[i] = ranking_key<S>(key, i);
  }
  if (tid < S) sh_rank[tid] = 0;
  __syncthreads();
  rank_samples<S, ANNOUNCED>(sh_skey, sh_rkey, sh_rank, sh_cut, seg, stride, p.split_ranks, p.cut_splits);
}

// One workgroup per 512 tokens (two slices of the ranking kernel's layout): scores, and the tokens at or above the
// segment's cut in p.cut_splits, stored as in gemv_cut_kernel.
// The first workgroups of the launch, one per segment, find the cuts (sample_segment) while the others score their tokens;
// each publishes its cut and part ends and
// then the call's epoch in the segment's word of p.tau_words, for which the first thread of a scoring workgroup waits
// before the compare - a bounded wait: a workgroup that never sees the word marks its slices (kCutGaveUp in the count),
// and the ranking kernel redoes such a segment from the keys.  The sampling workgroups come first in the grid, so they
// run before any workgroup that waits for them; nothing depends on that but the speed.  With p.samplers_score they are not
// extra workgroups: having published their segment's cut they score the tokens that their place in the grid names, like
// the others (the cut they then wait for is that of a sampling workgroup no later in the grid than themselves).
template <int DT, int L>
__global__ __launch_bounds__(kCutThreads, 8) void gemv_cut_slices_kernel(GemvParams p) {
  constexpr bool FRONT = true;   // (the cuts come from the first workgroups of this launch)
  constexpr int kTokens = 2 * kCutTokensPerWg;
  __shared__ uint32_t sh_key[kTokens];
  __shared__ uint32_t sh_wcnt[kTokens / kWave];
  __shared__ uint64_t sh_cutc[2];   // the cut composite, whether it has arrived
  __shared__ __attribute__((aligned(16))) float sh_q[8 * kHeadDim];   // the query heads of the group, converted
  const int tid = threadIdx.x;
  // FRONT: a flat grid, the sampling workgroups of all segments first (in a grid with the segments in y and z every
  // segment's own would come right before its scoring workgroups - too late on calls of several generations of
  // workgroups: 16 x 32768 tokens 56 instead of 50 us per decode step), then the scoring workgroups segment by segment -
  // or, with p.interleave_segs, token range by token range: consecutive workgroups then read neighbouring heads' rows of
  // the same tokens, which lie side by side in a cache of the usual layout
  int pair;
  SegPos at;
  if (FRONT) {
    const int segs = p.batch * p.num_kv_heads * p.num_chunks;
    uint32_t wg = blockIdx.x;
    if ((int)blockIdx.x < segs) {
      __builtin_amdgcn_s_setprio(3);   // everyone else waits for these few waves
      const SegPos mine = seg_position_flat(p, (int)blockIdx.x);
      sample_segment<DT, true, true>(p, mine, sh_q);
      // the part ends have completed (rank_samples) before the word that announces them leaves; relaxed device-scope
      // accesses on both sides, as for the thresholds of the candidate route: a fence would write back and invalidate
      // whole caches in the middle of the stream
      __syncthreads();
      if (tid == 0 && !(p.withhold_mod > 0 && mine.seg % p.withhold_mod == p.withhold_rem))   // (testing: this segment's word is withheld)
        __hip_atomic_store(p.tau_words + 2 * mine.seg, (uint64_t)p.epoch << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // (the epoch where the candidate route keeps its own)
      if (!p.samplers_score) return;
      __builtin_amdgcn_s_setprio(0);
    } else if (!p.samplers_score) {
      wg -= (uint32_t)segs;
    }
    uint32_t seg;
    if (p.interleave_segs) {
      const uint32_t usegs = (uint32_t)segs;
      const uint32_t q = (usegs & (usegs - 1u)) == 0u ? wg >> (31 - __builtin_clz(usegs)) : wg / usegs;
      seg = wg - q * usegs;
      pair = (int)q;
    } else {
      const uint32_t per_seg = (uint32_t)((p.chunk_len + kTokens - 1) / kTokens);
      seg = (per_seg & (per_seg - 1u)) == 0u ? wg >> (31 - __builtin_clz(per_seg)) : wg / per_seg;   // (mostly a power of two)
      pair = (int)(wg - seg * per_seg);
    }
    at = seg_position_flat(p, (int)seg);
  } else {
    at = seg_position(p);
    pair = (int)blockIdx.x;   // this workgroup's 512 tokens inside the segment
  }
  const int b = at.b, h = at.h, chunk = at.chunk, seg = at.seg;
  const int j = tid & 15, rg = tid >> 4;
  const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
  const int n = (int)p.chunk_len;
  const int t_begin = pair * kTokens;
  const int n_local = n - t_begin < kTokens ? n - t_begin : kTokens;

  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  // (the query piece first: it has arrived, and is converted, while the rows are still on their way)
  const u32x4 qpiece = group_query_piece(p, b, h, j);
  u32x4 kv[kCutUnroll];
#pragma unroll
  for (int u = 0; u < kCutUnroll; ++u) {
    const int row = rg * kCutUnroll + u;
    kv[u] = __builtin_nontemporal_load((const u32x4*)(kbase + (int64_t)(t_begin + (row < n_local ? row : n_local - 1)) * p.key_stride_n));
  }
  uint64_t cut = 0;
  __builtin_amdgcn_sched_barrier(0);
  float qf[8];
  group_query_through_lds<DT>(p, qpiece, j, sh_q, qf);
  __builtin_amdgcn_sched_barrier(0);
  float mine = 0.0f;
#pragma unroll
  for (int u = 0; u < kCutUnroll; ++u) {
    const float sc = row_score<DT>(qf, kv[u], p.scale);
    if (j == u) mine = sc;
    __builtin_amdgcn_sched_barrier(0);   // row after row: scheduled together, the rows' converted values take 100 registers
  }
  if (j < kCutUnroll) sh_key[rg * kCutUnroll + j] = score_key(mine);
  bool have_cut = true;
  if (FRONT) {
    if (tid == 0) {
      const uint64_t* word = p.tau_words + 2 * seg;
      uint64_t v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      for (int spin = 0; (uint32_t)(v >> 32) != p.epoch && spin < p.tau_spin_limit; ++spin) {
        __builtin_amdgcn_s_sleep(16);
        v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      const bool ok = (uint32_t)(v >> 32) == p.epoch;
      // The cut was written, and had completed, before the word that announces it; it is asked for only behind the poll
      // that has seen the word.  The hardware returns a wave's loads in the order they were issued; the fence keeps the
      // compiler from issuing them in another.
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
      sh_cutc[1] = ok ? 1ull : 0ull;
      sh_cutc[0] = ok ? __hip_atomic_load(p.cut_splits + (int64_t)seg * kCutParts + (kCutParts - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : ~0ull;
    }
  }
  __syncthreads();
  if (tid >= kTokens) return;
  if (FRONT) {
    cut = sh_cutc[0];
    have_cut = sh_cutc[1] != 0ull;
  }

  store_slices<kTokens, L>(p, seg, t_begin, n_local, sh_key, sh_wcnt, cut, have_cut);
}

}  // namespace

// p.tokens_per_wg: the slice length (256 or 128), p.wgs_per_chunk: the slices of a segment.
static bool slices_ok(const GemvParams& p) {
  return (p.tokens_per_wg == kCutTokensPerWg || p.tokens_per_wg == kCutTokensPerWg / 2) &&
         p.wgs_per_chunk == (int)((p.chunk_len + p.tokens_per_wg - 1) / p.tokens_per_wg) && p.wgs_per_chunk <= kCutMaxSlices && p.cand &&
         p.cand_head && p.cand_count && p.cut_splits;
}

int launch_gemv_cut(const GemvParams& p, int dtype, hipStream_t stream) {
  const int64_t segs = (int64_t)p.batch * p.num_kv_heads * p.num_chunks;
  const int64_t wgs_per_seg = (p.chunk_len + kCutTokensPerWg - 1) / kCutTokensPerWg;
  if (!slices_ok(p) || p.num_samples != 256 || p.chunk_len < p.num_samples || p.sample_rank < kCutParts || p.sample_rank > p.num_samples ||
      segs * wgs_per_seg > 0x7fffffffLL || !grid_ok(p))
    return TKA_EINVAL;
  const dim3 wgs((unsigned)wgs_per_seg, (unsigned)(p.num_kv_heads * p.num_chunks), (unsigned)p.batch);
  const unsigned threads = (unsigned)(kCutTokensPerWg + p.num_samples) / kCutUnroll * 16;   // 16 lanes per row, 8 rows each
  const bool short_slices = p.tokens_per_wg != kCutTokensPerWg;
  LaunchTimer timer("gemv_cut", stream);
  if (dtype == TKA_F16) {
    if (short_slices) gemv_cut_kernel<TKA_F16, 256, kCutTokensPerWg / 2><<<wgs, threads, 0, stream>>>(p);
    else gemv_cut_kernel<TKA_F16, 256, kCutTokensPerWg><<<wgs, threads, 0, stream>>>(p);
  } else {
    if (short_slices) gemv_cut_kernel<TKA_BF16, 256, kCutTokensPerWg / 2><<<wgs, threads, 0, stream>>>(p);
    else gemv_cut_kernel<TKA_BF16, 256, kCutTokensPerWg><<<wgs, threads, 0, stream>>>(p);
  }
  return hip_status(hipGetLastError());
}

// The cuts come from the first workgroups of the launch (p.tau_words, p.epoch, p.tau_spin_limit, p.num_samples = kCutSamplesOnce,
// p.sample_rank, p.split_ranks, p.cut_splits).
int launch_gemv_cut_slices(const GemvParams& p, int dtype, hipStream_t stream) {
  const int64_t segs = (int64_t)p.batch * p.num_kv_heads * p.num_chunks;
  const int64_t wgs_per_seg = (p.chunk_len + 2 * kCutTokensPerWg - 1) / (2 * kCutTokensPerWg);
  if (!slices_ok(p) || segs * (wgs_per_seg + 1) > 0x7fffffffLL || !grid_ok(p)) return TKA_EINVAL;
  const dim3 wgs((unsigned)(segs * (wgs_per_seg + (p.samplers_score ? 0 : 1))));
  if (p.num_samples != kCutSamplesOnce || p.chunk_len < p.num_samples || p.sample_rank < kCutParts || p.sample_rank > p.num_samples ||
      !p.cut_splits || !p.tau_words || p.epoch == 0 || p.tau_spin_limit < 1)
    return TKA_EINVAL;
  LaunchTimer timer("gemv_cut_slices", stream);
  typedef void (*Kernel)(GemvParams);
  constexpr int kLong = kCutTokensPerWg, kShort = kCutTokensPerWg / 2;
  static const Kernel kernels[2][2] = {   // [dtype][slices of 128 tokens]
      {gemv_cut_slices_kernel<TKA_F16, kLong>, gemv_cut_slices_kernel<TKA_F16, kShort>},
      {gemv_cut_slices_kernel<TKA_BF16, kLong>, gemv_cut_slices_kernel<TKA_BF16, kShort>}};
  hipLaunchKernelGGL(kernels[dtype == TKA_F16 ? 0 : 1][p.tokens_per_wg == kShort ? 1 : 0], wgs, dim3(kCutThreads), 0, stream, p);
  return hip_status(hipGetLastError());
}

// Samples per segment and rank of the cut for a segment of chunk_len tokens and k, or 0 samples when this route
// does not serve the shape.  With S = 256 samples spread evenly and m = k S / n of them expected inside the top k,
// the rank is R = m + 5.5 sqrt(m) + 2 (at least 8: every part of the candidates ends with a sample of its own):
// "fewer than k tokens pass" (the segment is then redone from the keys, still exact) needs R of the samples inside
// the top k, more than five deviations out; about n R / S candidates are stored.  Limits: a slice should stay within
// the kCutHead entries that the ranking kernel reads in its first round trip (40 expected at most: k up to about
// n / 14.5 with slices of 256 tokens; a larger k, up to n / 8, takes slices of 128 tokens where the segment then
// still has no more than kCutMaxSlices of them), and a segment within what it ranks in one go.
// (With 64 samples - enough for a small k on segments of a few thousand rows - the route was measured too: 32 x 4096
// rows, k = 64: 19.5 us against 13.3 on the route that selects in the registers of one workgroup per segment.)
void gemv_cut_plan(int64_t chunk_len, int k, bool sampled_once, int* num_samples, int* sample_rank, int* slice_len) {
  *num_samples = *sample_rank = *slice_len = 0;
  if (chunk_len < 2048 || chunk_len > (int64_t)kCutMaxSlices * kCutTokensPerWg || k > kCutMaxK || (int64_t)k * 8 > chunk_len) return;
  const int s = sampled_once ? kCutSamplesOnce : 256;   // (one workgroup per segment scores the sample, or every workgroup does)
  const double m = (double)k * s / (double)chunk_len;
  int r = (int)ceil(m + 5.5 * sqrt(m) + 2.0);
  if (r < kCutParts) r = kCutParts;
  int len = kCutTokensPerWg;
  if ((double)len * r / s > 40.0) len /= 2;
  const double per_slice = (double)len * r / s, per_segment = (double)chunk_len * r / s;
  if (r * 2 > s || per_slice > 40.0 || (chunk_len + len - 1) / len > kCutMaxSlices || per_segment * 1.2 > (double)kCutMaxCandidates) return;
  *num_samples = s;
  *sample_rank = r;
  *slice_len = len;
}

// Ranks (1-based, among the samples in descending order) of the samples that end the kCutParts parts of a segment's
// candidates, one per byte.  Only the parts that reach into the top k are ranked at all, and the top k ends near sample
// rank m = k S / n, far above the cut at rank R: seven parts share the ranks up to m + 2 sqrt(m) + 1 evenly, and the
// last part takes the rest down to the cut - it is ranked in one call in fifty (the k-th token two deviations below
// its expected place among the samples).  Splitting all R ranks evenly left five of the eight ranking workgroups
// without work and gave the others parts of twice the size.
uint64_t gemv_cut_split_ranks(int64_t chunk_len, int k, int num_samples, int sample_rank) {
  static_assert(kCutParts == 8, "one byte per part");
  const double m = (double)k * num_samples / (double)chunk_len;
  int upper = (int)ceil(m + 2.0 * sqrt(m) + 1.0);
  if (upper > sample_rank - 1) upper = sample_rank - 1;
  if (upper < kCutParts - 1) upper = kCutParts - 1;
  uint64_t ranks = 0;
  int last = 0;
  for (int g = 1; g < kCutParts; ++g) {
    int r = (upper * g + (kCutParts - 2)) / (kCutParts - 1);   // ceil(upper g / 7)
    if (r <= last) r = last + 1;
    last = r;
    ranks |= (uint64_t)r << (8 * (g - 1));
  }
  // (sample_rank >= kCutParts and upper <= sample_rank - 1: the last of the seven lies below sample_rank)
  ranks |= (uint64_t)sample_rank << (8 * (kCutParts - 1));
  return ranks;
}

}  // namespace tka
