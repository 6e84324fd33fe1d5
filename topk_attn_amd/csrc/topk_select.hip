// Stage 1, selection phase: exact top-k of fp32 scores per segment, ties to the lower index.
// Replaces the full cub::BlockRadixSort of the reference (gemv_topk.cu:353-378) with a radix SELECT;
// only a caller that wants rank order pays for a sort, and then of the k survivors only.
//
// Every element is ranked by the 64-bit composite (score key << 32) | ~index, so all elements are
// distinct and "top k" is unique: score descending, index ascending.
//
//   1. first-level histogram of the top 11 key bits (by the GEMV kernel, or select_hist_kernel);
//   2. filter (workgroups = slices x segments): find the threshold bin b1 from the histogram; every
//      thread reads a contiguous run of its slice with 16-byte loads and the workgroup writes the
//      composites with bin >= b1, in index order, to the slice's own list.  No atomics: the layout is
//      deterministic and each list is ascending in token index;
//   3. finalize (one workgroup per segment): turns the slice counts into offsets, refines the threshold
//      inside bin b1 with further 11-bit radix passes over the listed entries (stops as soon as a
//      bucket is taken whole), then walks the lists in order and
//        - writes the ascending union with the sink / local-window ranges by ordered compaction
//          (no sort), and / or
//        - gathers the k survivors in LDS, sorts them with a bitonic network (registers, DPP /
//          ds_swizzle across lanes, LDS across waves) and writes rank-ordered indices and values.
//
// No workgroup waits for another: the hand-off between 2 and 3 is the kernel boundary (a device-scope
// fence per workgroup would write back the whole L2 of its XCD each time).
// Traffic: 4 B read per score, 8 B written and read per listed element (about k + one bin per segment).
//
// Long segments skip 1 and 2: the GEMV stores only the tokens above a sampled threshold (candidate
// slices), and select_finalize_cand_kernel does step 3 on them from LDS, or, when the slices cannot be
// used, redoes the segment from the keys (fallback_segment).
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <utility>
#include <vector>

#include "kernels.hpp"
#include "bitonic.hpp"
#include "lse_combine.hpp"

namespace tka {

namespace {

constexpr int kSelThreads = kSortThreads;
constexpr int kSelWaves = kSelThreads / kWave;
constexpr int kEndsInLds = 4096;   // slice offsets of one segment kept in LDS by the finalize kernel
constexpr int kEntryCache = 16;    // listed entries per thread kept in registers by the finalize kernel

// ---- kernels ----------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void zero_u32_kernel(uint32_t* p, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// Exclusive prefix of v over the 1024 threads of the block; *total = block sum.  Two barriers.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* sh_wtot, uint32_t* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t inc = wave_inclusive_scan(v);
  __syncthreads();  // sh_wtot may still be read by the previous call
  if (lane == 63) sh_wtot[wave] = inc;
  __syncthreads();
  // the waves' totals: one read by sixteen lanes and two sums across them instead of sixteen reads per thread
  static_assert(kSelWaves == 16, "one lane per wave, summed across sixteen lanes");
  const uint32_t t = lane < kSelWaves ? sh_wtot[lane] : 0u;
  uint32_t all = t, before = lane < wave ? t : 0u;
  all += lane_xor<1>(all);   before += lane_xor<1>(before);
  all += lane_xor<2>(all);   before += lane_xor<2>(before);
  all += lane_xor<4>(all);   before += lane_xor<4>(before);
  all += lane_xor<8>(all);   before += lane_xor<8>(before);
  *total = (uint32_t)__builtin_amdgcn_readfirstlane((int)all);
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)before) + inc - v;
}

// Loads the `per_thread` (4 or 16) consecutive scores of this thread as keys; positions at or beyond
// seg_len get key 0 and valid = false.
template <int PT>
__device__ __forceinline__ void load_keys(const float* sc, int64_t first, int64_t seg_len, bool vec_ok, uint32_t (&keys)[PT],
                                          uint32_t* valid_mask) {
  uint32_t vm = 0;
#pragma unroll
  for (int v = 0; v < PT / 4; ++v) {
    const int64_t i = first + 4 * v;
    if (vec_ok && i + 3 < seg_len) {
      const f32x4 x = *(const f32x4*)(sc + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) keys[4 * v + e] = score_key(x[e]);
      vm |= 0xfu << (4 * v);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool ok = i + e < seg_len;
        keys[4 * v + e] = ok ? score_key(sc[ok ? i + e : 0]) : 0u;
        vm |= (ok ? 1u : 0u) << (4 * v + e);
      }
    }
  }
  *valid_mask = vm;
}

// First-level histogram when the scores do not come from the GEMV kernel.
template <int PT>
__global__ __launch_bounds__(kSelThreads) void select_hist_kernel(SelectParams p) {
  __shared__ uint32_t sh_hist[kHistBins];
  const int tid = threadIdx.x;
  const int seg = blockIdx.y;
  for (int i = tid; i < kHistBins; i += kSelThreads) sh_hist[i] = 0;
  __syncthreads();
  const float* sc = p.scores + (int64_t)seg * p.seg_stride;
  const bool vec_ok = (((uintptr_t)sc) & 15u) == 0;
  uint32_t keys[PT], vm;
  load_keys<PT>(sc, (int64_t)blockIdx.x * p.part_len + (int64_t)tid * PT, p.seg_len, vec_ok, keys, &vm);
#pragma unroll
  for (int e = 0; e < PT; ++e)
    if (vm >> e & 1u) atomicAdd(&sh_hist[keys[e] >> (32 - kHistBits)], 1u);
  __syncthreads();
  uint32_t* gh = p.hist + (int64_t)seg * kHistBins;
  for (int i = tid; i < kHistBins; i += kSelThreads) {
    uint32_t c = sh_hist[i];
    if (c) atomicAdd(&gh[i], c);
  }
}

template <int PT>
__global__ __launch_bounds__(kSelThreads) void select_filter_kernel(SelectParams p) {
  __shared__ uint32_t sh_hist[kHistBins];
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];

  const int tid = threadIdx.x;
  const int seg = blockIdx.y;
  const int part = blockIdx.x;

  // this thread's run of scores first: the loads do not depend on the threshold
  const float* sc = p.scores + (int64_t)seg * p.seg_stride;
  const bool vec_ok = (((uintptr_t)sc) & 15u) == 0;
  const int64_t first = (int64_t)part * p.part_len + (int64_t)tid * PT;
  uint32_t keys[PT], vm;
  load_keys<PT>(sc, first, p.seg_len, vec_ok, keys, &vm);

  // threshold bin from the first-level histogram
  const uint32_t* gh = p.hist + (int64_t)seg * kHistBins;
  sh_hist[2 * tid] = gh[2 * tid];
  sh_hist[2 * tid + 1] = gh[2 * tid + 1];
  __syncthreads();
  find_threshold_bin_1024(sh_hist, (uint32_t)p.k, sh_wtot, sh_res);
  const uint32_t b1 = sh_res[0];

  uint32_t mine = 0;
#pragma unroll
  for (int e = 0; e < PT; ++e) mine += ((vm >> e) & 1u) && (keys[e] >> (32 - kHistBits)) >= b1;
  uint32_t total;
  uint32_t slot = block_exclusive_scan(mine, sh_wtot, &total);
  uint64_t* list = p.list + (int64_t)seg * p.list_stride + (int64_t)part * p.part_len;
#pragma unroll
  for (int e = 0; e < PT; ++e)
    if (((vm >> e) & 1u) && (keys[e] >> (32 - kHistBits)) >= b1) list[slot++] = composite(keys[e], (uint32_t)(first + e));
  if (tid == 0) p.list_cnt[(int64_t)seg * p.parts + part] = total;
}


// Union list of one segment outside the selected middle part: the sink ids, the local window behind
// `mid` selected ids, -1 padding, and the count.
__device__ __forceinline__ void write_union_edges(int32_t* uo, const SelectParams& p, int seg, uint32_t lo, uint32_t hi, uint32_t mid) {
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));   // (inlined into long kernels, inside their loops: addresses are computed here, not kept from the top of the kernel on)
  const int64_t n = p.seg_len;
  const int cap = p.k + p.sink + p.local;
  for (uint32_t t = tid; t < lo; t += kSelThreads) uo[t] = (int32_t)t;
  const uint32_t mid_end = lo + mid;
  for (int64_t t = (int64_t)hi + tid; t < n; t += kSelThreads) uo[mid_end + (t - hi)] = (int32_t)t;
  const uint32_t count = mid_end + (uint32_t)(n - hi);
  for (int i = (int)count + tid; i < cap; i += kSelThreads) uo[i] = -1;
  if (tid == 0) p.union_count[seg] = (int32_t)count;
}

// Rank-ordered outputs of one segment from the sorted composites in sh_sort[0 .. k).
// (`chunk`: the segment's number inside its row, for a caller that has it without a division; -1: seg % p.segs_per_row)
__device__ __forceinline__ void write_rank_outputs(const uint64_t* sh_sort, const SelectParams& p, int seg, int chunk = -1) {
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));   // (as in write_union_edges)
  const uint32_t k = (uint32_t)p.k;
  const uint32_t idx_base = p.seg_base_ids ? (uint32_t)(p.seg_base_ids[seg] * p.seg_len)
                                           : (uint32_t)((chunk >= 0 ? chunk : seg % p.segs_per_row) * p.seg_len);
  int32_t* oi = p.out_idx + (int64_t)seg * p.out_stride;
  float* ov = p.out_val ? p.out_val + (int64_t)seg * p.out_stride : nullptr;
  for (uint32_t r = tid; r < k; r += kSelThreads) {
    uint64_t c = sh_sort[r];
    oi[r] = (int32_t)(~(uint32_t)c + idx_base);
    if (ov) ov[r] = key_score((uint32_t)(c >> 32));
  }
  if (p.out_expand) {
    // a wave per selected id, a lane per member of its cluster (no division by the cluster length)
    int32_t* oe = p.out_expand + (int64_t)seg * p.k * p.expand;
    const uint32_t lane = (uint32_t)tid & 63u, expand = (uint32_t)p.expand;
    for (uint32_t jj = (uint32_t)tid >> 6; jj < k; jj += kSelThreads / kWave) {
      const uint32_t first = ~(uint32_t)sh_sort[jj] * expand;
      for (uint32_t ii = lane; ii < expand; ii += kWave) oe[jj * expand + ii] = (int32_t)(first + ii);
    }
  }
}

// Rank order of the k selected composites in sh_sort[0 .. k) (any order on entry; [k, kpad) must be zero), descending
// on exit.  Instead of a bitonic network over all of them: key minus smallest key, cut to its 11 leading bits,
// gives up to 2048 buckets in rank order; a histogram and one suffix scan give every bucket its first rank; the
// composites are scattered to their bucket (sh_xchg) and each one counts the larger members of its own bucket.
// Buckets are small on ordinary data (k / (occupied buckets)); when one exceeds kRankBucketMax (heavy ties in
// the score AND neighbouring indices, or k < 3) the bitonic network does the job instead.
// sh_xchg: kpad composites; sh_hist, sh_off: 2048 words each; sh_mm: 2 composites + 1 word.  All 1024 threads call.
constexpr uint32_t kRankBucketMax = 96;
__device__ __forceinline__ void rank_sort_desc(uint64_t* sh_sort, uint64_t* sh_xchg, uint32_t k, int kpad, uint32_t* sh_hist,
                                               uint32_t* sh_off, uint32_t* sh_wtot, uint64_t* sh_mm) {
  if (kpad <= 1024) {   // a small network (one composite per thread) is quicker than the bucket bookkeeping
    sort_lds_desc(sh_sort, sh_xchg, kpad);
    return;
  }
  int tid = threadIdx.x;
  // (inlined into long kernels, some of them inside loops: the addresses below are computed here, from a thread number
  // that the compiler cannot trace, instead of being kept in registers from the top of the kernel on)
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = tid >> 6;
  constexpr int kMaxPer = TKA_MAX_TOPK / kSelThreads;   // 8 composites per thread at most
  uint32_t* sh_big = (uint32_t*)(sh_mm + 2);
  uint64_t c[kMaxPer];
  uint64_t cmin = ~0ull, cmax = 0ull;
#pragma unroll
  for (int e = 0; e < kMaxPer; ++e) {
    const uint32_t i = (uint32_t)e * kSelThreads + tid;
    c[e] = i < k ? sh_sort[i] : 0ull;
    if (i < k) {
      cmin = c[e] < cmin ? c[e] : cmin;
      cmax = c[e] > cmax ? c[e] : cmax;
    }
  }
  if (tid == 0) { sh_mm[0] = ~0ull; sh_mm[1] = 0ull; *sh_big = 0u; }
  sh_hist[2 * tid] = 0;
  sh_hist[2 * tid + 1] = 0;
  __syncthreads();
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint64_t a = __shfl_xor(cmin, d, 64), b = __shfl_xor(cmax, d, 64);
    cmin = a < cmin ? a : cmin;
    cmax = b > cmax ? b : cmax;
  }
  if (lane == 0) {
    atomicMin((unsigned long long*)&sh_mm[0], (unsigned long long)cmin);
    atomicMax((unsigned long long*)&sh_mm[1], (unsigned long long)cmax);
  }
  __syncthreads();
  cmin = sh_mm[0];
  cmax = sh_mm[1];
  // buckets are linear in (key - smallest key): the bits of a float key that two scores share say little once
  // the scores straddle a power of two
  const uint64_t base = cmin & 0xffffffff00000000ull;
  const int fixed = cmax - base == 0 ? 64 - kHistBits : __builtin_clzll(cmax - base);
  const int bits = (64 - fixed) >= kHistBits ? kHistBits : (64 - fixed);
  const int shift = 64 - fixed - bits;
  uint32_t slot[kMaxPer];
#pragma unroll
  for (int e = 0; e < kMaxPer; ++e) {
    const uint32_t i = (uint32_t)e * kSelThreads + tid;
    slot[e] = i < k ? atomicAdd(&sh_hist[(uint32_t)((c[e] - base) >> shift)], 1u) : 0u;
  }
  __syncthreads();
  // first rank of every bucket: number of composites in higher buckets (thread t owns buckets 2t, 2t+1)
  {
    const uint32_t h0 = sh_hist[2 * tid], h1 = sh_hist[2 * tid + 1];
    const uint32_t mine = h0 + h1;
    const uint32_t inc = wave_inclusive_scan(mine);
    const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
    const uint32_t ge = wave_total - inc + mine;   // this wave's composites in buckets >= 2t
    if (lane == 0) sh_wtot[wave] = ge;
    if (h0 > kRankBucketMax || h1 > kRankBucketMax) *sh_big = 1u;
    __syncthreads();
    uint32_t above = 0;
    for (int w = wave + 1; w < kSelWaves; ++w) above += sh_wtot[w];
    sh_off[2 * tid + 1] = above + ge - mine;        // buckets > 2t+1
    sh_off[2 * tid] = above + ge - h0;              // buckets > 2t
  }
  __syncthreads();
  if (*sh_big != 0u || k < 3u) {
    sort_lds_desc(sh_sort, sh_xchg, kpad);
    return;
  }
#pragma unroll
  for (int e = 0; e < kMaxPer; ++e) {
    const uint32_t i = (uint32_t)e * kSelThreads + tid;
    if (i < k) sh_xchg[sh_off[(uint32_t)((c[e] - base) >> shift)] + slot[e]] = c[e];
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < kMaxPer; ++e) {
    const uint32_t i = (uint32_t)e * kSelThreads + tid;
    if (i < k) {
      const uint64_t x = sh_xchg[i];
      const uint32_t bin = (uint32_t)((x - base) >> shift);
      const uint32_t first = sh_off[bin], cnt = sh_hist[bin];
      uint32_t larger = 0;
      for (uint32_t j = 0; j < cnt; ++j) larger += sh_xchg[first + j] > x ? 1u : 0u;
      sh_sort[first + larger] = x;
    }
  }
  __syncthreads();
}

// Dynamic LDS of select_finalize_kernel (rank mode only): kpad composites (sort buffer), then kpad
// composites (cross-wave exchange buffer).
__global__ __launch_bounds__(kSelThreads) void select_finalize_kernel(SelectParams p, int kpad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint64_t* sh_sort = (uint64_t*)smem;
  uint64_t* sh_xchg = sh_sort + kpad;
  __shared__ uint32_t sh_hist[kHistBins];
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];

  const int tid = threadIdx.x;
  const int seg = blockIdx.x;
  const uint32_t k = (uint32_t)p.k;

  // threshold bin, count above it, count inside it
  uint32_t b1, n_above, n_bin;
  {
    const uint32_t* gh = p.hist + (int64_t)seg * kHistBins;
    sh_hist[2 * tid] = gh[2 * tid];
    sh_hist[2 * tid + 1] = gh[2 * tid + 1];
    __syncthreads();
    find_threshold_bin_1024(sh_hist, k, sh_wtot, sh_res);
    b1 = sh_res[0], n_above = sh_res[1], n_bin = sh_res[2];
  }

  // slice counts -> inclusive offsets (entries of the segment get one running index); kept in LDS when
  // they fit, in place in global memory otherwise
  __shared__ uint32_t sh_ends[kEndsInLds];
  uint32_t* g_ends = p.list_cnt + (int64_t)seg * p.parts;
  const bool ends_in_lds = p.parts <= kEndsInLds;
  uint32_t n_listed = 0;
  {
    for (int base = 0; base < p.parts; base += kSelThreads) {
      const int i = base + tid;
      const uint32_t c = i < p.parts ? g_ends[i] : 0u;
      uint32_t total;
      const uint32_t ex = block_exclusive_scan(c, sh_wtot, &total);
      if (i < p.parts) {
        if (ends_in_lds) sh_ends[i] = n_listed + ex + c; else g_ends[i] = n_listed + ex + c;
      }
      n_listed += total;
    }
    __syncthreads();
  }
  const uint32_t* ends = ends_in_lds ? sh_ends : g_ends;
  const uint32_t n_entries = n_listed;  // == n_above + n_bin
  const uint64_t* lists = p.list + (int64_t)seg * p.list_stride;
  // entry v of the segment: slice s with ends[s-1] <= v < ends[s], position v - ends[s-1] in that slice
  auto fetch = [&](uint32_t v) -> uint64_t {
    int lo = 0, hi = p.parts - 1;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (ends[mid] > v) hi = mid; else lo = mid + 1;
    }
    const uint32_t start = lo ? ends[lo - 1] : 0u;
    return lists[(int64_t)lo * p.part_len + (v - start)];
  };
  // the first kEntryCache*1024 entries live in registers (typical segments fit entirely)
  uint64_t cache[kEntryCache];
#pragma unroll
  for (int i = 0; i < kEntryCache; ++i) {
    const uint32_t v = (uint32_t)i * kSelThreads + tid;
    cache[i] = v < n_entries ? fetch(v) : 0ull;
  }
  auto entry = [&](uint32_t v) -> uint64_t { return fetch(v); };

  // Refine inside bin b1: the listed entries of that bin share their top 11 bits.  Take `need` of them.
  uint32_t need = k - n_above;   // >= 1
  uint64_t prefix = b1;          // value of the bits fixed so far
  int fixed = kHistBits;         // number of top bits fixed
  bool done = need == n_bin;     // whole bin taken
  uint64_t threshold = (uint64_t)b1 << (64 - kHistBits);   // selected: composite >= threshold
  while (!done) {
    const int bits = (64 - fixed) >= kHistBits ? kHistBits : (64 - fixed);
    const int shift = 64 - fixed - bits;
    __syncthreads();
    sh_hist[2 * tid] = 0;
    sh_hist[2 * tid + 1] = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kEntryCache; ++i) {
      const uint64_t c = cache[i];
      if ((uint32_t)i * kSelThreads + tid < n_entries && (c >> (64 - fixed)) == prefix)
        atomicAdd(&sh_hist[(uint32_t)(c >> shift) & ((1u << bits) - 1u)], 1u);
    }
    for (uint32_t v = kEntryCache * kSelThreads + tid; v < n_entries; v += kSelThreads) {
      const uint64_t c = entry(v);
      if ((c >> (64 - fixed)) == prefix) atomicAdd(&sh_hist[(uint32_t)(c >> shift) & ((1u << bits) - 1u)], 1u);
    }
    __syncthreads();
    find_threshold_bin_1024(sh_hist, need, sh_wtot, sh_res);
    const uint32_t d = sh_res[0], gt = sh_res[1], cnt = sh_res[2];
    need -= gt;
    prefix = (prefix << bits) | d;
    fixed += bits;
    if (cnt == need || fixed == 64) {
      threshold = fixed == 64 ? prefix : (prefix << (64 - fixed));
      done = true;
    }
  }

  // Walk the entries in index order.  Union mode: ordered compaction of the selected ids that lie
  // between the sink range and the local window.  Rank mode: selected composites into the sort buffer.
  const bool want_rank = p.out_idx != nullptr;
  const bool want_union = p.union_idx != nullptr;
  const int64_t n = p.seg_len;
  const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
  const uint32_t hi = (uint32_t)(n - p.local > lo ? n - p.local : lo);
  int32_t* uo = want_union ? p.union_idx + (int64_t)seg * (p.k + p.sink + p.local) : nullptr;
  if (want_rank) {
    __syncthreads();
    for (int i = tid; i < kpad; i += kSelThreads) sh_sort[i] = 0;  // pad: below every real composite
  }
  if (want_rank && !want_union) {
    // The sort that follows takes the composites in any order: every wave reserves room for its selected
    // entries with one add, no walk in index order.
    if (tid == 0) sh_res[3] = 0u;
    __syncthreads();
    const int lane = tid & 63;
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < kEntryCache; ++i)
      mine += ((uint32_t)i * kSelThreads + tid < n_entries && cache[i] >= threshold) ? 1u : 0u;
    for (uint32_t v = kEntryCache * kSelThreads + tid; v < n_entries; v += kSelThreads) mine += entry(v) >= threshold ? 1u : 0u;
    const uint32_t inc = wave_inclusive_scan(mine);
    uint32_t first = 0;
    if (lane == 63) first = atomicAdd(&sh_res[3], inc);
    uint32_t pos = (uint32_t)__builtin_amdgcn_readlane((int)first, 63) + inc - mine;
#pragma unroll
    for (int i = 0; i < kEntryCache; ++i)
      if ((uint32_t)i * kSelThreads + tid < n_entries && cache[i] >= threshold) {
        if (pos < k) sh_sort[pos] = cache[i];
        ++pos;
      }
    for (uint32_t v = kEntryCache * kSelThreads + tid; v < n_entries; v += kSelThreads) {
      const uint64_t c = entry(v);
      if (c >= threshold) {
        if (pos < k) sh_sort[pos] = c;
        ++pos;
      }
    }
  }
  uint32_t run_sel = 0, run_mid = 0;
  for (uint32_t base = 0, step = 0; base < n_entries && want_union; base += kSelThreads, ++step) {
    const uint32_t v = base + tid;
    uint64_t c = 0;
    if (step < kEntryCache) {
#pragma unroll
      for (int i = 0; i < kEntryCache; ++i)
        if ((uint32_t)i == step) c = cache[i];
    } else if (v < n_entries) {
      c = entry(v);
    }
    const bool sel = v < n_entries && c >= threshold;
    const uint32_t idx = ~(uint32_t)c;
    uint32_t total;
    if (want_rank) {
      const uint32_t ex = block_exclusive_scan(sel ? 1u : 0u, sh_wtot, &total);
      if (sel && run_sel + ex < k) sh_sort[run_sel + ex] = c;
      run_sel += total;
    }
    if (want_union) {
      const bool mid = sel && idx >= lo && idx < hi;
      const uint32_t ex = block_exclusive_scan(mid ? 1u : 0u, sh_wtot, &total);
      if (mid) uo[lo + run_mid + ex] = (int32_t)idx;
      run_mid += total;
    }
  }
  if (want_union) write_union_edges(uo, p, seg, lo, hi, run_mid);
  if (!want_rank) return;
  __syncthreads();

  __shared__ uint64_t sh_mm[3];
  rank_sort_desc(sh_sort, sh_xchg, k, kpad, sh_hist, sh_ends, sh_wtot, sh_mm);   // (the slice offsets are spent)
  write_rank_outputs(sh_sort, p, seg);
}

// ---- fallback of the candidate mode ---------------------------------------------------------------

// A segment whose candidate slices cannot be used (fewer than k candidates, or more than fit) is redone from
// the keys: scores in the canonical order (stored, and a histogram of the top key bits), radix passes over the stored
// scores until the k-th largest key is fixed, then one walk in index order that takes every key above the threshold
// bucket and the first `need` keys inside it.  Exact for any data.  Two forms: one workgroup does all of it for its
// segment (fallback_segment: one CU streams the segment, about a millisecond per 131072 tokens; the short segments of
// the common-cut route and the combine launch of the one-launch selection + attention), or all workgroups of a launch of
// their own share the work on all flagged segments, phase by phase (redo_segments_kernel; the long segments of the
// candidate route).

// Scores of tokens [t0, t1) of segment `seg` (all 1024 threads: 64 row groups of 16 lanes, 16 rows in flight each),
// stored to the segment's place in g.scores, with the top key bits counted in sh_hist (LDS, 2048 bins; not cleared here).
template <int DT>
__device__ __forceinline__ void fallback_score_range(const GemvParams& g, const SelectParams& p, int seg, int64_t t0, int64_t t1, uint32_t* sh_hist) {
  const int tid = threadIdx.x;
  float* sc = g.scores + (int64_t)seg * p.seg_stride;
  constexpr int kRows = 16;
  const int j = tid & 15, rg = tid >> 4;
  const int chunk = seg % g.num_chunks, bh = seg / g.num_chunks;
  const int h = bh % g.num_kv_heads, b = bh / g.num_kv_heads;
  const int64_t chunk_base = g.cluster_ids ? (int64_t)g.cluster_ids[seg] * g.chunk_len : (int64_t)chunk * g.chunk_len;
  float qf[8];
  load_group_query<DT>(g.q, g.q_stride_b, b, h, g.group, j, qf);
  const uint16_t* kbase = (const uint16_t*)g.keys + (int64_t)b * g.key_stride_b + (int64_t)h * g.key_stride_h +
                          chunk_base * g.key_stride_n + 8 * j;
  for (int64_t base = t0; base < t1; base += (kSelThreads / 16) * kRows) {
    u32x4 kv[kRows];
#pragma unroll
    for (int u = 0; u < kRows; ++u) {
      const int64_t t = base + rg * kRows + u;
      kv[u] = *(const u32x4*)(kbase + (t < t1 ? t : t1 - 1) * g.key_stride_n);
    }
    __builtin_amdgcn_sched_barrier(0);   // all loads go out before the first score is computed
    float mine = 0.0f;
#pragma unroll
    for (int u = 0; u < kRows; ++u) {
      const float s = row_score<DT>(qf, kv[u], g.scale);
      if (j == u) mine = s;
    }
    const int64_t t = base + rg * kRows + j;
    if (j < kRows && t < t1) {
      sc[t] = mine;
      atomicAdd(&sh_hist[score_key(mine) >> (32 - kHistBits)], 1u);
    }
  }
}

template <int DT>
__device__ __forceinline__ void fallback_select_from_scores(const GemvParams& g, const SelectParams& p, int seg, int kpad, uint64_t* sh_sort,
                                                            uint32_t* sh_hist, uint32_t* sh_off, uint32_t* sh_wtot, uint32_t* sh_res,
                                                            uint64_t* sh_mm);

// sh_sort: 2*kpad composites (rank mode only); sh_hist, sh_off: 2048 words each.  Every thread of the block must call it.
template <int DT>
__device__ __forceinline__ void fallback_segment(const GemvParams& g, const SelectParams& p, int seg, int kpad, uint64_t* sh_sort,
                                                 uint32_t* sh_hist, uint32_t* sh_off, uint32_t* sh_wtot, uint32_t* sh_res,
                                                 uint64_t* sh_mm) {
  const int tid = threadIdx.x;
  sh_hist[2 * tid] = 0;
  sh_hist[2 * tid + 1] = 0;
  __syncthreads();
  fallback_score_range<DT>(g, p, seg, 0, p.seg_len, sh_hist);
  __syncthreads();   // also orders this workgroup's score stores before its loads below
  fallback_select_from_scores<DT>(g, p, seg, kpad, sh_sort, sh_hist, sh_off, sh_wtot, sh_res, sh_mm);
}

// The selection half: sh_hist holds the counts of the top key bits of the segment's stored scores.
template <int DT>
__device__ __forceinline__ void fallback_select_from_scores(const GemvParams& g, const SelectParams& p, int seg, int kpad, uint64_t* sh_sort,
                                                            uint32_t* sh_hist, uint32_t* sh_off, uint32_t* sh_wtot, uint32_t* sh_res,
                                                            uint64_t* sh_mm) {
  uint64_t* sh_xchg = sh_sort + kpad;
  const int tid = threadIdx.x;
  const uint32_t k = (uint32_t)p.k;
  const int64_t n = p.seg_len;
  float* sc = g.scores + (int64_t)seg * p.seg_stride;

  // radix passes: `prefix` = value of the top `fixed` key bits of the k-th largest key, `need` = how many
  // keys of that bucket belong to the top k
  const bool vec_ok = (((uintptr_t)sc) & 15u) == 0;
  uint32_t need = k, prefix = 0;
  int fixed = 0;
  bool whole = false;   // the bucket is taken whole
  while (!whole && fixed < 32) {
    const int bits = (32 - fixed) >= kHistBits ? kHistBits : (32 - fixed);
    const int shift = 32 - fixed - bits;
    if (fixed) {
      __syncthreads();
      sh_hist[2 * tid] = 0;
      sh_hist[2 * tid + 1] = 0;
      __syncthreads();
      for (int64_t first = (int64_t)tid * 4; first < n; first += 4 * kSelThreads) {
        uint32_t keys[4], vm;
        load_keys<4>(sc, first, n, vec_ok, keys, &vm);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if ((vm >> e & 1u) && (keys[e] >> (32 - fixed)) == prefix) atomicAdd(&sh_hist[(keys[e] >> shift) & ((1u << bits) - 1u)], 1u);
      }
      __syncthreads();
    }
    find_threshold_bin_1024(sh_hist, need, sh_wtot, sh_res);
    const uint32_t d = sh_res[0], gt = sh_res[1], cnt = sh_res[2];
    need -= gt;
    prefix = (prefix << bits) | d;
    fixed += bits;
    whole = cnt == need;
  }

  // walk in index order
  const bool want_rank = p.out_idx != nullptr;
  const bool want_union = p.union_idx != nullptr;
  const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
  const uint32_t hi = (uint32_t)(n - p.local > lo ? n - p.local : lo);
  int32_t* uo = want_union ? p.union_idx + (int64_t)seg * (p.k + p.sink + p.local) : nullptr;
  if (want_rank) {
    __syncthreads();
    for (int i = tid; i < kpad; i += kSelThreads) sh_sort[i] = 0;  // pad: below every real composite
  }
  uint32_t run_bucket = 0, run_sel = 0, run_mid = 0;
  for (int64_t base = 0; base < n; base += 4 * kSelThreads) {
    const int64_t first = base + (int64_t)tid * 4;
    uint32_t keys[4], vm;
    load_keys<4>(sc, first, n, vec_ok, keys, &vm);
    uint32_t above = 0, inside = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t top = keys[e] >> (32 - fixed);
      above |= ((vm >> e & 1u) && top > prefix ? 1u : 0u) << e;
      inside |= ((vm >> e & 1u) && top == prefix ? 1u : 0u) << e;
    }
    uint32_t total;
    uint32_t rank_in_bucket = run_bucket + block_exclusive_scan((uint32_t)__builtin_popcount(inside), sh_wtot, &total);
    run_bucket += total;
    uint32_t sel = above, mid = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (inside >> e & 1u) {
        sel |= (rank_in_bucket < need ? 1u : 0u) << e;
        ++rank_in_bucket;
      }
      const uint32_t idx = (uint32_t)(first + e);
      mid |= ((sel >> e & 1u) && idx >= lo && idx < hi ? 1u : 0u) << e;
    }
    const uint32_t ex = block_exclusive_scan(((uint32_t)__builtin_popcount(sel) << 16) | (uint32_t)__builtin_popcount(mid), sh_wtot, &total);
    uint32_t pos_sel = run_sel + (ex >> 16), pos_mid = lo + run_mid + (ex & 0xffffu);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (want_rank && (sel >> e & 1u)) sh_sort[pos_sel++] = composite(keys[e], (uint32_t)(first + e));
      if (want_union && (mid >> e & 1u)) uo[pos_mid++] = (int32_t)(first + e);
    }
    run_sel += total >> 16;
    run_mid += total & 0xffffu;
  }
  if (want_union) write_union_edges(uo, p, seg, lo, hi, run_mid);
  if (!want_rank) return;
  __syncthreads();
  rank_sort_desc(sh_sort, sh_xchg, k, kpad, sh_hist, sh_off, sh_wtot, sh_mm);
  write_rank_outputs(sh_sort, p, seg);
}

// ---- finalize of the candidate mode -------------------------------------------------------------

constexpr int kRedoPhasesMax = 8;   // item counters of the redo launch: two words per phase
constexpr int kCandCap = 16384;    // candidates of one segment held in LDS (128 KB of composites)
constexpr int kCandPerThread = kCandCap / kSelThreads;
constexpr int kCandMaxParts = 4096;
constexpr int kSmallBucket = 64;   // a threshold bucket of this many entries or fewer is ranked by one wave

// Candidate mode: the slices hold every token whose key reached the sampled threshold, ascending in token
// index inside and across slices (format: GemvParams::cand).  One workgroup per segment copies them into LDS
// as composites (entry v of the segment at position v), finds the k-th largest composite by radix passes that start below the common prefix of
// the smallest and largest candidate, and walks the entries once in index order.
// A segment with fewer than k candidates, or more than fit, or with a slice whose workgroup gave up waiting for
// the threshold (such a slice holds none of its candidates), is redone by fallback_segment (and flagged in
// seg_flags, for the curious).
// Dynamic LDS: kCandCap composites; rank mode reuses them as sort and exchange buffers.
template <int DT>
__global__ __launch_bounds__(kSelThreads) void select_finalize_cand_kernel(GemvParams g, SelectParams p, int kpad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint64_t* sh_ent = (uint64_t*)smem;
  __shared__ uint32_t sh_hist[kHistBins];
  constexpr int kSliceLanes = 32;   // lanes that copy one slice (a slice of 512 tokens holds about 18 candidates)
  constexpr int kGroups = kSelThreads / kSliceLanes, kInFlight = 8, kRound = kGroups * kInFlight;   // 256 slices per round
  __shared__ uint32_t sh_cnt[kRound], sh_start[kRound];
  __shared__ uint32_t sh_pos[kCandMaxParts + 1];   // start positions of all slices (segments with more than kRound slices)
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];
  __shared__ __attribute__((aligned(8))) uint32_t sh_wmm[2 * kSelWaves];   // smallest and largest key of every wave's entries
  __shared__ uint64_t sh_mm[3];
  __shared__ uint64_t sh_small[kSmallBucket];
  __shared__ uint32_t sh_small_cnt;
  __shared__ uint32_t sh_gave_up;   // slices of this segment whose workgroup never saw the threshold

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int seg = blockIdx.x;
  const uint32_t k = (uint32_t)p.k;
  if (tid == 0) sh_gave_up = 0u;
  sh_hist[2 * tid] = 0;       // (for the first radix pass: cleared here, in front of barriers that are needed anyway)
  sh_hist[2 * tid + 1] = 0;
  __syncthreads();

  // Copy the slices into LDS.  Up to kRound slices: 32 lanes per slice load its first 32 entries (entry 0 carries
  // the slice's count; entries beyond the count are stale memory and ignored), the counts are scanned into
  // start positions, and the entries go to their place: one memory round trip.
  const uint32_t cap = (uint32_t)(p.max_entries < kCandCap ? p.max_entries : kCandCap);
  const uint64_t* lists = p.list + (int64_t)seg * p.list_stride;   // (not read when the entries come from keys or scores)
  const uint64_t* heads = p.cand_head + (int64_t)seg * p.parts * kCandHead;   // entries 0 .. 31 of every slice
  static_assert(kSliceLanes == kCandHead, "one lane per head entry");
  const int sub = tid & (kSliceLanes - 1), grp = tid / kSliceLanes;
  uint32_t n_entries = 0;
  // (where the copy below has every entry in a register on its way, the smallest and the largest key are taken there)
  uint32_t reg_kmin = ~0u, reg_kmax = 0u;
  bool reg_minmax = false;
  if (p.from_keys) {
    // Short segments: no GEMV launch before this one.  The workgroup scores its segment itself (64 row groups
    // of 16 lanes, 16 rows in flight each, canonical order) and every token becomes an entry.
    const int j = tid & 15, rg = tid >> 4;
    const int chunk = seg % g.num_chunks, bh = seg / g.num_chunks;
    const int h = bh % g.num_kv_heads, b = bh / g.num_kv_heads;
    const int64_t chunk_base = g.cluster_ids ? (int64_t)g.cluster_ids[seg] * g.chunk_len : (int64_t)chunk * g.chunk_len;
    float qf[8];
    load_group_query<DT>(g.q, g.q_stride_b, b, h, g.group, j, qf);
    const uint16_t* kbase = (const uint16_t*)g.keys + (int64_t)b * g.key_stride_b + (int64_t)h * g.key_stride_h +
                            chunk_base * g.key_stride_n + 8 * j;
    const int n = (int)p.seg_len;
    constexpr int kRows = 16;   // rows in flight per lane
    for (int base = 0; base < n; base += (kSelThreads / 16) * kRows) {
      u32x4 kv[kRows];
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        const int t = base + rg * kRows + u;
        kv[u] = *(const u32x4*)(kbase + (int64_t)(t < n ? t : n - 1) * g.key_stride_n);
      }
      __builtin_amdgcn_sched_barrier(0);   // all loads go out before the first score is computed
      float mine = 0.0f;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        const float sc = row_score<DT>(qf, kv[u], g.scale);
        if (j == u) mine = sc;
      }
      const int t = base + rg * kRows + j;
      if (j < kRows && t < n) sh_ent[t] = composite(score_key(mine), (uint32_t)t);
    }
    n_entries = (uint32_t)n;
  } else if (p.from_scores) {
    // Segments that fit in LDS whole: the GEMV launch stored plain scores, every one of them becomes an entry.
    const float* sc = p.scores + (int64_t)seg * p.seg_stride;
    const bool vec_ok = (((uintptr_t)sc) & 15u) == 0;
    const int64_t n = p.seg_len;
    for (int64_t first = (int64_t)tid * 4; first < n; first += 4 * kSelThreads) {
      uint32_t keys[4], vm;
      load_keys<4>(sc, first, n, vec_ok, keys, &vm);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (vm >> e & 1u) sh_ent[first + e] = composite(keys[e], (uint32_t)(first + e));
    }
    n_entries = (uint32_t)n;
  } else   if (p.parts <= kRound) {
    for (int s0 = 0; s0 < p.parts; s0 += kRound) {
      uint64_t first[kInFlight];
      uint32_t cnt[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int sl = s0 + u * kGroups + grp;
        first[u] = sl < p.parts ? heads[(int64_t)sl * kCandHead + sub] : 0ull;
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        cnt[u] = ((uint32_t)__shfl((int)(uint32_t)first[u], lane & ~(kSliceLanes - 1), 64) >> 9) & 0x3ffu;
        if (cnt[u] == kSliceGaveUp) {
          cnt[u] = 0u;
          if (sub == 0) atomicAdd(&sh_gave_up, 1u);
        }
        if (sub == 0) sh_cnt[u * kGroups + grp] = cnt[u];
      }
      __syncthreads();
      uint32_t total;
      const uint32_t c = tid < kRound ? sh_cnt[tid] : 0u;
      const uint32_t ex = block_exclusive_scan(c, sh_wtot, &total);
      if (tid < kRound) sh_start[tid] = n_entries + ex;
      __syncthreads();
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int sl = s0 + u * kGroups + grp;
        const uint32_t start = sh_start[u * kGroups + grp];
        const uint32_t idx0 = (uint32_t)sl * (uint32_t)p.part_len;
        if ((uint32_t)sub < cnt[u] && start + sub < cap) {
          sh_ent[start + sub] = (first[u] & 0xffffffff00000000ull) | (uint32_t)~(idx0 + ((uint32_t)first[u] & 0x1ffu));
          reg_kmin = min(reg_kmin, (uint32_t)(first[u] >> 32));
          reg_kmax = max(reg_kmax, (uint32_t)(first[u] >> 32));
        }
        for (uint32_t j = kSliceLanes + sub; j < cnt[u] && start + j < cap; j += kSliceLanes) {   // rare: a slice with more than 32 candidates
          const uint64_t w = lists[(int64_t)sl * p.part_len + j];
          sh_ent[start + j] = (w & 0xffffffff00000000ull) | (uint32_t)~(idx0 + ((uint32_t)w & 0x1ffu));
          reg_kmin = min(reg_kmin, (uint32_t)(w >> 32));
          reg_kmax = max(reg_kmax, (uint32_t)(w >> 32));
        }
      }
      n_entries += total;
    }
    reg_minmax = true;
  } else {
    // many slices: all counts first (one round trip), one scan, then the entries with no barrier in between
    uint32_t c4[4], sum = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int sl = 4 * tid + q;
      c4[q] = sl < p.parts ? ((uint32_t)heads[(int64_t)sl * kCandHead] >> 9) & 0x3ffu : 0u;
      if (c4[q] == kSliceGaveUp) {
        c4[q] = 0u;
        atomicAdd(&sh_gave_up, 1u);
      }
      sum += c4[q];
    }
    uint32_t total;
    uint32_t running = block_exclusive_scan(sum, sh_wtot, &total);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      sh_pos[4 * tid + q] = running;
      running += c4[q];
    }
    if (tid == kSelThreads - 1) sh_pos[kCandMaxParts] = total;
    n_entries = total;
    __syncthreads();
    // long segments are sparse in candidates per slice: 8 lanes per slice, 1024 slices per trip
    constexpr int kLanes2 = 8, kGroups2 = kSelThreads / kLanes2, kRound2 = kGroups2 * kInFlight;
    const int sub2 = tid & (kLanes2 - 1), grp2 = tid / kLanes2;
    for (int s0 = 0; s0 < p.parts; s0 += kRound2) {
      uint64_t w[kInFlight];
      uint32_t start[kInFlight], cnt[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int sl = s0 + u * kGroups2 + grp2;
        start[u] = sl < p.parts ? sh_pos[sl] : 0u;
        cnt[u] = sl < p.parts ? sh_pos[sl + 1] - start[u] : 0u;
        w[u] = (uint32_t)sub2 < cnt[u] ? heads[(int64_t)sl * kCandHead + sub2] : 0ull;
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int sl = s0 + u * kGroups2 + grp2;
        const uint32_t idx0 = (uint32_t)sl * (uint32_t)p.part_len;
        if ((uint32_t)sub2 < cnt[u] && start[u] + sub2 < cap)
          sh_ent[start[u] + sub2] = (w[u] & 0xffffffff00000000ull) | (uint32_t)~(idx0 + ((uint32_t)w[u] & 0x1ffu));
        for (uint32_t j = kLanes2 + sub2; j < cnt[u] && start[u] + j < cap; j += kLanes2) {
          const uint64_t x = j < (uint32_t)kCandHead ? heads[(int64_t)sl * kCandHead + j] : lists[(int64_t)sl * p.part_len + j];
          sh_ent[start[u] + j] = (x & 0xffffffff00000000ull) | (uint32_t)~(idx0 + ((uint32_t)x & 0x1ffu));
        }
      }
    }
  }
  const bool whole = p.from_keys || p.from_scores;   // the entries are the whole segment, not candidate slices
  // (every add to sh_gave_up lies in front of a barrier of the copy)
  const uint32_t n_gave_up = sh_gave_up;
  const bool redo = !whole && (n_entries < k || n_entries > cap || n_gave_up != 0u);
  if (tid == 0) {
    sh_small_cnt = 0;
  }
  if (!whole) {
    if (tid == 0) p.seg_flags[seg] = (redo ? 1u : 0u) | (n_gave_up << 8);
    // the threshold and the arrival flags are spent: a replay of the same launches (a captured graph) must not
    // take them for its own
    if (tid >= 64 && tid < 128) p.sample_flags[(int64_t)seg * 64 + (tid - 64)] = 0u;
    if (tid == 0) p.tau_words[2 * seg] = 0ull;
  }
  if (redo) {
    if (p.redo_hist) {
      // the launch behind this one redoes the segment (redo_segments_kernel): its histogram and arrival count start at zero
      p.redo_hist[(int64_t)seg * kHistBins + 2 * tid] = 0u;
      p.redo_hist[(int64_t)seg * kHistBins + 2 * tid + 1] = 0u;
      if (tid < 2 * kRedoPhasesMax) p.redo_queue[tid] = 0u;   // (the item counters of that launch: every flagged segment clears them)
      return;
    }
    __syncthreads();
    fallback_segment<DT>(g, p, seg, kpad, sh_ent, sh_hist, sh_pos, sh_wtot, sh_res, sh_mm);
    return;
  }
  if (whole && p.out_idx != nullptr && p.union_idx == nullptr && n_entries <= 2u * kSelThreads) {
    // a short segment whose caller wants rank order only: sorting all of it is quicker than selecting first
    uint32_t npad = 64;
    while (npad < n_entries) npad <<= 1;
    for (uint32_t i = n_entries + tid; i < npad; i += kSelThreads) sh_ent[i] = 0;   // pad: below every real composite
    __syncthreads();
    sort_lds_desc(sh_ent, sh_ent + npad, (int)npad);   // (measured quicker here than the bucketed rank sort)
    write_rank_outputs(sh_ent, p, seg);
    return;
  }
  __syncthreads();

  // The passes over the entries (tid, tid + 1024, ...) are rolled loops over the LDS copy: the kernel runs a few workgroups,
  // every line of its code is fetched cold, and an unrolled pass for the 16 entries per thread that the capacity allows
  // costs that fetch whether or not the list reaches them.
  uint32_t kmin = reg_kmin, kmax = reg_kmax;   // smallest and largest key among the entries
  if (!reg_minmax) {
#pragma unroll 1
    for (uint32_t v = tid; v < n_entries; v += kSelThreads) {
      const uint32_t key = (uint32_t)(sh_ent[v] >> 32);
      kmin = min(kmin, key);
      kmax = max(kmax, key);
    }
  }

  uint64_t threshold = 0;   // selected: composite >= threshold
  if (n_entries > k) {
    // common prefix of all keys: the passes start below it (all keys equal: they start at the index bits)
    // (the waves' extremes through LDS, one lane per wave, and across sixteen lanes: no atomics)
    kmin = wave_min_in_last_lane(kmin);
    kmax = wave_max_in_last_lane(kmax);
    if (lane == 63) { sh_wmm[2 * (tid >> 6)] = kmin; sh_wmm[2 * (tid >> 6) + 1] = kmax; }
    __syncthreads();
    {
      static_assert(kSelWaves == 16, "sixteen lanes hold the waves' extremes");
      const uint2 mm = *(const uint2*)&sh_wmm[2 * (lane & 15)];
      kmin = mm.x;  kmax = mm.y;
      kmin = min(kmin, lane_xor<1>(kmin));   kmax = max(kmax, lane_xor<1>(kmax));
      kmin = min(kmin, lane_xor<2>(kmin));   kmax = max(kmax, lane_xor<2>(kmax));
      kmin = min(kmin, lane_xor<4>(kmin));   kmax = max(kmax, lane_xor<4>(kmax));
      kmin = min(kmin, lane_xor<8>(kmin));   kmax = max(kmax, lane_xor<8>(kmax));
    }
    // Radix passes on the composites relative to the smallest key: their leading bits are zero down to the
    // width of the key range, and the 11 bits below spread the candidates evenly (shared bits of the float
    // keys themselves say little once the scores straddle a power of two).
    const uint64_t base = (uint64_t)kmin << 32;
    int fixed = kmin == kmax ? 32 : __builtin_clz(kmax - kmin);
    uint64_t prefix = 0ull;
    uint32_t need = k;
    bool done = false, first_pass = true;
    while (!done) {
      const int bits = (64 - fixed) >= kHistBits ? kHistBits : (64 - fixed);
      const int shift = 64 - fixed - bits;
      if (!first_pass) {
        __syncthreads();
        sh_hist[2 * tid] = 0;
        sh_hist[2 * tid + 1] = 0;
        __syncthreads();
      }
      first_pass = false;
#pragma unroll 1
      for (uint32_t v = tid; v < n_entries; v += kSelThreads) {
        const uint64_t c = sh_ent[v] - base;
        if (fixed == 0 || (c >> (64 - fixed)) == prefix) atomicAdd(&sh_hist[(uint32_t)(c >> shift) & ((1u << bits) - 1u)], 1u);
      }
      __syncthreads();
      find_threshold_bin_1024(sh_hist, need, sh_wtot, sh_res);
      const uint32_t d = sh_res[0], gt = sh_res[1], cnt = sh_res[2];
      need -= gt;
      prefix = (prefix << bits) | d;
      fixed += bits;
      if (cnt == need || fixed == 64) {
        threshold = fixed == 64 ? prefix : (prefix << (64 - fixed));
        done = true;
      } else if (cnt <= (uint32_t)kSmallBucket) {
        // few entries left in the threshold bucket: every wave ranks them and picks the need-th largest
#pragma unroll 1
        for (uint32_t v = tid; v < n_entries; v += kSelThreads) {
          const uint64_t c = sh_ent[v] - base;
          if ((c >> (64 - fixed)) == prefix) sh_small[atomicAdd(&sh_small_cnt, 1u)] = c;
        }
        __syncthreads();
        const uint64_t e = (uint32_t)lane < cnt ? sh_small[lane] : 0ull;
        uint32_t greater = 0;
        for (uint32_t j = 0; j < cnt; ++j) greater += sh_small[j] > e ? 1u : 0u;
        const uint64_t hit = __ballot((uint32_t)lane < cnt && greater == need - 1u);
        threshold = __shfl(e, (int)__builtin_ctzll(hit), 64);
        done = true;
      }
    }
    threshold += base;   // back from the relative composites
  }

  // Walk in index order: thread t takes the run of `per` consecutive entries starting at t*per.
  const bool want_rank = p.out_idx != nullptr;
  const bool want_union = p.union_idx != nullptr;
  const int64_t n = p.seg_len;
  const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
  const uint32_t hi = (uint32_t)(n - p.local > lo ? n - p.local : lo);
  const uint32_t per = (n_entries + kSelThreads - 1) / kSelThreads;   // at most kCandPerThread
  uint32_t sel_mask = 0, mid_mask = 0;
#pragma unroll 1
  for (uint32_t i = 0; i < per; ++i) {
    const uint32_t v = (uint32_t)tid * per + i;
    if (v < n_entries) {
      const uint64_t c = sh_ent[v];
      const bool sel = c >= threshold;
      const uint32_t idx = ~(uint32_t)c;
      sel_mask |= (sel ? 1u : 0u) << i;
      mid_mask |= (sel && idx >= lo && idx < hi ? 1u : 0u) << i;
    }
  }
  // one scan for both counts (each total is at most 16384)
  uint32_t totals;
  const uint32_t ex = block_exclusive_scan(((uint32_t)__builtin_popcount(sel_mask) << 16) | (uint32_t)__builtin_popcount(mid_mask), sh_wtot, &totals);
  if (want_union) {
    int32_t* uo = p.union_idx + (int64_t)seg * (p.k + p.sink + p.local);
    uint32_t pos = lo + (ex & 0xffffu);
#pragma unroll 1
    for (uint32_t i = 0; i < per; ++i)
      if (mid_mask >> i & 1u) uo[pos++] = (int32_t)~(uint32_t)sh_ent[(uint32_t)tid * per + i];
    write_union_edges(uo, p, seg, lo, hi, totals & 0xffffu);
  }
  if (!want_rank) return;
  uint64_t* sh_sort = sh_ent;
  uint64_t* sh_xchg = sh_ent + kpad;
  uint64_t run[kCandPerThread];   // the selected of this thread's run, in registers: the buffer is about to be overwritten
#pragma unroll
  for (int i = 0; i < kCandPerThread; ++i) run[i] = (sel_mask >> i & 1u) ? sh_ent[(uint32_t)tid * per + i] : 0ull;
  __syncthreads();
  {
    uint32_t pos = ex >> 16;
#pragma unroll
    for (int i = 0; i < kCandPerThread; ++i)
      if (sel_mask >> i & 1u) sh_sort[pos++] = run[i];
    for (int i = (int)k + tid; i < kpad; i += kSelThreads) sh_sort[i] = 0;  // pad: below every real composite
  }
  __syncthreads();
  rank_sort_desc(sh_sort, sh_xchg, k, kpad, sh_hist, sh_pos, sh_wtot, sh_mm);   // (the slice positions are spent)
  write_rank_outputs(sh_sort, p, seg);
}

// ---- redo of flagged long segments, in a launch of its own --------------------------------------------------

// (redo_segments_kernel, below, says how the work is shared.)
constexpr int kRedoChunk = 4096;        // tokens of an item of the scoring phase
constexpr int kRedoMaxFlagged = 2048;   // segments of a call (the list of the flagged ones is kept in LDS)
constexpr int kRedoBucketCap = 16384;   // composites of the threshold bucket held in LDS (128 KB) while the cut inside it is searched

// U vectors of four stored keys per lane: vector u holds the keys of tokens base + u * stride + first .. + 3.  A block
// that lies inside [.., end) whole is loaded without a branch per vector (all U loads are in flight together: a pass over
// the stored keys is bound by their latency first); the last block of a range is guarded, key 0 and a clear bit in vm
// for a token at or beyond `end`.
template <int U>
__device__ __forceinline__ void load_stored_keys(const uint32_t* sk, int64_t base, int first, int stride, int64_t end, bool vec_ok,
                                                 uint32_t (&keys)[U][4], uint32_t (&vm)[U]) {
  if (vec_ok && base + (int64_t)stride * U <= end) {   // (uniform)
    u32x4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = *(const u32x4*)(sk + base + stride * u + first);
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < 4; ++e) keys[u][e] = x[u][e];
      vm[u] = 0xfu;
    }
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      vm[u] = 0u;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int64_t i = base + stride * u + first + e;
        const bool ok = i < end;
        keys[u][e] = ok ? sk[i] : 0u;
        vm[u] |= (ok ? 1u : 0u) << e;
      }
    }
  }
}

// How redo_wave_walk tells which of the ties (tokens whose top `fixed` key bits equal `prefix`) are selected.
enum : int {
  kTiesAll = 0,        // all of them
  kTiesByComposite,    // those whose composite (key, ~index) is at least `cut`
  kTiesByRank          // the first `need` of them in index order
};

// One walk of this wave over tokens [w0, w1) of the stored keys (w0 a multiple of 256; all 64 lanes).  The selected
// tokens are those whose top `fixed` key bits exceed `prefix`, and of the ties those that `mode` says; run_tie = ties
// in front of w0 (kTiesByRank).  Blocks of 256 tokens without a selected one (most, where k is small against the
// segment) cost a compare per token and a few scalar instructions.
//   WRITE = false: returns how many selected ties lie in [lo, hi) - for the one wave in whose range the cut among the
//                  ties falls (kTiesByRank), whose count of them cannot be had from totals.
//   WRITE = true:  writes the ids of the selected tokens in [lo, hi) to uo[run_mid ...] in index order, and (sort != 0)
//                  the composites of all selected tokens to sort[run_sel ...] (memory that another workgroup reads).
// U: vector loads in flight per lane.
template <bool WRITE, int U>
__device__ __forceinline__ uint32_t redo_wave_walk(const uint32_t* sk, bool vec_ok, int64_t w0, int64_t w1, uint32_t prefix, int fixed,
                                                   int mode, uint64_t cut, uint32_t need, uint32_t lo, uint32_t hi, uint32_t run_tie,
                                                   uint32_t run_mid, uint32_t run_sel, int32_t* uo, uint64_t* sort, uint32_t sort_cap) {
  int lane = threadIdx.x & 63;
  asm volatile("" : "+v"(lane));   // (addresses computed here, at every call: see redo_segments_kernel)
  const int shift = 32 - fixed;   // (0 .. 21)
  uint32_t tie_mid_selected = 0;   // (uniform)
  for (int64_t base = w0; base < w1; base += 256 * U) {
    uint32_t keys[U][4], vm[U];
    load_stored_keys<U>(sk, base, 4 * lane, 256, w1, vec_ok, keys, vm);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t first = (uint32_t)(base + 256 * u) + 4u * (uint32_t)lane;
      uint32_t above = 0, tie = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t top = keys[u][e] >> shift;
        const bool ok = vm[u] >> e & 1u;
        above |= (ok && top > prefix ? 1u : 0u) << e;
        tie |= (ok && top == prefix ? 1u : 0u) << e;
      }
      if (__ballot((above | tie) != 0u) == 0ull) continue;   // (uniform) nothing to select among these 256
      uint32_t sel = above | tie;
      if (mode == kTiesByComposite) {   // (uniform)
        sel = above;
#pragma unroll
        for (int e = 0; e < 4; ++e) sel |= ((tie >> e & 1u) && composite(keys[u][e], first + e) >= cut ? 1u : 0u) << e;
      } else if (mode == kTiesByRank) {
        const uint32_t mine = (uint32_t)__builtin_popcount(tie);
        const uint32_t inc = wave_inclusive_scan(mine);
        uint32_t r = run_tie + inc - mine;
        run_tie += (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
        sel = above;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (tie >> e & 1u) {
            sel |= (r < need ? 1u : 0u) << e;
            ++r;
          }
      }
      uint32_t mid = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) mid |= ((sel >> e & 1u) && first + e - lo < hi - lo ? 1u : 0u) << e;   // (lo <= hi)
      if (!WRITE) {
        tie_mid_selected += (uint32_t)__popcll(__ballot((mid & tie & 1u) != 0u)) + (uint32_t)__popcll(__ballot((mid & tie & 2u) != 0u)) +
                            (uint32_t)__popcll(__ballot((mid & tie & 4u) != 0u)) + (uint32_t)__popcll(__ballot((mid & tie & 8u) != 0u));
      } else {
        const uint32_t packed = ((uint32_t)__builtin_popcount(sel) << 16) | (uint32_t)__builtin_popcount(mid);
        const uint32_t inc = wave_inclusive_scan(packed);   // (at most 256 of either per wave and block)
        const uint32_t ex = inc - packed;
        uint32_t pos_sel = run_sel + (ex >> 16), pos_mid = run_mid + (ex & 0xffffu);
        const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
        run_sel += tot >> 16;
        run_mid += tot & 0xffffu;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (sort && (sel >> e & 1u)) {
            if (pos_sel < sort_cap) __hip_atomic_store(sort + pos_sel, composite(keys[u][e], first + e), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ++pos_sel;
          }
          if (uo && (mid >> e & 1u)) uo[pos_mid++] = (int32_t)(first + e);
        }
      }
    }
  }
  return tie_mid_selected;
}

// Exact selection for segment `seg` from its stored keys (redo_segments_kernel stores the keys of the scores, not the
// scores); sh_hist holds the counts of their top 11 bits.  Same result as fallback_select_from_scores, in two passes
// over the keys and few barriers.  Every wave takes a contiguous sixteenth of the segment.  Pass one counts, per wave,
// the tokens above the threshold bucket and its members (all, and those between the sink range and the local window),
// and gathers the members' composites in LDS, where the cut inside the bucket is then searched (radix passes over the
// composites: ties in the key fall to the smaller index, as everywhere); the waves' totals are summed once; pass two
// writes every wave's part in index order.  A bucket with more members than the LDS holds is narrowed by counting
// passes over the keys first; members that all carry one key (narrowing cannot help) are told apart by their rank
// among themselves in pass two instead.  Writes the ids of the selected tokens between the sink range and the local
// window to their place in the union list and returns how many they are (the ends of the list are the caller's), and
// (RANK) the composites of all selected tokens to `selection`, in memory, in index order.  The counts are kept on the scalar side (a compare per token gives a lane mask,
// its population is a scalar instruction): one CU has a million tokens to get through.
// Every thread of the block must call it.  smem: kRedoBucketCap composites.
template <int DT, bool RANK>
__device__ __forceinline__ uint32_t redo_select_from_scores(const GemvParams& g, const SelectParams& p, int seg, uint64_t* selection,
                                                            unsigned char* smem, uint32_t* sh_hist, uint32_t* sh_off, uint32_t* sh_wtot,
                                                            uint32_t* sh_res) {
  uint64_t* sh_buck = (uint64_t*)smem;
  int tid = threadIdx.x;
  // (Called from inside the loop of a long kernel: what follows is computed here, each time, from a thread number that
  // the compiler cannot trace - hoisted to the top of the kernel these values cost it more registers than it has.)
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = tid >> 6;
  const uint32_t k = (uint32_t)p.k;
  const int64_t n = p.seg_len;
  const uint32_t* sk = (const uint32_t*)(g.scores + (int64_t)seg * p.seg_stride);
  const bool vec_ok = (((uintptr_t)sk) & 15u) == 0;

  // the k-th largest key: `prefix` = its top `fixed` bits, `need` = how many of the `cnt` keys with these bits belong
  // to the top k
  find_threshold_bin_1024(sh_hist, k, sh_wtot, sh_res);
  uint32_t prefix = sh_res[0], need = k - sh_res[1], cnt = sh_res[2];
  int fixed = kHistBits;
  while (cnt != need && cnt > (uint32_t)kRedoBucketCap && fixed < 32) {   // (rare) narrow the bucket: count its members' next bits
    const int bits = (32 - fixed) >= kHistBits ? kHistBits : (32 - fixed);
    const int shift = 32 - fixed - bits;
    __syncthreads();
    sh_hist[2 * tid] = 0;
    sh_hist[2 * tid + 1] = 0;
    __syncthreads();
    constexpr int U = 4;
    for (int64_t base = 0; base < n; base += 4 * kSelThreads * U) {
      uint32_t keys[U][4], vm[U];
      load_stored_keys<U>(sk, base, 4 * tid, 4 * kSelThreads, n, vec_ok, keys, vm);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if ((vm[u] >> e & 1u) && (keys[u][e] >> (32 - fixed)) == prefix) atomicAdd(&sh_hist[(keys[u][e] >> shift) & ((1u << bits) - 1u)], 1u);
    }
    __syncthreads();
    find_threshold_bin_1024(sh_hist, need, sh_wtot, sh_res);
    need -= sh_res[1];
    prefix = (prefix << bits) | sh_res[0];
    cnt = sh_res[2];
    fixed += bits;
  }
  const bool gather = cnt != need && cnt <= (uint32_t)kRedoBucketCap;
  const int mode = cnt == need ? kTiesAll : (gather ? kTiesByComposite : kTiesByRank);

  constexpr bool want_rank = RANK;   // (p.out_idx set)
  const bool want_union = p.union_idx != nullptr;
  const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
  const uint32_t hi = (uint32_t)(n - p.local > lo ? n - p.local : lo);
  int32_t* uo = want_union ? p.union_idx + (int64_t)seg * (p.k + p.sink + p.local) : nullptr;

  // this wave's sixteenth (a multiple of 256 tokens: the vector loads stay aligned)
  const int64_t per_wave = (n + 256 * kSelWaves - 1) / (256 * kSelWaves) * 256;
  const int64_t w0 = (int64_t)wave * per_wave < n ? (int64_t)wave * per_wave : n;
  const int64_t w1 = w0 + per_wave < n ? w0 + per_wave : n;

  // pass one
  if (tid == 0) sh_res[3] = 0u;   // members gathered so far
  if (tid < 6 * kSelWaves + 1) sh_off[tid] = 0u;   // per wave: above, above in [lo, hi), ties, ties in [lo, hi), selected ties, selected ties in [lo, hi); then one word for the wave with the cut
  __syncthreads();
  uint32_t c_above = 0, c_above_mid = 0, c_tie = 0, c_tie_mid = 0;   // (uniform: totals of the wave)
  {
    const int shift = 32 - fixed;
    constexpr int U = 4;   // (what the registers allow)
    for (int64_t base = w0; base < w1; base += 256 * U) {
      uint32_t keys[U][4], vm[U];
      load_stored_keys<U>(sk, base, 4 * lane, 256, w1, vec_ok, keys, vm);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t block = (uint32_t)(base + 256 * u);
        // the block against [lo, hi): inside whole (nearly always), outside whole, or cut by an end of it
        const bool all_mid = block >= lo && block + 256u <= hi, some_mid = block < hi && block + 256u > lo;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t top = keys[u][e] >> shift;
          const bool ok = vm[u] >> e & 1u;
          const bool above = ok && top > prefix, tie = ok && top == prefix;
          const unsigned long long ma = __ballot(above), mt = __ballot(tie);
          c_above += (uint32_t)__popcll(ma);
          c_tie += (uint32_t)__popcll(mt);
          if (all_mid) {
            c_above_mid += (uint32_t)__popcll(ma);
            c_tie_mid += (uint32_t)__popcll(mt);
          } else if (some_mid) {
            const bool in_mid = block + 4u * (uint32_t)lane + e - lo < hi - lo;
            c_above_mid += (uint32_t)__popcll(__ballot(above && in_mid));
            c_tie_mid += (uint32_t)__popcll(__ballot(tie && in_mid));
          }
          if (gather && mt != 0ull) {   // (uniform) one reservation per wave
            uint32_t first = 0;
            if (lane == 0) first = atomicAdd(&sh_res[3], (uint32_t)__popcll(mt));
            first = (uint32_t)__builtin_amdgcn_readfirstlane((int)first);
            if (tie) sh_buck[first + (uint32_t)__popcll(mt & ((1ull << lane) - 1ull))] = composite(keys[u][e], block + 4u * (uint32_t)lane + e);
          }
        }
      }
    }
  }
  if (lane == 0) {
    sh_off[6 * wave] = c_above;
    sh_off[6 * wave + 1] = c_above_mid;
    sh_off[6 * wave + 2] = c_tie;
    sh_off[6 * wave + 3] = c_tie_mid;
  }
  __syncthreads();

  // the cut inside the bucket: the need-th largest of the gathered composites
  uint64_t cut = 0;
  if (gather) {
    uint64_t cprefix = prefix;   // top `cfixed` bits of the composite
    int cfixed = fixed;
    uint32_t left = need, among = cnt;
    while (among != left && cfixed < 64) {
      const int bits = (64 - cfixed) >= kHistBits ? kHistBits : (64 - cfixed);
      const int shift = 64 - cfixed - bits;
      sh_hist[2 * tid] = 0;
      sh_hist[2 * tid + 1] = 0;
      __syncthreads();
      for (uint32_t i = tid; i < cnt; i += kSelThreads) {
        const uint64_t c = sh_buck[i];
        if ((c >> (64 - cfixed)) == cprefix) atomicAdd(&sh_hist[(uint32_t)(c >> shift) & ((1u << bits) - 1u)], 1u);
      }
      __syncthreads();
      find_threshold_bin_1024(sh_hist, left, sh_wtot, sh_res);
      left -= sh_res[1];
      cprefix = (cprefix << bits) | sh_res[0];
      among = sh_res[2];
      cfixed += bits;
    }
    cut = cfixed == 64 ? cprefix : cprefix << (64 - cfixed);   // every composite with these leading bits is taken
    // the selected members of every wave's range
    for (uint32_t i = tid; i < cnt; i += kSelThreads) {
      const uint64_t c = sh_buck[i];
      if (c >= cut) {
        const uint32_t idx = ~(uint32_t)c;
        const uint32_t w = idx / (uint32_t)per_wave;
        atomicAdd(&sh_off[6 * w + 4], 1u);
        if (idx - lo < hi - lo) atomicAdd(&sh_off[6 * w + 5], 1u);
      }
    }
    __syncthreads();
  }
  // kTiesByRank: the wave in whose range the cut among the ties falls (at most one) counts its selected ties in [lo, hi) itself
  uint32_t tie_before = 0;
  for (int v = 0; v < wave; ++v) tie_before += sh_off[6 * v + 2];
  if (mode == kTiesByRank) {
    const uint32_t my_ties = sh_off[6 * wave + 2];
    if (tie_before < need && tie_before + my_ties > need) {
      const uint32_t c = redo_wave_walk<false, 2>(sk, vec_ok, w0, w1, prefix, fixed, mode, 0ull, need, lo, hi, tie_before, 0u, 0u, nullptr,
                                                  nullptr, 0u);
      if (lane == 0) sh_off[6 * kSelWaves] = c;
    }
  }
  __syncthreads();
  uint32_t mid_before = 0, sel_before = 0, mid_total = 0, run = 0;
  for (int v = 0; v < kSelWaves; ++v) {
    const uint32_t ties = sh_off[6 * v + 2];
    uint32_t taken, taken_mid;
    if (mode == kTiesAll) {
      taken = ties;
      taken_mid = sh_off[6 * v + 3];
    } else if (mode == kTiesByComposite) {
      taken = sh_off[6 * v + 4];
      taken_mid = sh_off[6 * v + 5];
    } else {
      taken = run >= need ? 0u : (need - run < ties ? need - run : ties);
      taken_mid = taken == ties ? sh_off[6 * v + 3] : (taken == 0u ? 0u : sh_off[6 * kSelWaves]);
    }
    run += ties;
    const uint32_t m = sh_off[6 * v + 1] + taken_mid, s = sh_off[6 * v] + taken;
    if (v < wave) {
      mid_before += m;
      sel_before += s;
    }
    mid_total += m;
  }
  // pass two
  redo_wave_walk<true, 4>(sk, vec_ok, w0, w1, prefix, fixed, mode, cut, need, lo, hi, tie_before, lo + mid_before, sel_before, uo,
                          want_rank ? selection : nullptr, k);
  return mid_total;
}

// The phases of redo_segments_kernel and the words of a segment's record in memory.
enum : int {
  kRedoScore = 0,   // per chunk of 4096 tokens: keys of the scores stored, top key bits counted
  kRedoCount,       // per batch of 32768 tokens: tokens above the threshold bucket counted, the bucket's members gathered
  kRedoCut,         // per segment: the cut inside the bucket, every batch's place in the outputs
  kRedoWrite,       // per batch: the selected tokens written
  kRedoFinish,      // per segment, rank-ordered output only: the rank order
  kRedoPhases
};
enum : int { kRecPrefix = 0, kRecMode, kRecCutLo, kRecCutHi, kRecMidTotal, kRecWords = 16 };   // (the first four: one 16-byte load)
enum : int {
  kRedoTakeBucket = 0,   // the whole bucket belongs to the top k
  kRedoCutBucket,        // the bucket's members are gathered and the cut among them searched
  kRedoAlone             // (a bucket beyond the LDS, a segment of more than 2048 batches) one workgroup selects: redo_select_from_scores
};
constexpr int kRedoBatch = 32 * kSelThreads;   // tokens of a batch: 32 consecutive ones per thread
constexpr int kRedoMaxBatches = kHistBins;     // batches of a segment whose counts one workgroup sums in LDS
constexpr int kRedoWaitSpins = 1 << 22;        // about a second

// The bucket of the k-th largest key from the segment's histogram in memory (all 1024 threads; sh_hist is overwritten):
// *prefix = its 11 bits, *need = how many of its *cnt members belong to the top k; returns how the segment goes on.
__device__ __forceinline__ int redo_threshold(const uint32_t* gh, uint32_t k, uint32_t batches_per_seg, uint32_t* sh_hist, uint32_t* sh_wtot,
                                              uint32_t* sh_res, uint32_t* prefix, uint32_t* need, uint32_t* cnt) {
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));   // (addresses computed here, at every call: see redo_segments_kernel)
  __syncthreads();
  sh_hist[2 * tid] = __hip_atomic_load(gh + 2 * tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  sh_hist[2 * tid + 1] = __hip_atomic_load(gh + 2 * tid + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  find_threshold_bin_1024(sh_hist, k, sh_wtot, sh_res);
  *prefix = sh_res[0];
  *need = k - sh_res[1];
  *cnt = sh_res[2];
  return *cnt == *need ? kRedoTakeBucket
                       : (*cnt <= (uint32_t)kRedoBucketCap && batches_per_seg <= (uint32_t)kRedoMaxBatches ? kRedoCutBucket : kRedoAlone);
}

// This thread's 32 consecutive stored keys from token `first` on (a multiple of 32); key 0 at and beyond `n`.
__device__ __forceinline__ void redo_load_run(const uint32_t* sk, uint32_t first, int64_t n, uint32_t (&keys)[32]) {
  if ((((uintptr_t)sk) & 15u) == 0 && (int64_t)first + 32 <= n) {
    u32x4 x[8];
#pragma unroll
    for (int v = 0; v < 8; ++v) x[v] = *(const u32x4*)(sk + first + 4 * v);
#pragma unroll
    for (int v = 0; v < 8; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) keys[4 * v + e] = x[v][e];
  } else {
#pragma unroll
    for (int e = 0; e < 32; ++e) keys[e] = (int64_t)first + e < n ? sk[first + e] : 0u;
  }
}

// acc = 2 * acc + (a > b), and the same for a == b: two instructions per token build a mask of 32 tokens in the reverse
// order of their bits.  (Written out: left to itself the compiler ors in one constant per bit position and keeps all of
// them in registers across the kernel's loops, more registers than are left.)
__device__ __forceinline__ void shift_in_gt(uint32_t& acc, uint32_t a, uint32_t b) {
  asm("v_cmp_gt_u32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(acc) : "v"(a), "v"(b) : "vcc");
}
__device__ __forceinline__ void shift_in_eq(uint32_t& acc, uint32_t a, uint32_t b) {
  asm("v_cmp_eq_u32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(acc) : "v"(a), "v"(b) : "vcc");
}

// Bits [a, b) of a 32-bit word, for 0 <= a, b <= 32 (none when b <= a).
__device__ __forceinline__ uint32_t bit_range(uint32_t a, uint32_t b) {
  const uint32_t below_b = b >= 32u ? ~0u : (1u << b) - 1u, below_a = a >= 32u ? ~0u : (1u << a) - 1u;
  return b > a ? below_b & ~below_a : 0u;
}

// Launched behind select_finalize_cand_kernel on the candidate route, one workgroup per CU.  Every workgroup reads the
// segment flags; when none is set (all but always) it leaves at once.  Otherwise the flagged segments are redone from
// the keys, exactly, by all workgroups together, in phases.  The work of a phase is a list of items - a run of tokens,
// or a segment - that the workgroups draw from a counter in memory; what an item leaves for a later phase goes out as
// stores performed at the point of coherence, and when a workgroup finds the counter exhausted it waits until its
// stores have completed and adds the number of its items to the phase's done count.  Then it waits until that count is
// complete: every item it waits for has been drawn, so it is in the hands of a workgroup that is running - no
// workgroup waits for one that has not started, and one workgroup alone would get through all phases by itself.  (The
// wait is bounded all the same; a workgroup whose wait runs out leaves - it holds no item then, and the others finish
// without it.)
//   score   per chunk of 4096 tokens: the keys of the scores stored (canonical order), their top 11 bits counted into
//           the segment's histogram in memory
//   count   per batch of 32768 tokens, 32 consecutive ones per thread: the bucket of the k-th key from the histogram (a
//           bucket that the top k take whole, or whose members fit the LDS, goes on here; any other segment is left to
//           one workgroup in `cut`, redo_select_from_scores); tokens above the bucket counted (all / between the sink
//           range and the local window), the members' composites written to the batch's part of the segment's list
//   cut     per segment: the need-th largest of the members by radix passes in LDS (ties in the key fall to the
//           smaller index, as everywhere), then every batch's first place in the union list and in the selection
//   write   per batch: ids of the selected tokens to their place in the union list (the batch at the front of a segment
//           also writes sink range, local window and count), composites to the selection
//   finish  per segment, rank-ordered output only: the selection sorted and written
// All 64 segments of 131072 tokens flagged: the step costs a bit over twice what it costs otherwise (the keys are read
// a second time at the rate of the first, and little else), where one workgroup per segment took 14 times as long.
template <int DT, bool RANK>
__global__ __launch_bounds__(kSelThreads) void redo_segments_kernel(GemvParams g, SelectParams p, int kpad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // the bucket's composites, then (rank mode) 2 * kpad composites
  __shared__ uint32_t sh_hist[kHistBins], sh_off[kHistBins];
  __shared__ uint32_t sh_wtot[kSelWaves], sh_res[4];
  __shared__ uint64_t sh_mm[3];
  __shared__ uint16_t sh_flagged[kRedoMaxFlagged];
  __shared__ uint32_t sh_item;
  const int wave = threadIdx.x >> 6;
  uint32_t n_flagged = 0;
  {
    // the flagged segments, in order (every workgroup builds the same list)
    const int tid = threadIdx.x, lane = tid & 63;
    for (int s0 = 0; s0 < p.num_segments; s0 += kSelThreads) {
      const int s = s0 + tid;
      const bool flagged = s < p.num_segments && (p.seg_flags[s] & 1u) != 0u;
      const unsigned long long m = __ballot(flagged);
      if (lane == 0) sh_wtot[wave] = (uint32_t)__popcll(m);
      __syncthreads();
      uint32_t before = n_flagged, all = 0;
      for (int w = 0; w < kSelWaves; ++w) {
        const uint32_t c = sh_wtot[w];
        before += w < wave ? c : 0u;
        all += c;
      }
      if (flagged) sh_flagged[before + (uint32_t)__popcll(m & ((1ull << lane) - 1ull))] = (uint16_t)s;
      n_flagged += all;
      __syncthreads();
    }
  }
  if (n_flagged == 0u) return;   // the ordinary case

  const uint32_t k = (uint32_t)p.k;
  const int64_t n = p.seg_len;
  const uint32_t chunks_per_seg = (uint32_t)((n + kRedoChunk - 1) / kRedoChunk);
  const uint32_t batches_per_seg = (uint32_t)((n + kRedoBatch - 1) / kRedoBatch);
  const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
  const uint32_t hi = (uint32_t)(n - p.local > lo ? n - p.local : lo);
  const bool want_union = p.union_idx != nullptr;
  constexpr int kTopShift = 32 - kHistBits;

  for (int phase = 0; phase < (RANK ? kRedoPhases : kRedoFinish); ++phase) {
    const uint32_t per_seg = phase == kRedoScore ? chunks_per_seg : (phase == kRedoCount || phase == kRedoWrite ? batches_per_seg : 1u);
    const uint32_t n_items = n_flagged * per_seg;
    uint32_t* drawn = p.redo_queue + 2 * phase;
    uint32_t* finished = drawn + 1;
    uint32_t done = 0, next = 0;
    if (threadIdx.x == 0) next = __hip_atomic_fetch_add(drawn, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (true) {
      if (threadIdx.x == 0) sh_item = next;
      __syncthreads();
      const uint32_t item = sh_item;
      __syncthreads();
      if (item >= n_items) break;
      ++done;
      // (the next item is asked for now: the answer is back when this one is done)
      if (threadIdx.x == 0) next = __hip_atomic_fetch_add(drawn, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // (What an item needs is computed at its start, from a thread number that the compiler cannot trace: kept in
      // registers from the top of the kernel on, for all phases, these values cost more registers than there are.)
      int tid = threadIdx.x;
      asm volatile("" : "+v"(tid));
      const int lane = tid & 63;
      const int seg = (int)sh_flagged[item / per_seg];
      const uint32_t part = item % per_seg;   // chunk or batch of the segment
      uint32_t* rec = p.redo_rec + (int64_t)seg * p.redo_rec_stride;        // the segment's record, then four words per batch:
      uint32_t* batch_words = rec + kRecWords + 4 * part;                    // above, above in [lo, hi), members (then: first place in the union list), first place in the selection
      uint32_t* sk = (uint32_t*)(g.scores + (int64_t)seg * p.seg_stride);   // (keys, not scores: what the selection compares)
      uint64_t* bucket = p.list + (int64_t)seg * p.list_stride;             // the bucket's members, every batch's at its own tokens' places
      uint64_t* selection = bucket;                                         // (rank mode, from `write` on, when the members are spent) the selected composites
      const uint32_t* gh = p.redo_hist + (int64_t)seg * kHistBins;
      int32_t* uo = want_union ? p.union_idx + (int64_t)seg * (p.k + p.sink + p.local) : nullptr;

      if (phase == kRedoScore) {
        const int64_t t0 = (int64_t)part * kRedoChunk;
        sh_hist[2 * tid] = 0;
        sh_hist[2 * tid + 1] = 0;
        __syncthreads();
        {
          // (as the streaming GEMV does it: a uniform base per chunk and one 32-bit lane offset serve all loads - the
          // launcher has checked that a chunk's rows lie within 2 GB of its first)
          const int j = tid & 15, rg = tid >> 4;
          const int bh = seg / g.num_chunks, chunk = seg % g.num_chunks;
          const int h = bh % g.num_kv_heads, b = bh / g.num_kv_heads;
          const int64_t chunk_base = g.cluster_ids ? (int64_t)g.cluster_ids[seg] * g.chunk_len : (int64_t)chunk * g.chunk_len;
          float qf[8];
          load_group_query<DT, 1>(g.q, g.q_stride_b, b, h, g.group, j, qf);
          const uint32_t row_bytes = (uint32_t)g.key_stride_n * 2u;
          const unsigned char* cbase = (const unsigned char*)g.keys +
                                       2 * ((int64_t)b * g.key_stride_b + (int64_t)h * g.key_stride_h + (chunk_base + t0) * g.key_stride_n);   // uniform
          const int n_local = (int)(n - t0 < kRedoChunk ? n - t0 : kRedoChunk);
          constexpr int kRows = 8;
          for (int base = 0; base < n_local; base += (kSelThreads / 16) * kRows) {
            u32x4 kv[kRows];
#pragma unroll
            for (int u = 0; u < kRows; ++u) {
              int lt = base + rg * kRows + u;
              lt = lt < n_local ? lt : n_local - 1;
              kv[u] = __builtin_nontemporal_load((const u32x4*)(cbase + ((uint32_t)lt * row_bytes + 16u * (uint32_t)j)));
            }
            __builtin_amdgcn_sched_barrier(0);   // all loads go out before the first score is computed
            float mine = 0.0f;
#pragma unroll
            for (int u = 0; u < kRows; ++u) {
              const float s = row_score<DT>(qf, kv[u], g.scale);
              if (j == u) mine = s;
            }
            const int lt = base + rg * kRows + j;
            if (j < kRows && lt < n_local) {
              const uint32_t key = score_key(mine);
              __hip_atomic_store(sk + t0 + lt, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              atomicAdd(&sh_hist[key >> kTopShift], 1u);
            }
          }
        }
        __syncthreads();
        uint32_t* ghw = p.redo_hist + (int64_t)seg * kHistBins;
        for (int i = tid; i < kHistBins; i += kSelThreads)
          if (sh_hist[i]) __hip_atomic_fetch_add(ghw + i, sh_hist[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else if (phase == kRedoCount) {
        // this thread's 32 tokens first: the loads do not depend on the threshold
        const uint32_t first = part * (uint32_t)kRedoBatch + 32u * (uint32_t)tid;
        uint32_t keys[32];
        redo_load_run(sk, first, n, keys);
        uint32_t prefix, need, cnt;
        const int mode = redo_threshold(gh, k, batches_per_seg, sh_hist, sh_wtot, sh_res, &prefix, &need, &cnt);
        if (mode != kRedoAlone) {   // (uniform)
          if (tid == 0) {
            sh_res[2] = 0u;
            sh_res[3] = 0u;
          }
          __syncthreads();
          const uint32_t valid = (int64_t)first < n ? bit_range(0u, (uint32_t)(n - first < 32 ? n - first : 32)) : 0u;
          const uint32_t in_mid = bit_range(lo > first ? lo - first : 0u, hi > first ? hi - first : 0u);
          uint32_t above = 0, tie = 0;
#pragma unroll
          for (int e = 0; e < 32; ++e) {
            const uint32_t top = keys[e] >> kTopShift;
            shift_in_gt(above, top, prefix);
            shift_in_eq(tie, top, prefix);
          }
          above = __builtin_bitreverse32(above) & valid;
          tie = __builtin_bitreverse32(tie) & valid;
          if (mode == kRedoTakeBucket) {   // the members are taken like the tokens above them
            above |= tie;
            tie = 0;
          }
          const uint32_t packed = ((uint32_t)__builtin_popcount(above) << 16) | (uint32_t)__builtin_popcount(above & in_mid);
          const uint32_t inc = wave_inclusive_scan(packed);   // (at most 2048 of either per wave)
          if (lane == 63 && inc != 0u) atomicAdd(&sh_res[3], inc);
          // the members: to the batch's own part of the segment's list (as many places as it has tokens), in any order
          uint64_t* mine_at = bucket + (int64_t)part * kRedoBatch;
          while (tie != 0u) {   // (few)
            const uint32_t e = (uint32_t)__builtin_ctz(tie);
            tie &= tie - 1u;
            uint32_t key = 0;
#pragma unroll
            for (int q = 0; q < 32; ++q) key = (uint32_t)q == e ? keys[q] : key;   // (registers cannot be indexed)
            __hip_atomic_store(mine_at + atomicAdd(&sh_res[2], 1u), composite(key, first + e), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          __syncthreads();
          if (tid == 0) {
            __hip_atomic_store(batch_words, sh_res[3] >> 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(batch_words + 1, sh_res[3] & 0xffffu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(batch_words + 2, sh_res[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      } else if (phase == kRedoCut) {
        uint32_t prefix, need, cnt;
        const int mode = redo_threshold(gh, k, batches_per_seg, sh_hist, sh_wtot, sh_res, &prefix, &need, &cnt);
        uint64_t cut = (uint64_t)prefix << (64 - kHistBits);   // kRedoTakeBucket: every member is taken
        uint32_t mid_total;
        if (mode == kRedoAlone) {
          mid_total = redo_select_from_scores<DT, RANK>(g, p, seg, selection, smem, sh_hist, sh_off, sh_wtot, sh_res);
        } else {
          uint64_t* sh_buck = (uint64_t*)smem;
          // (kRedoTakeBucket: the members were counted with the tokens above them, nothing was gathered and nothing is cut)
          if (mode == kRedoCutBucket) {
            // the members lie in their batches' parts of the list: first place of every batch's members among all of them
            // (thread t: batches 2t, 2t+1), then every thread fetches members by their number
            uint32_t held[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const uint32_t b = 2u * (uint32_t)tid + e;
              held[e] = b < batches_per_seg ? __hip_atomic_load(rec + kRecWords + 4 * b + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
            }
            uint32_t total;
            const uint32_t ex = block_exclusive_scan(held[0] + held[1], sh_wtot, &total);
            sh_off[2 * tid] = ex;
            sh_off[2 * tid + 1] = ex + held[0];
            __syncthreads();
            for (uint32_t i = tid; i < cnt; i += kSelThreads) {
              uint32_t b = 0;   // the last batch whose first place is at or below i
#pragma unroll
              for (uint32_t step = kRedoMaxBatches / 2; step != 0u; step >>= 1)
                if (b + step < batches_per_seg && sh_off[b + step] <= i) b += step;
              sh_buck[i] = bucket[(int64_t)b * kRedoBatch + (i - sh_off[b])];
            }
            // the cut inside the bucket: the need-th largest of its members
            uint64_t cprefix = prefix;   // top `cfixed` bits of the composite
            int cfixed = kHistBits;
            uint32_t left = need, among = cnt;
            while (among != left && cfixed < 64) {
              const int bits = (64 - cfixed) >= kHistBits ? kHistBits : (64 - cfixed);
              const int shift = 64 - cfixed - bits;
              __syncthreads();
              sh_hist[2 * tid] = 0;
              sh_hist[2 * tid + 1] = 0;
              __syncthreads();
              for (uint32_t i = tid; i < cnt; i += kSelThreads) {
                const uint64_t cc = sh_buck[i];
                if ((cc >> (64 - cfixed)) == cprefix) atomicAdd(&sh_hist[(uint32_t)(cc >> shift) & ((1u << bits) - 1u)], 1u);
              }
              __syncthreads();
              find_threshold_bin_1024(sh_hist, left, sh_wtot, sh_res);
              left -= sh_res[1];
              cprefix = (cprefix << bits) | sh_res[0];
              among = sh_res[2];
              cfixed += bits;
            }
            cut = cfixed == 64 ? cprefix : cprefix << (64 - cfixed);   // every composite with these leading bits is taken
          }
          // the selected members of every batch (all / in [lo, hi))
          __syncthreads();
          sh_hist[2 * tid] = 0;
          sh_hist[2 * tid + 1] = 0;
          sh_off[2 * tid] = 0;
          sh_off[2 * tid + 1] = 0;
          __syncthreads();
          for (uint32_t i = tid; i < (mode == kRedoCutBucket ? cnt : 0u); i += kSelThreads) {
            const uint64_t cc = sh_buck[i];
            if (cc >= cut) {
              const uint32_t idx = ~(uint32_t)cc;
              atomicAdd(&sh_hist[idx / (uint32_t)kRedoBatch], 1u);
              if (idx - lo < hi - lo) atomicAdd(&sh_off[idx / (uint32_t)kRedoBatch], 1u);
            }
          }
          __syncthreads();
          // every batch's first place: thread t sums batches 2t, 2t+1 (selected << 16 | selected in [lo, hi): at most k each)
          uint32_t mine[2];
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const uint32_t b = 2u * (uint32_t)tid + e;
            mine[e] = 0u;
            if (b < batches_per_seg) {
              const uint32_t* bw = rec + kRecWords + 4 * b;
              mine[e] = ((__hip_atomic_load(bw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + sh_hist[b]) << 16) |
                        (__hip_atomic_load(bw + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + sh_off[b]);
            }
          }
          uint32_t total;
          const uint32_t ex = block_exclusive_scan(mine[0] + mine[1], sh_wtot, &total);
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const uint32_t b = 2u * (uint32_t)tid + e;
            if (b < batches_per_seg) {
              const uint32_t at = ex + (e ? mine[0] : 0u);
              uint32_t* bw = rec + kRecWords + 4 * b;
              __hip_atomic_store(bw + 2, at & 0xffffu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              __hip_atomic_store(bw + 3, at >> 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
          }
          mid_total = total & 0xffffu;
        }
        if (tid == 0) {
          __hip_atomic_store(rec + kRecPrefix, prefix, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(rec + kRecMode, (uint32_t)mode, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(rec + kRecCutLo, (uint32_t)cut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(rec + kRecCutHi, (uint32_t)(cut >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(rec + kRecMidTotal, mid_total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else if (phase == kRedoWrite) {
        // (the record and the batch's words were written by other workgroups in earlier phases, and what this CU's caches
        // held was dropped at the end of the last one: plain loads, all of them in flight together)
        const uint32_t first = part * (uint32_t)kRedoBatch + 32u * (uint32_t)tid;
        uint32_t keys[32];
        redo_load_run(sk, first, n, keys);
        const u32x4 r = *(const u32x4*)rec;          // prefix, mode, cut
        const u32x4 w = *(const u32x4*)batch_words;   // .., .., first place in the union list, in the selection
        const uint32_t mid_total = rec[kRecMidTotal];
        const int mode = (int)r[kRecMode];
        if (mode != kRedoAlone) {   // (uniform)
          // selected: the composite (key, ~index) is at least the cut
          const uint32_t cut_key = r[kRecCutHi], cut_low = r[kRecCutLo];
          const uint32_t valid = (int64_t)first < n ? bit_range(0u, (uint32_t)(n - first < 32 ? n - first : 32)) : 0u;
          const uint32_t in_mid = bit_range(lo > first ? lo - first : 0u, hi > first ? hi - first : 0u);
          uint32_t sel = 0, same = 0;
#pragma unroll
          for (int e = 0; e < 32; ++e) {
            shift_in_gt(sel, keys[e], cut_key);
            shift_in_eq(same, keys[e], cut_key);
          }
          sel = __builtin_bitreverse32(sel);
          same = __builtin_bitreverse32(same);
          while (same != 0u) {   // (few: tokens with the key of the cut fall to the smaller index)
            const uint32_t e = (uint32_t)__builtin_ctz(same);
            same &= same - 1u;
            sel |= (~(first + e) >= cut_low ? 1u : 0u) << e;
          }
          sel &= valid;
          const uint32_t mid = sel & in_mid;
          uint32_t total;
          const uint32_t ex = block_exclusive_scan(((uint32_t)__builtin_popcount(sel) << 16) | (uint32_t)__builtin_popcount(mid), sh_wtot, &total);
          uint32_t pos_mid = lo + w[2] + (ex & 0xffffu), pos_sel = w[3] + (ex >> 16);
          uint32_t rest = sel;
          while (rest != 0u) {   // (few: k tokens out of the whole segment)
            const uint32_t e = (uint32_t)__builtin_ctz(rest);
            rest &= rest - 1u;
            uint32_t key = 0;
#pragma unroll
            for (int q = 0; q < 32; ++q) key = (uint32_t)q == e ? keys[q] : key;   // (registers cannot be indexed)
            if (RANK) {
              if (pos_sel < k) __hip_atomic_store(selection + pos_sel, composite(key, first + e), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              ++pos_sel;
            }
            if (uo && (mid >> e & 1u)) uo[pos_mid++] = (int32_t)(first + e);
          }
        }
        if (part == 0u && uo) write_union_edges(uo, p, seg, lo, hi, mid_total);
      } else {   // kRedoFinish (RANK)
        uint64_t* sh_sort = (uint64_t*)smem;
        for (int i = tid; i < kpad; i += kSelThreads) sh_sort[i] = (uint32_t)i < k ? selection[i] : 0ull;  // pad: below every real composite
        __syncthreads();
        rank_sort_desc(sh_sort, sh_sort + kpad, k, kpad, sh_hist, sh_off, sh_wtot, sh_mm);
        write_rank_outputs(sh_sort, p, seg);
      }
    }
    if (phase == (RANK ? kRedoFinish : kRedoWrite)) break;
    // what this workgroup's items leave for later phases has completed before they count as done
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // ... and the items of this phase that other workgroups hold
    if (threadIdx.x == 0) {
      if (done != 0u) __hip_atomic_fetch_add(finished, done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      int spins = 0;
      while (__hip_atomic_load(finished, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < n_items && spins < kRedoWaitSpins) {
        __builtin_amdgcn_s_sleep(8);
        ++spins;
      }
      sh_item = spins < kRedoWaitSpins ? 1u : 0u;
    }
    __syncthreads();
    const bool go_on = sh_item != 0u;
    __syncthreads();
    if (!go_on) return;   // (this workgroup holds no item: the others finish without it)
    // what the other workgroups stored is read from here on: drop what the caches of this CU and its L2 hold (one wave
    // does that for the workgroup; 4096 waves at it cost tens of microseconds per phase)
    if (wave == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    __syncthreads();
  }
}

// ---- combine launch of the fused selection + attention, with the redo of flagged segments ----------------

// Attention of one workgroup of 1024 threads over a token list in memory, all G query heads of one KV head, result
// written directly (the only "split" of its rows).  The slow path of a slow path: one head after the other, a 16-lane
// row group per token, four rows in flight.  sh_acc: 64 x 128 floats, sh_ml: 128 floats.
template <int DT>
__device__ __forceinline__ void redo_attention(const AttnParams& a, const int32_t* list, int count, int b, int h, void* out,
                                               int64_t out_stride_b, int out_dtype, float* sh_acc, float* sh_ml) {
  constexpr int kRowGroups = kSelThreads / 16, U = 4;
  const int tid = threadIdx.x, j = tid & 15, rg = tid >> 4;
  const int64_t head_off = (int64_t)b * a.kv_stride_b + (int64_t)h * a.kv_stride_h + 8 * j;
  const uint16_t* kbase = (const uint16_t*)a.keys + head_off;
  const uint16_t* vbase = (const uint16_t*)a.values + head_off;
  for (int g = 0; g < a.group; ++g) {
    float qf[8];
    {
      const u32x4 v = *(const u32x4*)((const uint16_t*)a.q + (int64_t)b * a.q_stride_b + ((int64_t)h * a.group + g) * kHeadDim + 8 * j);
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[i] = Elem<DT>::get(v, i);
    }
    float m = -INFINITY, l = 0.0f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (int base = 0; base < count; base += kRowGroups * U) {
      u32x4 kv[U], vv[U];
      bool ok[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int pos = base + rg * U + u;
        int64_t t = pos < count ? (int64_t)list[pos] : -1;
        ok[u] = t >= 0 && t < a.seq_len;
        if (!ok[u]) t = 0;
        kv[u] = *(const u32x4*)(kbase + t * a.kv_stride_n);
        vv[u] = *(const u32x4*)(vbase + t * a.kv_stride_n);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) s = __builtin_fmaf(qf[i], Elem<DT>::get(kv[u], i), s);
        s = row16_sum(s) * a.scale_log2e;
        if (!ok[u]) continue;   // (uniform over the row group; a skipped row is never multiplied)
        const float mx = fmaxf(m, s);
        const float alpha = __builtin_amdgcn_exp2f(m - mx), pu = __builtin_amdgcn_exp2f(s - mx);
        m = mx;
        l = l * alpha + pu;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(pu, Elem<DT>::get(vv[u], i), acc[i] * alpha);
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) sh_acc[rg * kHeadDim + 8 * j + i] = acc[i];
    if (j == 0) { sh_ml[rg] = m; sh_ml[kRowGroups + rg] = l; }
    __syncthreads();
    if (tid < kHeadDim) {
      float M = -INFINITY;
      for (int r = 0; r < kRowGroups; ++r) M = fmaxf(M, sh_ml[r]);
      float L = 0.0f, o = 0.0f;
      if (M != -INFINITY) {
        for (int r = 0; r < kRowGroups; ++r) {
          const float w = __builtin_amdgcn_exp2f(sh_ml[r] - M);
          L += sh_ml[kRowGroups + r] * w;
          o += sh_acc[r * kHeadDim + tid] * w;
        }
      }
      const float res = L > 0.0f ? o / L : 0.0f;
      uint16_t* dst = (uint16_t*)out + (int64_t)b * out_stride_b + ((int64_t)h * a.group + g) * kHeadDim;
      dst[tid] = out_dtype == TKA_F16 ? Elem<TKA_F16>::narrow(res) : Elem<TKA_BF16>::narrow(res);
    }
  }
}

// Grid: c.rows combine workgroups, then one redo workgroup per segment (they come last so that the combine rows are
// not held up by workgroups that in all likelihood look at one word and leave).
template <int DT, int ODT>
__global__ __launch_bounds__(kSelThreads) void lse_combine_redo_kernel(CombineParams c, GemvParams g, SelectParams p, AttnParams a) {
  static_assert(kCombineThreads == kSelThreads, "one workgroup shape for both roles");
  struct RedoLds {
    uint32_t hist[kHistBins], off[kHistBins], wtot[kSelWaves], res[4];
    uint64_t mm[3];
    float acc[(kSelThreads / 16) * kHeadDim], ml[2 * (kSelThreads / 16)];
  };
  union Lds {
    CombineLds combine;
    RedoLds redo;
  };
  __shared__ __attribute__((aligned(16))) unsigned char raw[sizeof(Lds)];
  if ((int)blockIdx.x < c.rows) {
    const int row = (int)blockIdx.x;
    if (p.seg_flags[row / a.group] & 1u) return;   // its segment is redone: the redo workgroup writes the row
    lse_combine_row<ODT>(c, row, *(CombineLds*)raw);
    return;
  }
  const int seg = (int)blockIdx.x - c.rows;
  if (!(p.seg_flags[seg] & 1u)) return;
  RedoLds& sh = *(RedoLds*)raw;
  fallback_segment<DT>(g, p, seg, 0, nullptr, sh.hist, sh.off, sh.wtot, sh.res, sh.mm);
  __threadfence_block();
  __syncthreads();   // the list and its count, written by this workgroup, are read by it below
  const int count = __hip_atomic_load(p.union_count + seg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  redo_attention<DT>(a, p.union_idx + (int64_t)seg * (p.k + p.sink + p.local), count, seg / g.num_kv_heads, seg % g.num_kv_heads,
                     c.out, c.out_stride_b, c.out_dtype, sh.acc, sh.ml);
}

// ---- ranking of the common-cut route ---------------------------------------------------------------

// One lane's add to a 64-bit word in LDS, returning the word's old value.  (Written out: around an atomic that one lane of
// a wave executes the compiler builds its wave-wide aggregation - three loops over the active lanes - and this kernel
// pays for every instruction sixteen times.)
__device__ __forceinline__ uint64_t lds_add_rtn_u64(uint64_t* word, uint64_t v) {
  uint64_t old;
  const uint32_t offset = (uint32_t)(uintptr_t)word;   // (the low half of a shared-memory address is its place in LDS)
  asm volatile("ds_add_rtn_u64 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=v"(old) : "v"(offset), "v"(v) : "memory");
  return old;
}
__device__ __forceinline__ void lds_max_u32(uint32_t* word, uint32_t v) {
  const uint32_t offset = (uint32_t)(uintptr_t)word;
  asm volatile("ds_max_u32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(offset), "v"(v) : "memory");
}

constexpr uint32_t kCutBucketMax = 192;   // a bucket with more members than this sends the part to the sorting network

// Rank-ordered outputs of one candidate: index, value and expansion at position `rank` of segment `seg`.
__device__ __forceinline__ void write_ranked(const SelectParams& p, int seg, uint32_t idx_base, uint32_t rank, uint64_t c) {
  const uint32_t id = ~(uint32_t)c + idx_base;
  p.out_idx[(int64_t)seg * p.out_stride + rank] = (int32_t)id;
  if (p.out_val) p.out_val[(int64_t)seg * p.out_stride + rank] = key_score((uint32_t)(c >> 32));
  if (p.out_expand) {
    int32_t* oe = p.out_expand + ((int64_t)seg * p.k + rank) * p.expand;
    for (int i = 0; i < p.expand; ++i) oe[i] = (int32_t)(~(uint32_t)c * (uint32_t)p.expand + (uint32_t)i);
  }
}

// Size of the largest of those of the kCutParts parts of a segment's candidates that reach into the top k (the parts
// with fewer than k candidates above them; the others are never ranked): `pairs` pairs of head entries (zeros are no
// candidates), `n_extra` entries from beyond the heads, sh_split[1 .. kCutParts - 1] the inner ends of the parts in
// descending order.  sh_words: kCutParts words that are zero on entry and on exit.  Every thread of the workgroup calls it.
// Kept out of line: it runs when a segment has more candidates than one part may hold, which is rare, and the kernel
// around it is one whose every instruction counts.
__device__ __noinline__ uint32_t largest_part(const uint64_t* heads_flat, int n_pairs, const uint64_t* extra, uint32_t n_extra,
                                              const uint64_t* sh_split, uint32_t* sh_words, uint32_t k) {
  typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
  const u64x2* heads = (const u64x2*)heads_flat;
  const int tid = threadIdx.x, lane = tid & 63;
  static_assert(kCutParts % 8 == 0, "eight counts per word");
  uint64_t sizes[kCutParts / 8] = {};   // counts of 8 bits (a thread sees 24 entries at most)
  auto count = [&](uint64_t x) {
    uint32_t below = 0;
#pragma unroll
    for (int i = 1; i < kCutParts; ++i) below += x < sh_split[i] ? 1u : 0u;
#pragma unroll
    for (int w = 0; w < kCutParts / 8; ++w) sizes[w] += x != 0ull && (int)(below >> 3) == w ? 1ull << (8 * (below & 7u)) : 0ull;
  };
#pragma unroll 1
  for (int q = tid; q < n_pairs; q += kSelThreads) {
    const u64x2 two = heads[q];
    count(two[0]);
    count(two[1]);
  }
  if (extra) {
#pragma unroll 1
    for (uint32_t i = tid; i < n_extra; i += kSelThreads) count(extra[i]);
  }
#pragma unroll
  for (int i = 0; i < kCutParts / 2; ++i) {   // two parts per word, 16 bits each (at most 24 x 64 per wave)
    const uint64_t word = sizes[i / 4];
    const uint32_t one = (uint32_t)(word >> (16 * (i % 4))) & 0xffu, other = (uint32_t)(word >> (16 * (i % 4) + 8)) & 0xffu;
    const uint32_t inc = wave_inclusive_scan(one | (other << 16));
    if (lane == 63) {
      atomicAdd(&sh_words[2 * i], inc & 0xffffu);
      atomicAdd(&sh_words[2 * i + 1], inc >> 16);
    }
  }
  __syncthreads();
  uint32_t largest = 0, above = 0;
#pragma unroll
  for (int i = 0; i < kCutParts; ++i) {
    const uint32_t size = sh_words[i];
    largest = above < k ? max(largest, size) : largest;
    above += size;
  }
  __syncthreads();
  if (tid < kCutParts) sh_words[tid] = 0;
  __syncthreads();
  return largest;
}

// Common-cut route: the slices (256 tokens each, written by gemv_cut_kernel) hold every token at or above the
// segment's cut, as composites, and kCutParts sample composites split the order into parts: seven of about equal size
// that cover the top k with some room, and the rest down to the cut (gemv_cut_split_ranks).
// kCutParts workgroups per segment (one CU executes 64 lane-operations per cycle, and this is a kernel of a few
// workgroups: what one workgroup would spend on all candidates is the kernel's duration).  Each reads the head
// entries of ALL slices (a dense array, zeros behind a slice's last candidate) and the slice counts in one round
// trip (the rare slice with more than kCutHead candidates costs a second trip), counts the candidates above its
// part, and ranks the candidates of its part by counting instead of selecting and then sorting: composite minus the
// part's lower end, cut to its 11 leading bits, gives 2048 buckets in rank order; a histogram and one suffix scan
// give every bucket its first rank, the composites are scattered to their bucket, and each one counts the larger
// members of its own bucket.  rank < k: selected, and the rank is the output position.  Heavy ties that fill a bucket
// send the part to the bitonic network; a segment with fewer than k candidates (the sample misjudged it), with a part
// of more than kCutMaxCandidates or with more than kCutMaxExtras entries beyond the heads is redone from the keys by
// its first workgroup (fallback_segment).
// A caller that takes the selected tokens in any order and skips ids outside the cache (the attention of the decode
// step) gets the union list from the same workgroups: sink range and local window first, then one place per rank,
// which holds the token, or -1 when the token lies inside the ranges (it is listed there).
// Dynamic LDS: kCutMaxCandidates composites (the part, as found), then as many again (the part in bucket order;
// before that, entries from beyond the heads); the tie path and the fallback reuse both.
// PAIRS: pairs of head entries per thread, 4 (up to 128 slices) or 8 (up to 256); UNION: the union list is written (the
// rank-ordered outputs then only if asked for); ANNOUNCED: the GEMV launch announced the cuts to its own workgroups
// (p.tau_words), some of which may have given up waiting.  (Template arguments, not flags: a dozen instructions of
// bookkeeping on this kernel's straight path cost 0.4 of its 6.5 us.)
template <int DT, int PAIRS, bool UNION, bool ANNOUNCED>
__global__ __launch_bounds__(kSelThreads) void select_rank_kernel(GemvParams g, SelectParams p, int kpad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint64_t* sh_own = (uint64_t*)smem;
  uint64_t* sh_x = sh_own + kCutMaxCandidates;
  uint64_t* sh_extra = sh_x;
  __shared__ uint32_t sh_hist[kHistBins], sh_off[kHistBins], sh_cur[kHistBins];
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];
  __shared__ uint64_t sh_mm[3];
  __shared__ uint64_t sh_split[kCutParts + 1];
  __shared__ uint32_t sh_ovf[kCutMaxSlices];
  __shared__ __attribute__((aligned(8))) uint32_t sh_n[8];   // [0] slices with more than kCutHead entries, [1] entries beyond the heads, [2] candidates,
                                 // [3] a bucket too large, [4] candidates above the part, [5] candidates of the part (one 64-bit word
                                 // with [4]), [6] the largest key, [7] slices whose workgroup gave up waiting for the cut

  typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
  constexpr int kPairs = PAIRS;
  constexpr int kHeadMine = 2 * kPairs;                                  // head entries per thread
  constexpr int kMine = kHeadMine + kCutMaxExtras / kSelThreads;        // composites per thread, with those from beyond the heads

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // Grid: workgroups go to the eight XCDs in turn, and every workgroup of a segment reads all of the segment's candidates,
  // which the GEMV launch left in memory - with workgroup w on XCD w % 8, the eight of a segment are given numbers that
  // put them on one XCD, whose L2 they share (sixty-four workgroups of eight segments: 1.1 us less than with every XCD
  // fetching every segment).  The grid is rounded up to whole groups of eight segments; the workgroups of the others leave.
  static_assert(kCutParts == 8, "a segment's workgroups: one per step of eight in the grid");
  const int part = (int)(blockIdx.x >> 3) & 7;
  const int seg = (int)((blockIdx.x >> 6) << 3 | (blockIdx.x & 7u));
  if (seg >= p.num_segments) return;
  const int chunk = p.segs_per_row == 1 ? 0 : seg % p.segs_per_row;   // (a division only where a call has chunks)
  const uint32_t k = (uint32_t)p.k;
  const u64x2* heads = (const u64x2*)(p.cand_head + (int64_t)seg * p.parts * kCutHead);
  const int n_pairs = p.parts * (kCutHead / 2);

  u64x2 w[kPairs];
#pragma unroll
  for (int e = 0; e < kPairs; ++e) {
    const int q = e * kSelThreads + tid;
    w[e] = q < n_pairs ? heads[q] : (u64x2){0ull, 0ull};
  }
  const uint32_t slice_cnt = tid < p.parts ? p.list_cnt[(int64_t)seg * p.parts + tid] : 0u;

  // ends of the parts, in descending order: [part] above this workgroup's part, [part + 1] its lower end
  // (as a running minimum: the samples were ranked by keys whose last bits were replaced, so two of them may come
  // in the other order here)
  if (tid == 0) {
    uint64_t sp[kCutParts];
#pragma unroll
    for (int i = 0; i < kCutParts; ++i) sp[i] = p.cut_splits[(int64_t)seg * kCutParts + i];
    uint64_t low = ~0ull;
    sh_split[0] = low;
#pragma unroll
    for (int i = 0; i < kCutParts; ++i) {
      low = sp[i] < low ? sp[i] : low;
      sh_split[i + 1] = low;
    }
  }
  sh_hist[2 * tid] = 0;
  sh_hist[2 * tid + 1] = 0;
  if (tid < 8) sh_n[tid] = 0;
  __syncthreads();
  // (the slice of a workgroup that never saw its segment's cut holds no candidates)
  if (ANNOUNCED && slice_cnt == kCutGaveUp) atomicAdd(&sh_n[7], 1u);
  else if (slice_cnt > (uint32_t)kCutHead) sh_ovf[atomicAdd(&sh_n[0], 1u)] = (uint32_t)tid | (slice_cnt << 16);
  if ((tid & ~63) < p.parts) {   // the segment's candidates: the sum of the slice counts, in the waves that hold them
    const uint32_t total = wave_inclusive_scan(ANNOUNCED && slice_cnt == kCutGaveUp ? 0u : slice_cnt);
    if (lane == 63) atomicAdd(&sh_n[2], total);
  }
  __syncthreads();
  const uint32_t n_ovf = sh_n[0];
  if (n_ovf) {   // rare: slices whose candidates go beyond the head entries (scores that cluster in one place)
    // One such slice per wave, sixteen at a time, every load asked for before the first one is used: one round trip for
    // up to sixteen slices (slice after slice, each with its own trip, cost 1.6 us on a step of eight heads whose cuts
    // sat low).  A slice holds at most kCutTokensPerWg - kCutHead entries beyond its head: three per lane.
    const uint64_t* wide = p.list + (int64_t)seg * p.list_stride;
    constexpr int kBeyond = (kCutTokensPerWg - kCutHead + kWave - 1) / kWave;
    for (uint32_t first = 0; first < n_ovf; first += kSelWaves) {
      const uint32_t i = first + (uint32_t)(tid >> 6);
      uint64_t x[kBeyond];
#pragma unroll
      for (int u = 0; u < kBeyond; ++u) x[u] = 0ull;   // (no composite is zero)
      if (i < n_ovf) {
        const uint32_t sl = sh_ovf[i] & 0xffffu, cnt = sh_ovf[i] >> 16;
#pragma unroll
        for (int u = 0; u < kBeyond; ++u) {
          const uint32_t j = (uint32_t)kCutHead + (uint32_t)lane + (uint32_t)(u * kWave);
          if (j < cnt) x[u] = wide[(int64_t)sl * p.part_len + j];
        }
      }
#pragma unroll
      for (int u = 0; u < kBeyond; ++u)
        if (x[u] != 0ull) {
          const uint32_t pos = atomicAdd(&sh_n[1], 1u);
          if (pos < (uint32_t)kCutMaxExtras) sh_extra[pos] = x[u];
        }
    }
    __syncthreads();
  }
  const uint32_t n_extra = sh_n[1];
  uint64_t c[kMine];
#pragma unroll
  for (int e = 0; e < kPairs; ++e) {
    c[2 * e] = w[e][0];
    c[2 * e + 1] = w[e][1];
  }
#pragma unroll
  for (int e = 0; e < kCutMaxExtras / kSelThreads; ++e) c[2 * kPairs + e] = 0ull;
  if (n_ovf) {
#pragma unroll
    for (int e = 0; e < kCutMaxExtras / kSelThreads; ++e) {
      const uint32_t i = (uint32_t)e * kSelThreads + tid;
      if (i < n_extra && i < (uint32_t)kCutMaxExtras) c[2 * kPairs + e] = sh_extra[i];
    }
    __syncthreads();   // the extras are in registers: their place becomes the bucket-ordered part
  }

  // the candidates above this part, those of the part (marked here, collected below once the part is known to be ranked:
  // one add per wave gives them their places - an add per candidate on one LDS word is a cycle or more per candidate
  // of the workgroup, 0.3 to 1.5 us of this kernel), the part's largest key
  const uint64_t t_hi = sh_split[part], t_lo = sh_split[part + 1];
  uint32_t own_mask = 0, own_pos = 0;
  {
    // Two compares per entry and nothing else: at or above the part's lower end, and above the part (beyond the largest
    // composite below its upper end; nothing is above the first part).  No candidate is zero and no end of a part is: an
    // empty place is below every part.
    const uint64_t t_top = part == 0 ? ~0ull : t_hi - 1ull;
    uint32_t in_mask = 0, above_mask = 0;
#pragma unroll
    for (int i = 0; i < kHeadMine; ++i) {
      in_mask |= (c[i] >= t_lo ? 1u : 0u) << i;
      above_mask |= (c[i] > t_top ? 1u : 0u) << i;
    }
    if (n_ovf) {
#pragma unroll
      for (int i = kHeadMine; i < kMine; ++i) {
        in_mask |= (c[i] >= t_lo ? 1u : 0u) << i;
        above_mask |= (c[i] > t_top ? 1u : 0u) << i;
      }
    }
    own_mask = in_mask & ~above_mask;
    const uint32_t n_above = (uint32_t)__builtin_popcount(above_mask);
    const uint32_t mine = (uint32_t)__builtin_popcount(own_mask);
    const uint32_t inc = wave_inclusive_scan((mine << 16) | n_above);   // (at most 22 x 64 per wave each)
    uint64_t before = 0;
    if (lane == 63) before = lds_add_rtn_u64((uint64_t*)&sh_n[4], ((uint64_t)(inc >> 16) << 32) | (inc & 0xffffu));
    own_pos = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(before >> 32), 63) + (inc >> 16) - mine;
    if (part == 0) {   // the first part ends at the segment's largest key
      uint32_t kmax = 0;
#pragma unroll
      for (int i = 0; i < kHeadMine; ++i) kmax = max(kmax, (uint32_t)(c[i] >> 32));
      if (n_ovf) {
#pragma unroll
        for (int i = kHeadMine; i < kMine; ++i) kmax = max(kmax, (uint32_t)(c[i] >> 32));
      }
      kmax = wave_max_in_last_lane(kmax);
      if (lane == 63) lds_max_u32(&sh_n[6], kmax);
    }
  }
  __syncthreads();
  const uint32_t n_cand = sh_n[2], n_above = sh_n[4], n_own = sh_n[5];
  // More candidates than one part may hold (the sample sat low: at 65536 tokens and k = 2048 one call in ten): fine as
  // long as every part that reaches into the top k fits, which all workgroups of the segment have to see alike - each
  // counts the sizes of all parts.
  uint32_t max_part = 0;   // (no more candidates than one part may hold: every part fits)
  if (n_cand > (uint32_t)kCutMaxCandidates)
    max_part = largest_part((const uint64_t*)heads, n_pairs, n_ovf ? sh_extra : nullptr, min(n_extra, (uint32_t)kCutMaxExtras), sh_split, sh_hist, k);
  const uint32_t n_gave_up = ANNOUNCED ? sh_n[7] : 0u;
  const bool redo = n_cand < k || n_cand > (uint32_t)p.max_entries || n_extra > (uint32_t)kCutMaxExtras || max_part > (uint32_t)kCutMaxCandidates ||
                    n_gave_up != 0u;
  if (tid == 0 && part == 0) {
    p.seg_flags[seg] = (redo ? 1u : 0u) | (n_gave_up << 8);   // (as on the candidate route: bit 0 redone, bits 8.. slices that gave up)
    if (ANNOUNCED) p.tau_words[2 * seg] = 0ull;   // the word that announced the segment's cut: spent (a replayed graph brings the same epoch)
  }
  if (redo) {   // every workgroup of the segment sees the same counts: the first one redoes it, the others leave
    if (part != 0) return;
    __syncthreads();
    fallback_segment<DT>(g, p, seg, kpad, sh_own, sh_hist, sh_off, sh_wtot, sh_res, sh_mm);
    return;
  }
  if (n_above >= k || n_own == 0u) return;   // nothing of this part is selected

  // buckets: linear in the composite between the ends of the part (the first part ends at its largest key)
  const uint64_t base = t_lo;
  const uint64_t span = (part == 0 ? (((uint64_t)sh_n[6] << 32) | 0xffffffffull) : t_hi) - base;
  const int fixed = __builtin_clzll(span | 1ull);
  const int shift = 64 - fixed > kHistBits ? 64 - fixed - kHistBits : 0;
  // (a part that is ranked holds at most kCutMaxCandidates, see the checks above)
  {
    uint64_t* place = sh_own + own_pos;
#pragma unroll
    for (int i = 0; i < kHeadMine; ++i)
      if (own_mask >> i & 1u) *place++ = c[i];
    if (n_ovf) {
#pragma unroll
      for (int i = kHeadMine; i < kMine; ++i)
        if (own_mask >> i & 1u) *place++ = c[i];
    }
  }
  __syncthreads();
#pragma unroll 1
  for (uint32_t i = tid; i < n_own; i += kSelThreads) atomicAdd(&sh_hist[(uint32_t)((sh_own[i] - base) >> shift)], 1u);
  __syncthreads();
  // first rank of every bucket: number of composites in higher buckets (thread t owns buckets 2t, 2t+1)
  {
    const int wave = tid >> 6;
    const uint32_t h0 = sh_hist[2 * tid], h1 = sh_hist[2 * tid + 1];
    const uint32_t mine = h0 + h1;
    const uint32_t inc = wave_inclusive_scan(mine);
    const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
    const uint32_t ge = wave_total - inc + mine;   // this wave's composites in buckets >= 2t
    if (lane == 0) sh_wtot[wave] = ge;
    if (h0 > kCutBucketMax || h1 > kCutBucketMax) sh_n[3] = 1u;
    __syncthreads();
    // the composites of the waves above: one read and a sum across the wave instead of a loop of up to fifteen reads
    static_assert(kSelWaves <= 64, "one lane per wave");
    uint32_t above = lane > wave && lane < kSelWaves ? sh_wtot[lane] : 0u;
    above += lane_xor<1>(above);
    above += lane_xor<2>(above);
    above += lane_xor<4>(above);
    above += lane_xor<8>(above);
    above = (uint32_t)__builtin_amdgcn_readfirstlane((int)above);   // (sixteen waves: the sum stands in each of lanes 0 .. 15)
    sh_off[2 * tid + 1] = sh_cur[2 * tid + 1] = above + ge - mine;   // buckets > 2t+1
    sh_off[2 * tid] = sh_cur[2 * tid] = above + ge - h0;             // buckets > 2t
  }
  __syncthreads();
  const uint32_t idx_base = p.seg_base_ids ? (uint32_t)(p.seg_base_ids[seg] * p.seg_len) : (uint32_t)(chunk * p.seg_len);
  // What a ranked candidate leaves behind.  The union list of this route: sink range [0, lo) and local window [hi, n)
  // first, then one place per rank; a selected token that lies inside the ranges is listed there already, and its place
  // holds -1, which the attention kernels skip like any id outside the cache.  So the place is the rank: nobody needs to
  // know how many of the tokens above fall into the ranges.
  constexpr bool want_union = UNION;
  const uint32_t lo = (uint32_t)(p.sink < p.seg_len ? p.sink : p.seg_len);
  const uint32_t hi = (uint32_t)(p.seg_len - p.local > (int64_t)lo ? p.seg_len - p.local : (int64_t)lo);
  const uint32_t edges = lo + ((uint32_t)p.seg_len - hi);
  int32_t* uo = want_union ? p.union_idx + (int64_t)seg * (p.k + p.sink + p.local) : nullptr;
  if (want_union && part == 0) {
    // the ranges, the count and the padding come from the first workgroup, which always gets this far (its part holds
    // the first splitter)
    for (uint32_t i = (uint32_t)tid; i < edges; i += kSelThreads) uo[i] = (int32_t)(i < lo ? i : hi + (i - lo));
    for (uint32_t i = edges + k + (uint32_t)tid; i < (uint32_t)(p.k + p.sink + p.local); i += kSelThreads) uo[i] = -1;
    if (tid == 0) p.union_count[seg] = (int32_t)(edges + k);
  }
  auto emit = [&](uint32_t rank, uint64_t x) {
    if (rank >= k) return;
    if (!want_union || p.out_idx) write_ranked(p, seg, idx_base, rank, x);
    if (want_union) {
      const uint32_t t = ~(uint32_t)x;
      uo[edges + rank] = t >= lo && t < hi ? (int32_t)t : -1;
    }
  };
  if (sh_n[3] != 0u) {
    // heavy ties: sort the part and take it in order
    uint32_t npad = 64;
    while (npad < n_own) npad <<= 1;
    for (uint32_t i = n_own + tid; i < npad; i += kSelThreads) sh_own[i] = 0;   // pad: below every real composite
    __syncthreads();
    sort_lds_desc(sh_own, sh_x, (int)npad);
    for (uint32_t i = tid; i < n_own; i += kSelThreads) emit(n_above + i, sh_own[i]);
    return;
  }
#pragma unroll 1
  for (uint32_t i = tid; i < n_own; i += kSelThreads) {
    const uint64_t x = sh_own[i];
    sh_x[atomicAdd(&sh_cur[(uint32_t)((x - base) >> shift)], 1u)] = x;
  }
  __syncthreads();
  // every candidate of the part: its rank is the candidates above the part, plus the first rank of its bucket, plus the
  // larger members of the bucket
#pragma unroll 1
  for (uint32_t i = tid; i < n_own; i += kSelThreads) {
    const uint64_t x = sh_x[i];
    const uint32_t bin = (uint32_t)((x - base) >> shift);
    const uint32_t start = sh_off[bin], cnt = sh_hist[bin];
    uint32_t larger = 0;
    for (uint32_t j = 0; j < cnt; ++j) larger += sh_x[start + j] > x ? 1u : 0u;
    emit(n_above + start + larger, x);
  }
}

// ---- a small k out of a few thousand scores, few segments -------------------------------------------------

constexpr int kSmallMaxLen = 4096;    // scores per segment: four per thread
constexpr int kSmallMaxK = 256;
constexpr int kSmallMaxCand = 1024;   // entries of the threshold bucket and above that are ranked by counting

// Rank-ordered top k of a segment of up to 4096 scores by one workgroup, for calls of a few segments (the centroids of
// a few dozen heads): such a launch is a matter of instructions per thread - sixteen waves share a CU's four SIMDs, and
// every line of code is fetched cold - so the program is kept short.  Four keys per thread; one histogram of 2048 bins
// linear between the smallest and the largest key; the threshold bin from one suffix scan; the entries of that bin and
// above (k and a handful) ranked by counting, which is also their output position.  When that bin is crowded (ties)
// the whole segment goes through the sorting network instead.
// Dynamic LDS: 2 x 4096 composites (the sort and its exchange buffer; the candidates and the selected otherwise).
// FROM_KEYS: no GEMV launch before this one; the workgroup scores its segment itself (64 row groups of 16 lanes, 16 rows
// in flight each, canonical order), the keys go through LDS to the threads that own them.
template <int DT, bool FROM_KEYS>
__global__ __launch_bounds__(kSelThreads) void select_small_kernel(GemvParams g, SelectParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint64_t* sh_all = (uint64_t*)smem;
  uint64_t* sh_cand = sh_all;
  uint64_t* sh_sort = sh_all + kSmallMaxCand;
  __shared__ uint32_t sh_hist[kHistBins];
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];
  __shared__ uint32_t sh_n[3];   // (two spare words), candidates collected
  __shared__ __attribute__((aligned(8))) uint32_t sh_wmm[2 * kSelWaves];   // smallest and largest key of every wave

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // (grid: x = the segment inside its row, y = batch entry and KV head: a division by a run-time value is some
  // twenty-five instructions, and this kernel's every instruction counts)
  const int chunk = (int)blockIdx.x;
  const int seg = (int)blockIdx.y * (int)gridDim.x + chunk;
  const uint32_t k = (uint32_t)p.k;
  const int64_t n = p.seg_len;
  uint32_t keys[4], vm;
  if constexpr (FROM_KEYS) {
    uint32_t* sh_key = (uint32_t*)(sh_all + kSmallMaxLen);   // (the exchange half of the buffer: free until a sort)
    const int j = tid & 15, rg = tid >> 4;
    int b = 0, h = (int)blockIdx.y;
    if (g.batch != 1) {
      b = (int)(blockIdx.y / (uint32_t)g.num_kv_heads);
      h = (int)blockIdx.y - b * g.num_kv_heads;
    }
    const int64_t chunk_base = g.cluster_ids ? (int64_t)g.cluster_ids[seg] * g.chunk_len : (int64_t)chunk * g.chunk_len;
    const uint16_t* kbase = (const uint16_t*)g.keys + (int64_t)b * g.key_stride_b + (int64_t)h * g.key_stride_h +
                            chunk_base * g.key_stride_n + 8 * j;
    constexpr int kRows = 16;   // rows in flight per lane
    const int nn = (int)n;
    float qf[8];
    for (int base = 0; base < nn; base += (kSelThreads / 16) * kRows) {
      u32x4 kv[kRows];
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        const int t = base + rg * kRows + u;
        kv[u] = *(const u32x4*)(kbase + (int64_t)(t < nn ? t : nn - 1) * g.key_stride_n);
      }
      __builtin_amdgcn_sched_barrier(0);   // the rows are asked for before the query (whose conversion waits for it)
      if (base == 0) load_group_query<DT, 1>(g.q, g.q_stride_b, b, h, g.group, j, qf);   // (head after head: sixteen rows per lane are in flight, and two heads beside them spilled registers)
      float mine = 0.0f;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        const float s = row_score<DT>(qf, kv[u], g.scale);
        if (j == u) mine = s;
        if (u % 4 == 3) __builtin_amdgcn_sched_barrier(0);   // (four rows at a time: all sixteen scheduled together spilled registers)
      }
      const int t = base + rg * kRows + j;
      if (t < nn) sh_key[t] = score_key(mine);
    }
    __syncthreads();
    vm = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int t = 4 * tid + e;
      const bool ok = t < nn;
      keys[e] = ok ? sh_key[t] : 0u;
      vm |= (ok ? 1u : 0u) << e;
    }
  } else {
    const float* sc = p.scores + (int64_t)seg * p.seg_stride;
    load_keys<4>(sc, (int64_t)tid * 4, n, (((uintptr_t)sc) & 15u) == 0, keys, &vm);
  }
  sh_hist[2 * tid] = 0;
  sh_hist[2 * tid + 1] = 0;
  if (tid == 0) { sh_n[0] = ~0u; sh_n[1] = 0u; sh_n[2] = 0u; sh_res[0] = 0u; sh_res[1] = 0u; sh_res[2] = 0u; }
  uint32_t kmin = ~0u, kmax = 0u;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (vm >> e & 1u) {
      kmin = min(kmin, keys[e]);
      kmax = max(kmax, keys[e]);
    }
  }
  kmin = wave_min_in_last_lane(kmin);
  kmax = wave_max_in_last_lane(kmax);
  // (the waves' extremes through LDS, one lane per wave, and across sixteen lanes: one barrier and no atomics)
  if (lane == 63) { sh_wmm[2 * (tid >> 6)] = kmin; sh_wmm[2 * (tid >> 6) + 1] = kmax; }
  __syncthreads();
  {
    static_assert(kSelWaves == 16, "sixteen lanes hold the waves' extremes");
    const uint2 mm = *(const uint2*)&sh_wmm[2 * (lane & 15)];
    kmin = mm.x;  kmax = mm.y;
    kmin = min(kmin, lane_xor<1>(kmin));   kmax = max(kmax, lane_xor<1>(kmax));
    kmin = min(kmin, lane_xor<2>(kmin));   kmax = max(kmax, lane_xor<2>(kmax));
    kmin = min(kmin, lane_xor<4>(kmin));   kmax = max(kmax, lane_xor<4>(kmax));
    kmin = min(kmin, lane_xor<8>(kmin));   kmax = max(kmax, lane_xor<8>(kmax));
  }
  // bins: the 11 leading bits of key - smallest key, counted from the leading bit of the range
  const int fixed = kmax == kmin ? 31 : __builtin_clz(kmax - kmin);
  const int shift = 32 - fixed > kHistBits ? 32 - fixed - kHistBits : 0;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (vm >> e & 1u) atomicAdd(&sh_hist[(keys[e] - kmin) >> shift], 1u);
  __syncthreads();
  find_threshold_bin_1024(sh_hist, k, sh_wtot, sh_res);
  const uint32_t d = sh_res[0], n_cand = sh_res[1] + sh_res[2];   // the threshold bin; entries in it and above
  if (n_cand > (uint32_t)kSmallMaxCand) {
    // a crowded threshold bin (ties): sort the whole segment
    uint32_t npad = 64;
    while (npad < (uint32_t)n) npad <<= 1;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t i = (uint32_t)tid * 4 + e;
      if (i < npad) sh_all[i] = (vm >> e & 1u) ? composite(keys[e], i) : 0ull;   // pad: below every real composite
    }
    __syncthreads();
    sort_lds_desc(sh_all, sh_all + npad, (int)npad);
    write_rank_outputs(sh_all, p, seg, chunk);
    return;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if ((vm >> e & 1u) && ((keys[e] - kmin) >> shift) >= d) sh_cand[atomicAdd(&sh_n[2], 1u)] = composite(keys[e], (uint32_t)tid * 4 + e);
  __syncthreads();
  // rank = number of larger candidates: eight neighbouring lanes per candidate, each with an eighth of the list, add up
  // across the lanes; the rank is the place
  {
    const uint32_t part = (uint32_t)tid & 7u, per = (n_cand + 7u) / 8u;
    const uint32_t j0 = part * per, j1 = min(j0 + per, n_cand);
    for (uint32_t first = 0; first < n_cand; first += kSelThreads / 8) {
      const uint32_t i = first + ((uint32_t)tid >> 3);
      const uint64_t x = sh_cand[i < n_cand ? i : 0u];
      uint32_t larger = 0;
      for (uint32_t j = j0; j < j1; ++j) larger += sh_cand[j] > x ? 1u : 0u;
      larger += lane_xor<1>(larger);
      larger += lane_xor<2>(larger);
      larger += lane_xor<4>(larger);
      if (part == 0u && i < n_cand && larger < k) sh_sort[larger] = x;
    }
  }
  __syncthreads();
  write_rank_outputs(sh_sort, p, seg, chunk);
}

// The same for sequences of up to 262144 tokens, without a sort: the selected ids between the ranges are marked in a
// bitmap of the sequence in LDS (WORDS x 4 KB: 8 KB for 65536 tokens), every thread counts the bits of its 32 WORDS
// tokens, one scan gives it its place, and it writes its tokens in order - ascending because the threads own ascending
// stretches of the sequence.  Ids outside the sequence are dropped, an id given twice is listed once (as the sorting form
// does).
constexpr int kUnionBitmapMaxLen = 262144;
template <int WORDS>
__global__ __launch_bounds__(kSelThreads) void index_union_bitmap_kernel(UnionParams p) {
  __shared__ uint32_t sh_bits[WORDS * kSelThreads];
  __shared__ uint32_t sh_wtot[kSelWaves];
  const int tid = threadIdx.x;
  const int seg = blockIdx.x;
  const uint32_t n = (uint32_t)p.seq_len;
  const uint32_t lo = (uint32_t)(p.sink < p.seq_len ? p.sink : p.seq_len);
  const uint32_t hi = (uint32_t)(p.seq_len - p.local > (int64_t)lo ? p.seq_len - p.local : (int64_t)lo);
  const int32_t* in = p.idx + (int64_t)seg * p.k;
#pragma unroll
  for (int w = 0; w < WORDS; ++w) sh_bits[WORDS * tid + w] = 0u;
  __syncthreads();
  for (int i = tid; i < p.k; i += kSelThreads) {
    const uint32_t id = (uint32_t)in[i];   // (a negative id is a large one here)
    if (id >= lo && id < hi) atomicOr(&sh_bits[id >> 5], 1u << (id & 31u));
  }
  __syncthreads();
  uint32_t bits[WORDS], mine = 0;
#pragma unroll
  for (int w = 0; w < WORDS; ++w) {
    bits[w] = sh_bits[WORDS * tid + w];
    mine += (uint32_t)__builtin_popcount(bits[w]);
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan(mine, sh_wtot, &total);
  int32_t* out = p.out_idx + (int64_t)seg * (p.k + p.sink + p.local);
  const uint32_t cap = (uint32_t)(p.k + p.sink + p.local);
  uint32_t pos = lo + before;
#pragma unroll
  for (int w = 0; w < WORDS; ++w) {
    const uint32_t first = 32u * (uint32_t)(WORDS * tid + w);
    uint32_t left = bits[w];
    while (left) {
      out[pos++] = (int32_t)(first + (uint32_t)__builtin_ctz(left));
      left &= left - 1u;
    }
  }
  const uint32_t count = lo + total + (n - hi);
  for (uint32_t i = (uint32_t)tid; i < lo; i += kSelThreads) out[i] = (int32_t)i;
  for (uint32_t i = (uint32_t)tid; i < n - hi; i += kSelThreads) out[lo + total + i] = (int32_t)(hi + i);
  for (uint32_t i = count + (uint32_t)tid; i < cap; i += kSelThreads) out[i] = -1;
  if (tid == 0) p.out_count[seg] = (int32_t)count;
}

// Ascending duplicate-free union of the selected ids with [0,sink) and [n-local,n).
// One workgroup per segment; the middle part is sorted ascending with the same bitonic network
// (ids complemented so that "descending" composites are ascending ids).
__global__ __launch_bounds__(kSelThreads) void index_union_kernel(UnionParams p, int kpad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint64_t* sh_sort = (uint64_t*)smem;
  uint64_t* sh_xchg = sh_sort + kpad;
  const int tid = threadIdx.x;
  const int seg = blockIdx.x;
  const int64_t n = p.seq_len;
  const int64_t lo = p.sink < n ? p.sink : n;
  const int64_t hi = n - p.local > lo ? n - p.local : lo;
  const int32_t* in = p.idx + (int64_t)seg * p.k;
  for (int i = tid; i < kpad; i += kSelThreads) {
    uint64_t c = 0;
    if (i < p.k) {
      int32_t id = in[i];
      if (id >= lo && id < hi) c = (uint64_t)(uint32_t)~(uint32_t)id + 1u;  // > 0, larger = smaller id
    }
    sh_sort[i] = c;
  }
  __syncthreads();
  sort_lds_desc(sh_sort, sh_xchg, kpad);
  // count distinct non-zero entries; entry i is kept when it differs from entry i-1
  int32_t* out = p.out_idx + (int64_t)seg * (p.k + p.sink + p.local);
  const int cap = p.k + p.sink + p.local;
  // positions: a prefix count of "kept" flags.  kpad <= 8192: each thread scans its contiguous run.
  const int per = kpad >= kSelThreads ? kpad / kSelThreads : 1;
  uint32_t mine = 0;
  for (int s = 0; s < per; ++s) {
    int i = tid * per + s;
    if (i >= kpad) break;
    uint64_t c = sh_sort[i];
    if (c != 0 && (i == 0 || sh_sort[i - 1] != c)) ++mine;
  }
  __shared__ uint32_t sh_wtot[kSelWaves];
  const int lane = tid & 63, wave = tid >> 6;
  uint32_t pre = mine;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    uint32_t t = __shfl_up(pre, d, 64);
    if (lane >= d) pre += t;
  }
  if (lane == 63) sh_wtot[wave] = pre;
  __syncthreads();
  uint32_t wbase = 0, total = 0;
  for (int w = 0; w < kSelWaves; ++w) {
    if (w < wave) wbase += sh_wtot[w];
    total += sh_wtot[w];
  }
  uint32_t pos = (uint32_t)lo + wbase + (pre - mine);
  for (int s = 0; s < per; ++s) {
    int i = tid * per + s;
    if (i >= kpad) break;
    uint64_t c = sh_sort[i];
    if (c != 0 && (i == 0 || sh_sort[i - 1] != c)) out[pos++] = (int32_t)~(uint32_t)(c - 1u);
  }
  for (int64_t t = tid; t < lo; t += kSelThreads) out[t] = (int32_t)t;
  const uint32_t mid_end = (uint32_t)lo + total;
  for (int64_t t = hi + tid; t < n; t += kSelThreads) out[mid_end + (t - hi)] = (int32_t)t;
  const uint32_t count = mid_end + (uint32_t)(n - hi);
  for (int i = (int)count + tid; i < cap; i += kSelThreads) out[i] = -1;
  if (tid == 0) p.out_count[seg] = (int32_t)count;
}

int kpad_for(int k) {
  int kpad = 64;
  while (kpad < k) kpad <<= 1;
  return kpad;
}

}  // namespace

// Workspace layout (each part 256-byte aligned):
//   hist [S][2048] u32 (cleared per call) | flags [S] u32 | tau [S] u64 | arrival flags [S][64] u32 | sample pool [S][8192] u32 |
//   candidate heads [S][slices][32] u64 | list_cnt [S][slices] u32 |
//   list [S][slices*slice_len] u64      (slices: dense 4096/16384 scores, candidate mode one per GEMV workgroup)
namespace {
struct SelectLayout {
  size_t hist, flags, tau, ctr, pool, head, list_cnt, list, arrive, total;
  int64_t list_stride;
};
SelectLayout select_layout(int num_segments, int64_t seg_len) {
  SelectLayout l;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t at = off; off += align_up(bytes, 256); return at; };
  const int64_t max_parts = seg_len / 128 + 2;   // candidate mode: one slice per GEMV workgroup of >= 128 tokens
  l.list_stride = (seg_len + 16 * kSelThreads - 1) / (16 * kSelThreads) * (16 * kSelThreads);  // whole slices
  l.hist = take((size_t)num_segments * kHistBins * sizeof(uint32_t));
  l.flags = take((size_t)num_segments * sizeof(uint32_t));
  l.tau = take((size_t)num_segments * 2 * sizeof(uint64_t));
  const size_t cand_segs = seg_len >= kCandMinSegLen ? (size_t)num_segments : 0;   // sampling state: long segments only
  l.ctr = take(cand_segs * 64 * sizeof(uint32_t));
  l.pool = take(cand_segs * kGemvMaxSamples * sizeof(uint32_t));
  // head entries of the slices: the candidate route (32 per slice of 512 tokens) or the common-cut route (64 per slice of 256)
  const size_t cut_segs = seg_len <= (int64_t)kCutMaxSlices * kCutTokensPerWg ? (size_t)num_segments : 0;
  const size_t head_cand = cand_segs * (size_t)(seg_len / kGemvCandTokensPerWg + 1) * kCandHead * sizeof(uint64_t);
  // (slices of 128 tokens where a segment has no more than kCutMaxSlices of them, see gemv_cut_plan)
  const int64_t cut_slices = seg_len <= (int64_t)kCutMaxSlices * (kCutTokensPerWg / 2) ? seg_len / (kCutTokensPerWg / 2) + 1 : seg_len / kCutTokensPerWg + 1;
  const size_t head_cut = cut_segs * (size_t)cut_slices * kCutHead * sizeof(uint64_t);
  l.head = take(head_cand > head_cut ? head_cand : head_cut);
  l.list_cnt = take((size_t)num_segments * (size_t)max_parts * sizeof(uint32_t));
  l.list = take((size_t)num_segments * (size_t)l.list_stride * sizeof(uint64_t));
  l.arrive = take(cand_segs ? 2 * kRedoPhasesMax * sizeof(uint32_t) : 0);   // item counters of the redo launch (cleared by the selection when it flags a segment)
  l.total = off;
  return l;
}
}  // namespace

size_t select_workspace_bytes(int num_segments, int64_t seg_len) { return select_layout(num_segments, seg_len).total; }

// Carves the workspace; returns how many leading 32-bit words (the histograms) need clearing.
size_t select_carve(void* ws, int num_segments, int64_t seg_len, SelectParams* p) {
  const SelectLayout l = select_layout(num_segments, seg_len);
  unsigned char* c = (unsigned char*)ws;
  p->hist = (uint32_t*)(c + l.hist);
  p->seg_flags = (uint32_t*)(c + l.flags);
  p->tau_words = (uint64_t*)(c + l.tau);
  p->sample_flags = (uint32_t*)(c + l.ctr);
  p->sample_pool = (uint32_t*)(c + l.pool);
  p->cand_head = (const uint64_t*)(c + l.head);
  p->list_cnt = (uint32_t*)(c + l.list_cnt);
  p->list = (uint64_t*)(c + l.list);
  p->list_stride = l.list_stride;
  p->redo_queue = (uint32_t*)(c + l.arrive);
  p->redo_rec = p->list_cnt;   // (the slice counts of the other routes: a record and four words per chunk of 4096 tokens fit)
  p->redo_rec_stride = (seg_len / 128 + 2) & ~(int64_t)3;   // (whole 16-byte groups: the record is read with vector loads)
  // (redo_hist: the histograms, on the route that does not use them otherwise; set by the caller)
  return (size_t)num_segments * kHistBins;  // the flags follow the histograms; candidate mode writes them itself
}

// The words of a carved workspace that tell a call's sampling state from older contents (segment flags, thresholds,
// arrival flags: contiguous): *words = their start, returns how many 32-bit words they are.
size_t select_epoch_words(void* ws, int num_segments, int64_t seg_len, uint32_t** words) {
  const SelectLayout l = select_layout(num_segments, seg_len);
  *words = (uint32_t*)((unsigned char*)ws + l.flags);
  return (l.pool - l.flags) / sizeof(uint32_t);
}

// Slice per workgroup: 16384 scores (16 per thread) when that still gives every CU work, else 4096.
void select_plan(int64_t seg_len, int num_segments, SelectParams* p) {
  const int64_t big = 16 * kSelThreads;
  const int64_t parts_big = (seg_len + big - 1) / big;
  p->part_len = parts_big * num_segments >= 256 ? (int)big : 4 * kSelThreads;
  p->parts = (int)((seg_len + p->part_len - 1) / p->part_len);
}

int launch_zero_u32(uint32_t* ptr, size_t count, hipStream_t stream) {
  if (count == 0) return TKA_OK;
  LaunchTimer timer("zero_u32", stream);
  zero_u32_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(ptr, count);
  return hip_status(hipGetLastError());
}

int launch_select_hist(const SelectParams& p, hipStream_t stream) {
  LaunchTimer timer("select_hist", stream);
  const dim3 grid((unsigned)p.parts, (unsigned)p.num_segments);
  if (p.part_len == 16 * kSelThreads)
    select_hist_kernel<16><<<grid, kSelThreads, 0, stream>>>(p);
  else
    select_hist_kernel<4><<<grid, kSelThreads, 0, stream>>>(p);
  return hip_status(hipGetLastError());
}

// Raises a kernel's dynamic-LDS limit once per (kernel, device); safe to call from several host threads.
int allow_dynamic_lds(const void* kernel, int bytes) {
  static std::mutex guard;
  static std::vector<std::pair<const void*, int>> done;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return TKA_EHIP;
  std::lock_guard<std::mutex> lock(guard);
  for (const auto& d : done)
    if (d.first == kernel && d.second == device) return TKA_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return TKA_EHIP;
  done.emplace_back(kernel, device);
  return TKA_OK;
}

static int set_finalize_attr() {
  return allow_dynamic_lds((const void*)select_finalize_kernel, 130 * 1024);   // 2 x 8192 composites; 25 KB are static
}

int launch_select_filter(const SelectParams& p, hipStream_t stream) {
  LaunchTimer timer("select_filter", stream);
  const dim3 grid((unsigned)p.parts, (unsigned)p.num_segments);
  if (p.part_len == 16 * kSelThreads)
    select_filter_kernel<16><<<grid, kSelThreads, 0, stream>>>(p);
  else
    select_filter_kernel<4><<<grid, kSelThreads, 0, stream>>>(p);
  return hip_status(hipGetLastError());
}

int launch_select_finalize(const SelectParams& p, hipStream_t stream) {
  const bool want_rank = p.out_idx != nullptr;
  const int kpad = kpad_for(p.k);
  const size_t lds = want_rank ? 2 * (size_t)kpad * sizeof(uint64_t) : 0;
  if (set_finalize_attr() != TKA_OK) return TKA_EHIP;
  LaunchTimer timer("select_finalize", stream);
  select_finalize_kernel<<<(unsigned)p.num_segments, kSelThreads, lds, stream>>>(p, kpad);
  return hip_status(hipGetLastError());
}

int select_cand_max_parts() { return kCandMaxParts; }
int select_cand_capacity() { return kCandCap; }

int launch_select_finalize_cand(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream) {
  if ((p.from_keys || p.from_scores) ? p.seg_len > kCandCap : p.parts > kCandMaxParts) return TKA_EINVAL;
  if (p.k > kCandCap / 2) return TKA_EINVAL;
  if (allow_dynamic_lds((const void*)select_finalize_cand_kernel<TKA_F16>, kCandCap * (int)sizeof(uint64_t)) != TKA_OK ||
      allow_dynamic_lds((const void*)select_finalize_cand_kernel<TKA_BF16>, kCandCap * (int)sizeof(uint64_t)) != TKA_OK)
    return TKA_EHIP;
  LaunchTimer timer(p.from_keys ? "gemv_topk_fused" : (p.from_scores ? "select_whole" : "select_finalize_cand"), stream);
  // entries of the segment; rank mode reuses the buffer as sort + exchange buffers (2 x kpad, or 2 x the padded
  // segment when a short segment is sorted whole).  Short segments leave room for two workgroups per CU.
  size_t entries = kCandCap;
  if (p.from_keys || p.from_scores) {
    entries = (size_t)p.seg_len;
    if (p.out_idx) {
      size_t pad = (size_t)kpad_for(p.k);
      if (!p.union_idx && p.seg_len <= 2 * kSelThreads) pad = (size_t)kpad_for((int)p.seg_len);
      if (entries < 2 * pad) entries = 2 * pad;
    }
  }
  const size_t lds = entries * sizeof(uint64_t);
  if (dtype == TKA_F16)
    select_finalize_cand_kernel<TKA_F16><<<(unsigned)p.num_segments, kSelThreads, lds, stream>>>(g, p, kpad_for(p.k));
  else
    select_finalize_cand_kernel<TKA_BF16><<<(unsigned)p.num_segments, kSelThreads, lds, stream>>>(g, p, kpad_for(p.k));
  return hip_status(hipGetLastError());
}

int launch_select_rank(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream) {
  if (p.parts < 1 || p.parts > kCutMaxSlices || (p.part_len != kCutTokensPerWg && p.part_len != kCutTokensPerWg / 2) || p.k > kCutMaxK || (!p.out_idx && !p.union_idx) || !p.cand_head ||
      !p.list_cnt || !p.cut_splits || !p.seg_flags || (p.union_idx && !p.union_count))
    return TKA_EINVAL;
  const int lds = 2 * kCutMaxCandidates * (int)sizeof(uint64_t);
  typedef void (*RankKernel)(GemvParams, SelectParams, int);
#define TKA_RANK_KERNELS(DT, PAIRS) \
  {{select_rank_kernel<DT, PAIRS, false, false>, select_rank_kernel<DT, PAIRS, false, true>}, \
   {select_rank_kernel<DT, PAIRS, true, false>, select_rank_kernel<DT, PAIRS, true, true>}}
  static const RankKernel kernels[2][2][2][2] = {   // [dtype][more than 8 head entries per thread][union list][cuts announced in the GEMV launch]
      {TKA_RANK_KERNELS(TKA_F16, 4), TKA_RANK_KERNELS(TKA_F16, 8)}, {TKA_RANK_KERNELS(TKA_BF16, 4), TKA_RANK_KERNELS(TKA_BF16, 8)}};
#undef TKA_RANK_KERNELS
  const bool wide = p.parts * kCutHead > 8 * kSelThreads;
  const RankKernel kernel = kernels[dtype == TKA_F16 ? 0 : 1][wide ? 1 : 0][p.union_idx ? 1 : 0][p.tau_words ? 1 : 0];
  if (allow_dynamic_lds((const void*)kernel, lds) != TKA_OK) return TKA_EHIP;
  LaunchTimer timer("select_rank", stream);
  if (p.segs_per_row < 1 || p.num_segments % p.segs_per_row || p.num_segments > (1 << 24)) return TKA_EINVAL;
  const dim3 wgs((unsigned)((p.num_segments + 7) / 8 * 8 * kCutParts));   // (see the kernel)
  hipLaunchKernelGGL(kernel, wgs, dim3(kSelThreads), lds, stream, g, p, kpad_for(p.k));
  return hip_status(hipGetLastError());
}

// Behind launch_select_finalize_cand on the candidate route (p.redo_hist / p.redo_queue set there too): redoes the segments
// that the selection flagged, all workgroups of the launch sharing the work; leaves at once when there is none.
bool redo_segments_fits(const GemvParams& g, int num_segments) {
  return g.key_stride_n * 2 * (int64_t)kRedoChunk <= 0x7fffffffLL && num_segments <= kRedoMaxFlagged;
}

int launch_redo_segments(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream) {
  if (!p.redo_hist || !p.redo_queue || !p.redo_rec || !p.list || !p.seg_flags || !g.scores || !redo_segments_fits(g, p.num_segments) ||
      p.list_stride < p.seg_len || p.redo_rec_stride < kRecWords + 4 * ((p.seg_len + kRedoBatch - 1) / kRedoBatch))
    return TKA_EINVAL;
  const bool want_rank = p.out_idx != nullptr;
  const int kpad = kpad_for(p.k);
  const size_t bucket = (size_t)kRedoBucketCap * sizeof(uint64_t), sort = want_rank ? 2 * (size_t)kpad * sizeof(uint64_t) : 0;
  const size_t lds = bucket > sort ? bucket : sort;
  const int lds_max = 2 * kpad_for(TKA_MAX_TOPK) * (int)sizeof(uint64_t) > (int)bucket ? 2 * kpad_for(TKA_MAX_TOPK) * (int)sizeof(uint64_t) : (int)bucket;
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
    return n;
  }();
  const void* fn = dtype == TKA_F16 ? (want_rank ? (const void*)redo_segments_kernel<TKA_F16, true> : (const void*)redo_segments_kernel<TKA_F16, false>)
                                    : (want_rank ? (const void*)redo_segments_kernel<TKA_BF16, true> : (const void*)redo_segments_kernel<TKA_BF16, false>);
  if (allow_dynamic_lds(fn, lds_max) != TKA_OK) return TKA_EHIP;
  LaunchTimer timer("redo_segments", stream);
#define TKA_LAUNCH_REDO(DT, RANK) redo_segments_kernel<DT, RANK><<<(unsigned)cus, kSelThreads, lds, stream>>>(g, p, kpad)
  if (dtype == TKA_F16) {
    if (want_rank) TKA_LAUNCH_REDO(TKA_F16, true); else TKA_LAUNCH_REDO(TKA_F16, false);
  } else {
    if (want_rank) TKA_LAUNCH_REDO(TKA_BF16, true); else TKA_LAUNCH_REDO(TKA_BF16, false);
  }
#undef TKA_LAUNCH_REDO
  return hip_status(hipGetLastError());
}

int launch_lse_combine_redo(const CombineParams& c, const GemvParams& g, const SelectParams& s, const AttnParams& a, int dtype,
                            hipStream_t stream) {
  if (s.out_idx || !s.union_idx || !s.union_count || !s.seg_flags || g.num_chunks != 1 || c.rows != s.num_segments * a.group)
    return TKA_EINVAL;
  LaunchTimer timer("lse_combine_redo", stream);
  const unsigned grid = (unsigned)(c.rows + s.num_segments);
#define TKA_LAUNCH_COMBINE_REDO(DT, ODT) lse_combine_redo_kernel<DT, ODT><<<grid, kSelThreads, 0, stream>>>(c, g, s, a)
  if (dtype == TKA_F16) {
    if (c.out_dtype == TKA_F16) TKA_LAUNCH_COMBINE_REDO(TKA_F16, TKA_F16);
    else TKA_LAUNCH_COMBINE_REDO(TKA_F16, TKA_BF16);
  } else {
    if (c.out_dtype == TKA_F16) TKA_LAUNCH_COMBINE_REDO(TKA_BF16, TKA_F16);
    else TKA_LAUNCH_COMBINE_REDO(TKA_BF16, TKA_BF16);
  }
#undef TKA_LAUNCH_COMBINE_REDO
  return hip_status(hipGetLastError());
}

int select_small_max_len() { return kSmallMaxLen; }
int select_small_max_k() { return kSmallMaxK; }

int launch_select_small(const SelectParams& p, hipStream_t stream) {
  if (p.seg_len > kSmallMaxLen || p.k > kSmallMaxK || p.k > p.seg_len || !p.out_idx || p.union_idx) return TKA_EINVAL;
  const int lds = 2 * kSmallMaxLen * (int)sizeof(uint64_t);
  if (allow_dynamic_lds((const void*)select_small_kernel<TKA_F16, false>, lds) != TKA_OK) return TKA_EHIP;
  if (p.segs_per_row < 1 || p.num_segments % p.segs_per_row || p.num_segments / p.segs_per_row > 65535) return TKA_EINVAL;
  const dim3 small_grid((unsigned)p.segs_per_row, (unsigned)(p.num_segments / p.segs_per_row));
  LaunchTimer timer("select_small", stream);
  GemvParams none;
  memset(&none, 0, sizeof none);
  select_small_kernel<TKA_F16, false><<<small_grid, kSelThreads, lds, stream>>>(none, p);
  return hip_status(hipGetLastError());
}

// The same in one launch: every workgroup scores its own segment first (segments of up to select_small_max_len() rows).
int launch_gemv_select_small(const GemvParams& g, const SelectParams& p, int dtype, hipStream_t stream) {
  if (p.seg_len > kSmallMaxLen || p.k > kSmallMaxK || p.k > p.seg_len || !p.out_idx || p.union_idx) return TKA_EINVAL;
  const int lds = 2 * kSmallMaxLen * (int)sizeof(uint64_t);
  if (allow_dynamic_lds((const void*)select_small_kernel<TKA_F16, true>, lds) != TKA_OK ||
      allow_dynamic_lds((const void*)select_small_kernel<TKA_BF16, true>, lds) != TKA_OK)
    return TKA_EHIP;
  if (p.segs_per_row != g.num_chunks || p.num_segments != g.batch * g.num_kv_heads * g.num_chunks || p.num_segments / p.segs_per_row > 65535)
    return TKA_EINVAL;
  const dim3 small_grid((unsigned)p.segs_per_row, (unsigned)(p.num_segments / p.segs_per_row));
  LaunchTimer timer("gemv_select_small", stream);
  if (dtype == TKA_F16)
    select_small_kernel<TKA_F16, true><<<small_grid, kSelThreads, lds, stream>>>(g, p);
  else
    select_small_kernel<TKA_BF16, true><<<small_grid, kSelThreads, lds, stream>>>(g, p);
  return hip_status(hipGetLastError());
}

int launch_select(const SelectParams& p, hipStream_t stream) {
  int rc = launch_select_filter(p, stream);
  if (rc != TKA_OK) return rc;
  return launch_select_finalize(p, stream);
}

int launch_index_union(const UnionParams& p, hipStream_t stream) {
  if (p.seq_len <= kUnionBitmapMaxLen) {
    LaunchTimer timer("index_union", stream);
    if (p.seq_len <= 65536) index_union_bitmap_kernel<2><<<(unsigned)p.num_segments, kSelThreads, 0, stream>>>(p);
    else index_union_bitmap_kernel<8><<<(unsigned)p.num_segments, kSelThreads, 0, stream>>>(p);
    return hip_status(hipGetLastError());
  }
  const int kpad = kpad_for(p.k);
  const size_t lds = 2 * (size_t)kpad * sizeof(uint64_t);
  if (allow_dynamic_lds((const void*)index_union_kernel, 144 * 1024) != TKA_OK) return TKA_EHIP;
  LaunchTimer timer("index_union", stream);
  index_union_kernel<<<(unsigned)p.num_segments, kSelThreads, lds, stream>>>(p, kpad);
  return hip_status(hipGetLastError());
}

}  // namespace tka
