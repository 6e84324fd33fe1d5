// Selection and gathered attention of a long segment in ONE launch: the select -> attention hand-off stays on chip.
//
// After the candidate GEMV (gemv_scores.hip) a segment's tokens at or above its sampled threshold lie in slices of
// 512 tokens (format: GemvParams::cand).  The decode step whose caller only wants the attention output does not
// need the selected ids anywhere in memory, so every attention workgroup of a (batch entry, KV head) takes the
// segment's candidates (a few thousand composites: 64 KB of slice heads, served by the L2) into LDS, finds the k-th
// largest composite by the radix passes of the selection kernel, and keeps the part of the token list that is its
// split's: sink range, selected tokens between the ranges in the order of LDS, local window.  The ids go to
// LDS and the matrix-core attention starts at once (the reference keeps the ids in shared memory between its top-k and
// its attention in the same way, baseline_2.cu:583-1058, ids at :824-834).  Every workgroup of a segment derives the
// same threshold from the same candidates, so nobody waits for anybody; what the splits compute twice is a few
// microseconds of LDS histogram work, against a launch, a list written and read, and the round trips of a kernel of
// one workgroup per segment.
//
// A segment whose candidates cannot be used (fewer than k, more than the selection accepts, a slice whose streaming
// workgroup gave up waiting for the threshold) is left out here: its splits write empty partials and the segment is
// flagged in seg_flags; the combine launch that follows redoes it from the keys (redo role of lse_combine_redo_kernel).
#include "attention_mfma.hpp"

namespace tka {

namespace {

using namespace mfma_attn;

constexpr int kSelSmallBucket = 64;   // a threshold bucket of this many entries or fewer is ranked by every wave directly

// Finds the bin d with  count(bins > d) < need <= count(bins >= d)  in sh_hist[2048]; every one of the 256 threads
// must call it, behind a barrier that completes the histogram.  sh_res[0] = d, [1] = count(bins > d), [2] = sh_hist[d].
__device__ __forceinline__ void find_threshold_bin_256(const uint32_t* sh_hist, uint32_t need, uint32_t* sh_wtot, uint32_t* sh_res) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  constexpr int kBins = kHistBins / kThreads;   // 8 bins per thread
  uint32_t h[kBins], mine = 0;
  {
    const u32x4 a = *(const u32x4*)&sh_hist[kBins * tid], b = *(const u32x4*)&sh_hist[kBins * tid + 4];
#pragma unroll
    for (int e = 0; e < 4; ++e) { h[e] = a[e]; h[4 + e] = b[e]; }
  }
#pragma unroll
  for (int e = 0; e < kBins; ++e) mine += h[e];
  const uint32_t inc = wave_inclusive_scan(mine);
  const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
  const uint32_t v = wave_total - inc + mine;   // this wave's count in the bins of threads >= tid
  if (lane == 0) sh_wtot[wave] = wave_total;
  __syncthreads();
  uint32_t above = 0;
  for (int w = wave + 1; w < kWaves; ++w) above += sh_wtot[w];
  const uint32_t ge = above + v;                // count(bins >= 8 tid)
  if (ge >= need && ge - mine < need) {         // the bin is one of this thread's: walk them from the top
    uint32_t a = ge - mine;
    bool found = false;
#pragma unroll
    for (int e = kBins - 1; e >= 0; --e) {
      if (!found && a + h[e] >= need) { sh_res[0] = (uint32_t)(kBins * tid + e); sh_res[1] = a; sh_res[2] = h[e]; found = true; }
      if (!found) a += h[e];
    }
  }
  __syncthreads();
}

// Sum of v over the 256 threads (every thread gets it) and the exclusive prefix of this thread.  Two barriers.
__device__ __forceinline__ uint32_t block_scan_256(uint32_t v, uint32_t* sh_wtot, uint32_t* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t inc = wave_inclusive_scan(v);
  __syncthreads();   // sh_wtot may still be read
  if (lane == 63) sh_wtot[wave] = inc;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const uint32_t t = sh_wtot[w];
    before += w < wave ? t : 0u;
    all += t;
  }
  *total = all;
  return before + inc - v;
}

// L lanes per slice ask for its first 2 L entries (16 bytes a lane: whole lines per slice), R slices per lane group, all
// R loads in flight together: one round trip for up to R * 256 / L slices.
// Dynamic LDS: f.lds_entries composites (the candidates; what does not fit is read again from memory by every pass),
// then f.parts + 1 words (where every slice's candidates start); behind the selection the partial results of the
// attention take the place of the composites.
template <int DT, int G, int L, int R>
__global__ __launch_bounds__(kThreads) void attn_select_mfma_kernel(AttnParams p, FusedSelectParams f) {
  constexpr int E = 2 * L;                    // entries of a slice that the round trip brings
  constexpr int kGroups = kThreads / L;       // slices per round
  static_assert(E <= kCandHead, "entries of the slice heads");
  // histogram of a radix pass; afterwards the tokens of this split (p.tokens_per_split ids)
  __shared__ __attribute__((aligned(16))) uint32_t sh_hist[kHistBins];
  __shared__ uint32_t sh_wtot[2 * kWaves];
  __shared__ uint32_t sh_res[4];
  __shared__ uint64_t sh_small[kSelSmallBucket];
  __shared__ uint32_t sh_small_cnt;
  extern __shared__ __attribute__((aligned(16))) unsigned char sh_dyn[];
  uint64_t* sh_ent = (uint64_t*)sh_dyn;
  uint32_t* sh_pos = (uint32_t*)(sh_ent + f.lds_entries);   // [parts + 1]
  int32_t* sh_ids = (int32_t*)sh_hist;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  // The workgroups of a launch go to the eight XCDs in turn.  All splits of a segment read the same 64 KB of slice
  // heads, so they are given numbers that put them on ONE XCD, whose L2 then fetches those heads once (with the splits
  // of a segment spread over all XCDs every L2 fetched the heads of every segment, and the copy below took 2 us longer).
  int split, seg32;
  {
    const uint32_t id = blockIdx.x, S = (uint32_t)p.num_splits, segs = (uint32_t)(p.batch * p.num_kv_heads);
    if ((segs & 7u) == 0u) {
      const uint32_t x = id & 7u, r = id >> 3;
      seg32 = (int)(8u * (r / S) + x);
      split = (int)(r % S);
    } else {
      seg32 = (int)(id / S);
      split = (int)(id % S);
    }
  }
  const int h = seg32 % p.num_kv_heads, b = seg32 / p.num_kv_heads;
  const int64_t seg = seg32;
  const uint32_t k = (uint32_t)f.k;
  const uint64_t* heads = f.cand_head + seg * f.parts * kCandHead;
  const uint64_t* lists = f.cand + seg * f.cand_seg_stride;
  const uint32_t cap = (uint32_t)f.lds_entries;
  const int parts = f.parts;

  // ---- the segment's candidates into LDS as composites (key << 32 | ~token), slice after slice.  Entry 0 of a slice
  // carries its count; entries past the count are older contents of the workspace and never looked at.
  uint32_t n_entries, n_gave_up;
  uint32_t kmin = ~0u, kmax = 0u;   // smallest and largest key among the candidates this thread has seen
  {
    const int sub = tid & (L - 1), grp = tid / L;
    u32x4 raw[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int s = r * kGroups + grp;
      raw[r] = *(const u32x4*)(heads + (int64_t)(s < parts ? s : 0) * kCandHead + 2 * sub);
    }
    for (int i = tid; i < kHistBins; i += kThreads) sh_hist[i] = 0;
    if (tid == 0) sh_small_cnt = 0;
    uint32_t cnt[R];
    uint32_t gave_up = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int s = r * kGroups + grp;
      uint32_t c = ((uint32_t)__shfl((int)raw[r][0], lane & ~(L - 1), 64) >> 9) & 0x3ffu;   // entry 0 sits in the group's first lane
      if (s >= parts) c = 0;
      if (c == kSliceGaveUp) { c = 0; gave_up += sub == 0 ? 1u : 0u; }
      cnt[r] = c;
      if (sub == 0 && s < parts) sh_pos[s] = c;
    }
    __syncthreads();
    // where every slice starts: thread t adds up slices t * spt .. and the threads are scanned
    const int spt = (parts + kThreads - 1) / kThreads;
    uint32_t mine = 0;
    for (int i = 0; i < spt; ++i) {
      const int s = tid * spt + i;
      mine += s < parts ? sh_pos[s] : 0u;
    }
    // (counts and given-up slices in one scan: at most 4096 slices of at most 512 candidates; a sum that runs into the
    // upper field reads as slices given up, and the segment is redone, which is what such a count asks for anyway)
    uint32_t run = block_scan_256(mine | (gave_up << 22), sh_wtot, &n_entries) & 0x3fffffu;
    n_gave_up = n_entries >> 22;
    n_entries &= 0x3fffffu;
    for (int i = 0; i < spt; ++i) {
      const int s = tid * spt + i;
      if (s < parts) {
        const uint32_t c = sh_pos[s];
        sh_pos[s] = run;
        run += c;
      }
    }
    if (tid == kThreads - 1) sh_pos[parts] = n_entries;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int s = r * kGroups + grp;
      const uint32_t start = sh_pos[s < parts ? s : 0], idx0 = (uint32_t)s * (uint32_t)f.part_len;
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const uint32_t e = 2u * (uint32_t)sub + (uint32_t)x;
        if (e < cnt[r]) {
          kmin = min(kmin, raw[r][2 * x + 1]);
          kmax = max(kmax, raw[r][2 * x + 1]);
          if (start + e < cap) sh_ent[start + e] = ((uint64_t)raw[r][2 * x + 1] << 32) | (uint32_t)~(idx0 + (raw[r][2 * x] & 0x1ffu));
        }
      }
    }
  }
  // candidate j of slice s, read from memory
  auto load_entry = [&](uint32_t s, uint32_t j) -> uint64_t {
    const uint64_t w = j < (uint32_t)kCandHead ? heads[(int64_t)s * kCandHead + j] : lists[(int64_t)s * f.part_len + j];
    return (w & 0xffffffff00000000ull) | (uint32_t)~(s * (uint32_t)f.part_len + ((uint32_t)w & 0x1ffu));
  };
  // what the round trip above did not bring (a slice with more than E candidates: heavy ties, or scores that cluster)
#pragma unroll 1
  for (int s = tid; s < parts; s += kThreads) {
    const uint32_t start = sh_pos[s], c = sh_pos[s + 1] - start;
#pragma unroll 1
    for (uint32_t j = E; j < c; ++j) {
      const uint64_t w = load_entry((uint32_t)s, j);
      kmin = min(kmin, (uint32_t)(w >> 32));
      kmax = max(kmax, (uint32_t)(w >> 32));
      if (start + j < cap) sh_ent[start + j] = w;
    }
  }

  const bool redo = n_entries < k || n_entries > (uint32_t)f.max_entries || n_gave_up != 0u;
  if (split == 0) {
    if (tid == 0) f.seg_flags[seg] = (redo ? 1u : 0u) | (n_gave_up << 8);
    // the threshold and the arrival flags are spent: a replay of the same launches (a captured graph) must not take
    // them for its own
    if (tid >= 64 && tid < 128) f.sample_flags[seg * 64 + (tid - 64)] = 0u;
    if (tid == 0) f.tau_words[2 * seg] = 0ull;
  }
  if (redo) {
    // empty partials (a split with l == 0 contributes nothing); the combine launch redoes the segment from the keys
    if (tid < G) {
      const int64_t slot = (seg * G + tid) * p.num_splits + split;
      p.part_m[slot] = -INFINITY;
      p.part_l[slot] = 0.0f;
    }
    return;
  }
  __syncthreads();

  // A pass over all candidates: those in LDS in a rolled loop, and, when the segment has more than LDS holds (the
  // whole workgroup knows), the rest of this thread's slices from memory.
  const uint32_t n_lds = n_entries < cap ? n_entries : cap;
  auto for_each_late = [&](auto&& fn) {   // the candidates beyond LDS, slice by slice (slow; segments with very many candidates only)
#pragma unroll 1
    for (int s = tid; s < parts; s += kThreads) {
      const uint32_t start = sh_pos[s], c = sh_pos[s + 1] - start;
#pragma unroll 1
      for (uint32_t j = start >= cap ? 0u : min(c, cap - start); j < c; ++j) fn(load_entry((uint32_t)s, j));
    }
  };
  auto for_each_entry = [&](auto&& fn) {   // (four reads in flight: a pass is a handful of trips to LDS)
#pragma unroll 1
    for (uint32_t v = tid; v < n_lds; v += 4 * kThreads) {
      uint64_t c[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] = sh_ent[v + u * kThreads < n_lds ? v + u * kThreads : v];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (v + u * kThreads < n_lds) fn(c[u]);
    }
    if (n_entries > cap) for_each_late(fn);
  };

  // ---- the k-th largest composite: radix passes relative to the smallest key (as select_finalize_cand_kernel)
  uint64_t threshold = 0;   // selected: composite >= threshold
  if (n_entries > k) {
    kmin = wave_min_in_last_lane(kmin);
    kmax = wave_max_in_last_lane(kmax);
    if (lane == 63) { sh_wtot[kWaves + wave] = kmin; sh_wtot[wave] = kmax; }
    __syncthreads();
    kmin = sh_wtot[kWaves];
    kmax = sh_wtot[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) { kmin = min(kmin, sh_wtot[kWaves + w]); kmax = max(kmax, sh_wtot[w]); }
    __syncthreads();
    const uint64_t base = (uint64_t)kmin << 32;
    int fixed = kmin == kmax ? 32 : __builtin_clz(kmax - kmin);
    uint64_t prefix = 0ull;
    uint32_t need = k;
    bool done = false, first_pass = true;
    while (!done) {
      const int bits = (64 - fixed) >= kHistBits ? kHistBits : (64 - fixed);
      const int shift = 64 - fixed - bits;
      if (!first_pass) {
        for (int i = tid; i < kHistBins; i += kThreads) sh_hist[i] = 0;
        __syncthreads();
      }
      first_pass = false;
      for_each_entry([&](uint64_t c0) {
        const uint64_t c = c0 - base;
        if (fixed == 0 || (c >> (64 - fixed)) == prefix) atomicAdd(&sh_hist[(uint32_t)(c >> shift) & ((1u << bits) - 1u)], 1u);
      });
      __syncthreads();
      find_threshold_bin_256(sh_hist, need, sh_wtot, sh_res);
      const uint32_t d = sh_res[0], gt = sh_res[1], in_bin = sh_res[2];
      need -= gt;
      prefix = (prefix << bits) | d;
      fixed += bits;
      if (in_bin == need || fixed == 64) {
        threshold = fixed == 64 ? prefix : (prefix << (64 - fixed));
        done = true;
      } else if (in_bin <= (uint32_t)kSelSmallBucket) {
        // few entries left in the threshold bucket: every wave ranks them and picks the need-th largest
        for_each_entry([&](uint64_t c0) {
          const uint64_t c = c0 - base;
          if ((c >> (64 - fixed)) == prefix) sh_small[atomicAdd(&sh_small_cnt, 1u)] = c;
        });
        __syncthreads();
        const uint64_t e = (uint32_t)lane < in_bin ? sh_small[lane] : 0ull;
        uint32_t greater = 0;
        for (uint32_t jj = 0; jj < in_bin; ++jj) {   // (the others come from the lanes' registers, not from LDS again)
          const uint64_t o = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(e >> 32), (int)jj) << 32) |
                             (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)e, (int)jj);
          greater += o > e ? 1u : 0u;
        }
        const uint64_t hit = __ballot((uint32_t)lane < in_bin && greater == need - 1u);
        threshold = __shfl(e, (int)__builtin_ctzll(hit), 64);
        done = true;
      }
      __syncthreads();   // sh_res and the histogram are read
    }
    threshold += base;
  }

  // ---- this split's part of the token list: [0, lo) ++ selected tokens of [lo, hi) in the order of LDS ++ [hi, n)
  const int64_t n = p.seq_len;
  const uint32_t lo = (uint32_t)(f.sink < n ? f.sink : n);
  const uint32_t hi = (uint32_t)(n - f.local > lo ? n - f.local : lo);
  // thread t takes a contiguous run of the entries in LDS (and the entries beyond LDS of slices t, t + 256, .. behind all of them)
  const uint32_t per = (n_lds + kThreads - 1) / kThreads;
  const uint32_t v0 = min((uint32_t)tid * per, n_lds), v1 = min(v0 + per, n_lds);
  auto is_mid = [&](uint64_t c) {
    const uint32_t t = ~(uint32_t)c;
    return c >= threshold && t >= lo && t < hi;
  };
  uint32_t my_mid = 0, my_late = 0;
  uint64_t mid_mask = 0;   // (a run has at most 16384 / 256 = 64 entries)
#pragma unroll 1
  for (uint32_t v = v0; v < v1; v += 4) {
    uint64_t c[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) c[u] = sh_ent[v + u < v1 ? v + u : v];
#pragma unroll
    for (int u = 0; u < 4; ++u) mid_mask |= (uint64_t)(v + u < v1 && is_mid(c[u]) ? 1u : 0u) << ((v + u - v0) & 63u);
  }
  my_mid = (uint32_t)__popcll(mid_mask);
  if (n_entries > cap) for_each_late([&](uint64_t c) { my_late += is_mid(c) ? 1u : 0u; });
  uint32_t totals;
  const uint32_t ex = block_scan_256(my_mid | (my_late << 16), sh_wtot, &totals);   // (each total is at most 16384)
  const uint32_t total_mid = (totals & 0xffffu) + (totals >> 16);
  const uint32_t list_len = lo + total_mid + (uint32_t)(n - hi);
  const uint32_t begin = (uint32_t)split * (uint32_t)p.tokens_per_split;
  const uint32_t end = min(list_len, begin + (uint32_t)p.tokens_per_split);
  __syncthreads();   // the histogram is spent: its memory takes the ids
  {
    uint32_t pos = lo + (ex & 0xffffu);
    if (pos < end && pos + my_mid > begin) {
#pragma unroll 1
      for (uint64_t m = mid_mask; m != 0ull; m &= m - 1ull, ++pos)
        if (pos >= begin && pos < end) sh_ids[pos - begin] = (int32_t)~(uint32_t)sh_ent[v0 + (uint32_t)__builtin_ctzll(m)];
    }
    pos = lo + (totals & 0xffffu) + (ex >> 16);
    if (n_entries > cap && pos < end && pos + my_late > begin) {
      for_each_late([&](uint64_t c) {
        if (is_mid(c)) {
          if (pos >= begin && pos < end) sh_ids[pos - begin] = (int32_t)~(uint32_t)c;
          ++pos;
        }
      });
    }
  }
  for (uint32_t v = begin + (uint32_t)tid; v < end; v += kThreads) {
    if (v < lo) sh_ids[v - begin] = (int32_t)v;
    else if (v >= lo + total_mid) sh_ids[v - begin] = (int32_t)(hi + (v - lo - total_mid));
  }
  __syncthreads();   // the ids are written; the candidates are spent: their memory takes the partial results

  attend<DT, G, true>(p, sh_ids, 0, begin < end ? (int64_t)(end - begin) : 0, b, h, split, *(AttendLds<G>*)sh_dyn);
}

template <int DT, int G, int L, int R>
int launch_one(const AttnParams& p, const FusedSelectParams& f, dim3 grid, size_t lds, hipStream_t stream) {
  if (lds > 48 * 1024 && allow_dynamic_lds((const void*)attn_select_mfma_kernel<DT, G, L, R>, 144 * 1024) != TKA_OK) return TKA_EHIP;
  attn_select_mfma_kernel<DT, G, L, R><<<grid, kThreads, lds, stream>>>(p, f);
  return hip_status(hipGetLastError());
}

template <int DT, int G>
int launch_ns(const AttnParams& p, const FusedSelectParams& f, dim3 grid, size_t lds, hipStream_t stream) {
  return launch_one<DT, G, 16, 16>(p, f, grid, lds, stream);   // up to 256 slices: one round trip brings all their heads
}

template <int DT>
int launch_g(const AttnParams& p, const FusedSelectParams& f, dim3 grid, size_t lds, hipStream_t stream) {
  switch (p.group) {
    case 2: return launch_ns<DT, 2>(p, f, grid, lds, stream);
    case 4: return launch_ns<DT, 4>(p, f, grid, lds, stream);
    case 8: return launch_ns<DT, 8>(p, f, grid, lds, stream);
    default: return TKA_EUNSUPPORTED;
  }
}

}  // namespace

// Segments of up to 256 slices (131072 tokens).  Longer ones keep the selection launch: with 2048 slices (a million tokens)
// the splits of a segment, each reading all of its slice heads, took 35.7 us against 29.8 for the two launches.
bool attn_select_fits(int parts, int group) { return parts <= 256 && (group == 2 || group == 4 || group == 8); }

// p.kv_idx / p.kv_count are not used: the token list of a split exists in LDS only.  p.tokens_per_split ids per workgroup
// (at most 2048: they take the place of the histogram).
int launch_attn_select_mfma(const AttnParams& p, const FusedSelectParams& f0, int dtype, hipStream_t stream) {
  if (!attn_select_fits(f0.parts, p.group) || p.tokens_per_split < 1 || p.tokens_per_split > kHistBins ||
      (int64_t)p.num_splits * p.num_kv_heads * p.batch > 0x7fffffffLL)
    return TKA_EINVAL;
  FusedSelectParams f = f0;
  // Candidates kept in LDS: room for two workgroups per CU (68 KB of composites beside the 9 KB of fixed arrays: twice
  // the candidates that a segment of 131072 tokens brings for k = 2048), and all 16384 that the selection accepts when
  // the launch has no more workgroups than CUs.
  const int64_t wgs = (int64_t)p.num_splits * p.num_kv_heads * p.batch;
  int entries = wgs > 256 ? 8704 : 16384;
  const int floor_entries = (int)((sizeof(AttendLds<8>) + 7) / 8);   // the partial results of the attention lie in the same place
  if (entries < floor_entries) entries = floor_entries;
  f.lds_entries = entries;
  const dim3 grid((unsigned)wgs);
  const size_t lds = (size_t)entries * sizeof(uint64_t) + (size_t)(f.parts + 1) * sizeof(uint32_t);
  LaunchTimer timer("attn_select_mfma", stream);
  return dtype == TKA_F16 ? launch_g<TKA_F16>(p, f, grid, lds, stream) : launch_g<TKA_BF16>(p, f, grid, lds, stream);
}

}  // namespace tka
