// Exact top-k of segments whose keys fit in the registers of one workgroup: W wavefronts per segment.
//
// The operator of the reference selects inside 2048-key chunks, one chunk per (batch entry, head, quarter of
// the sequence) (retrieval_attention.cu:335-354 sorts each chunk whole), so a call has hundreds to thousands of
// short segments; the centre-only selection (center_only_topk/gemv_topk.cu:251-279) has one of 1024 to 4096
// centroids per head.  Here the keys of a segment sit in the registers of W waves, EPT per lane:
//     W = 4,  EPT = 8        2048 keys     several segments in flight per compute unit
//     W = 8,  EPT = 8        4096 keys
//     W = 16, EPT = 8, 16    8192, 16384 keys (k up to 2048)
// and the whole selection is a few hundred instructions per wave with about eight barriers.  (A one-wave form,
// 32 keys per lane and no s_barrier at all, measured the same or slower from 256 to 16384 segments of 2048: what
// a launch of this kernel costs at a few hundred segments is mostly the first fetch of its instructions, so
// the form with less code per phase wins.  32 keys per lane in 16 waves, for 32768 keys, does not fit the 128
// registers a 1024-thread workgroup has: it spilled and was slower than the multi-launch path.)
//
//   1. fp32 scores -> order-preserving keys, relative to the smallest key of the segment and shifted so that the
//      largest one fills 32 bits;
//   2. one 11-bit histogram pass in LDS, suffix scans by DPP, the bin of the k-th largest.  If that bin is taken
//      whole, or holds at most 64 entries (they are ranked directly, one per lane), the selection is known -
//      ordinary data.  Otherwise up to two more passes over the remaining 11 and 10 bits of the key, and if the
//      threshold key itself is shared by more entries than are still needed, a scan in token order gives them
//      their rank among equals: lower index first;
//   3. the k selected composites are compacted into LDS (the histogram's space) and sorted with the bitonic
//      network of bitonic.hpp (registers, DPP, and LDS for the strides that cross waves); rank-ordered ids and
//      scores are written.  A caller that takes any order skips the sort.
#include "bitonic.hpp"
#include "kernels.hpp"

namespace tka {

namespace {

constexpr int kWsBins = 2048;
constexpr int kWsMaxWaves = 16;
constexpr int kWsMaxLen = kWsMaxWaves * kWave * 16;   // 16384 keys per segment at most

// (the same value in every lane: six DPP steps bring it to the last lane, one read hands it out)
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readlane((int)wave_min_in_last_lane(v), 63);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readlane((int)wave_max_in_last_lane(v), 63);
}

// The per-wave slots of a workgroup of W waves, combined by the first W lanes of every wave: one LDS read and log2(W)
// steps across the lanes instead of W reads per thread.  `lane` < `below` picks the slots that count (W: all of them).
template <int W>
__device__ __forceinline__ uint32_t ws_slots_sum(const uint32_t* slots, int lane, int from, int below) {
  uint32_t v = lane >= from && lane < below ? slots[lane < W ? lane : 0] : 0u;
  if (W > 1) v += lane_xor<1>(v);
  if (W > 2) v += lane_xor<2>(v);
  if (W > 4) v += lane_xor<4>(v);
  if (W > 8) v += lane_xor<8>(v);
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
}

// Order-preserving key of a score, as score_key() (NaN lowest, -0 == +0).
__device__ __forceinline__ uint32_t ws_key(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x + 0.0f);
  const uint32_t key = u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
  return x != x ? 0u : key;
}

// Most composites the sort buffer holds: 2048 for the 1024-thread form, else 1024 (the histogram's 8 KB).
constexpr int ws_max_k(int W) { return W >= 16 ? 2048 : 1024; }

// What the W waves of a segment share.
template <int W>
struct WsShared {
  __align__(16) uint32_t bins[2 * ws_max_k(W)];   // the histogram (2048 bins), then the sort buffer (composites)
  uint64_t cand[kWave];                           // entries of the threshold bucket when there are few
  uint64_t trash[W * kWave];                      // where a thread stores what is not selected
  uint32_t wave_a[kWsMaxWaves], wave_b[kWsMaxWaves];   // per-wave partial results
  uint32_t owner[4];                              // find_bin: owning thread, entries above its bins, entries in its bins
  uint64_t thr;                                   // the k-th largest composite, when one thread finds it
};

// Register e of thread t holds token (e / 4) * (256 W) + 4 t + e % 4: 16-byte loads, consecutive across threads.
// The part of it that does not depend on the thread:
__device__ __forceinline__ constexpr uint32_t ws_token_base(int e, int W) { return (uint32_t)((e >> 2) * (256 * W) + (e & 3)); }

template <int W>
__device__ __forceinline__ void ws_clear(uint32_t* bins, int tid) {
  constexpr int kPer = kWsBins / (W * kWave);   // words per thread
  if constexpr (kPer >= 4) {
#pragma unroll
    for (int i = 0; i < kPer / 4; ++i) *(u32x4*)(bins + (256 * W) * i + 4 * tid) = u32x4{0u, 0u, 0u, 0u};
  } else {
    *(u32x2*)(bins + 2 * tid) = u32x2{0u, 0u};
  }
}

// The bin d of the histogram with  count(bins > d) < need <= count(bins >= d);  `above` = count(bins > d),
// `cnt` = its own count.  The histogram must hold at least `need` entries.  Two levels: a thread sums its
// 2048 / (64 W) consecutive bins, suffix sums over the threads find the thread that owns d; then the first lanes of every
// wave take one of that thread's bins each and scan again.  All threads return the same values.
template <int W>
__device__ __forceinline__ void ws_find_bin(WsShared<W>& sh, uint32_t need, int tid, uint32_t& d, uint32_t& above, uint32_t& cnt) {
  constexpr int BPT = kWsBins / (W * kWave);   // bins per thread
  const int lane = tid & 63, wave = tid >> 6;
  uint32_t tot = 0;
  if constexpr (BPT >= 4) {
#pragma unroll
    for (int i = 0; i < BPT / 4; ++i) {
      const u32x4 v = *(const u32x4*)(sh.bins + BPT * tid + 4 * i);
      tot += (v[0] + v[1]) + (v[2] + v[3]);
    }
  } else {
    const u32x2 v = *(const u32x2*)(sh.bins + 2 * tid);
    tot = v[0] + v[1];
  }
  const uint32_t inc = wave_inclusive_scan(tot);
  const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
  uint32_t higher = wave_total - inc;            // entries in the bins of higher lanes of this wave
  if (lane == 0) sh.wave_a[wave] = wave_total;
  __syncthreads();
  higher += ws_slots_sum<W>(sh.wave_a, lane, wave + 1, W);   // the waves above
  if (higher < need && need <= higher + tot) {   // exactly one thread
    sh.owner[0] = (uint32_t)tid;
    sh.owner[1] = higher;
    sh.owner[2] = tot;
  }
  __syncthreads();
  const uint32_t owner = sh.owner[0], owner_higher = sh.owner[1], owner_tot = sh.owner[2];
  const uint32_t v = lane < BPT ? sh.bins[BPT * owner + lane] : 0u;
  const uint32_t vinc = wave_inclusive_scan(v);
  const uint32_t vhigher = owner_higher + (owner_tot - vinc);   // entries in bins above bin BPT*owner + lane
  const int bin = __builtin_ctzll(__ballot(lane < BPT && vhigher < need && need <= vhigher + v));
  d = (uint32_t)BPT * owner + (uint32_t)bin;
  above = (uint32_t)__builtin_amdgcn_readlane((int)vhigher, bin);
  cnt = (uint32_t)__builtin_amdgcn_readlane((int)v, bin);
}

// One radix pass below the first, among the entries that share the digits found so far: PASS 1 = key bits 20..10,
// PASS 2 = key bits 9..0.  `thr` is the threshold key so far (digits of later passes zero), `need` how many
// entries of the current bucket are still to be taken.  Returns true when the bucket found is taken whole.
template <int PASS, int W, int EPT>
__device__ __forceinline__ bool ws_pass(const uint32_t (&rel)[EPT], int tid, WsShared<W>& sh, uint32_t& thr, uint32_t& need) {
  __syncthreads();              // the previous histogram has been read
  ws_clear<W>(sh.bins, tid);
  __syncthreads();
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    bool active;
    uint32_t digit;
    if constexpr (PASS == 1) {
      active = (rel[e] >> 21) == (thr >> 21);
      digit = (rel[e] >> 10) & 2047u;
    } else {
      active = (rel[e] >> 10) == (thr >> 10);
      digit = rel[e] & 1023u;
    }
    if (active) atomicAdd(&sh.bins[digit], 1u);
  }
  __syncthreads();
  uint32_t d, above, cnt;
  ws_find_bin<W>(sh, need, tid, d, above, cnt);
  need -= above;
  thr |= PASS == 1 ? d << 10 : d;
  return cnt == need;
}

// Exclusive prefix of `mine` over the threads of the workgroup, and the total.  Two barriers (the first one lets
// the per-wave slots be reused right after an earlier call): every thread must call it.
template <int W>
__device__ __forceinline__ uint32_t ws_exclusive(uint32_t mine, int tid, WsShared<W>& sh, uint32_t* total = nullptr) {
  const int lane = tid & 63, wave = tid >> 6;
  const uint32_t inc = wave_inclusive_scan(mine);
  uint32_t pos = inc - mine;
  __syncthreads();
  if (lane == 63) sh.wave_a[wave] = inc;
  __syncthreads();
  pos += ws_slots_sum<W>(sh.wave_a, lane, 0, wave);   // the waves before
  if (total) *total = ws_slots_sum<W>(sh.wave_a, lane, 0, W);
  return pos;
}

// Order-preserving composite of an entry: (relative key << 32) | ~token.  Larger = earlier in the order
// (key descending, token ascending); all composites of a segment are distinct.
__device__ __forceinline__ uint64_t ws_composite(uint32_t rel, uint32_t not_token) { return ((uint64_t)rel << 32) | not_token; }

// The entries whose key equals the threshold key, when more of them exist than are still needed: the `need`
// with the lowest tokens are in.  Token order is (register group of four, thread, register in the group), so a
// scan over the threads per group of four registers ranks them; the thread that holds the need-th publishes its
// composite, which is the k-th largest of the segment, in sh.thr.
template <int W, int EPT>
__device__ __forceinline__ void ws_rank_equals(const uint32_t (&rel)[EPT], int tid, WsShared<W>& sh, uint32_t thr, uint32_t need) {
  const uint32_t not_t0 = ~(uint32_t)(4 * tid);
  uint32_t before = 0;
#pragma unroll
  for (int c = 0; c < EPT / 4; ++c) {
    uint32_t eq[4], mine = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      eq[r] = rel[4 * c + r] == thr ? 1u : 0u;
      mine += eq[r];
    }
    uint32_t total;
    uint32_t rank = before + ws_exclusive<W>(mine, tid, sh, &total);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (eq[r] && rank == need - 1u) sh.thr = ws_composite(thr, not_t0 - ws_token_base(4 * c + r, W));
      rank += eq[r];
    }
    before += total;
  }
}

// How many of the thread's entries satisfy PRED(relative key, ~token).
template <int W, int EPT, typename PRED>
__device__ __forceinline__ uint32_t ws_count(const uint32_t (&rel)[EPT], int tid, PRED pred) {
  const uint32_t not_t0 = ~(uint32_t)(4 * tid);
  uint32_t count[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < EPT; ++e) count[e & 3] += pred(rel[e], not_t0 - ws_token_base(e, W)) ? 1u : 0u;
  return (count[0] + count[1]) + (count[2] + count[3]);
}

// Stores the thread's entries that satisfy PRED to dst[pos ...] as composites.  Straight-line: the thread stores
// all its entries, the ones that do not qualify into its own trash slot.
template <int W, int EPT, typename PRED>
__device__ __forceinline__ void ws_scatter(const uint32_t (&rel)[EPT], int tid, uint64_t* dst, uint32_t pos, uint64_t* trash, PRED pred) {
  const uint32_t not_t0 = ~(uint32_t)(4 * tid);
  uint64_t* own = trash + tid;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t not_t = not_t0 - ws_token_base(e, W);   // ~token
    const bool take = pred(rel[e], not_t);
    uint64_t* at = take ? dst + pos : own;
    *at = ws_composite(rel[e], not_t);
    pos += take ? 1u : 0u;
  }
}

// The composites sh_sort[0 .. N) (zero past the k-th) into descending order, by the first N / E threads.
template <int N, int W>
__device__ __forceinline__ void ws_sort(uint64_t* sh_sort, int tid) {
  constexpr int T = W * kWave;
  constexpr int E = N > T ? N / T : 1;
  constexpr int NT = N / E;
  uint64_t v[E];
  const bool active = tid < NT;
  if (active) {
#pragma unroll
    for (int s = 0; s < E; ++s) v[s] = sh_sort[tid * E + s];
  }
  bitonic_net<N, E, 2, 1>(v, sh_sort, tid, active);   // (the exchange stages write the buffer only behind a barrier)
  __syncthreads();
  if (active) {
#pragma unroll
    for (int s = 0; s < E; ++s) sh_sort[tid * E + s] = v[s];
  }
}

template <int W, int EPT>
__global__ __launch_bounds__(W * kWave) void select_wave_kernel(SelectParams p, int kpad) {
  constexpr int T = W * kWave;
  constexpr int kMaxLen = T * EPT;
  __shared__ WsShared<W> sh;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int seg = blockIdx.x;
  const int n = (int)p.seg_len;
  const uint32_t k = (uint32_t)p.k;
  const float* sc = p.scores + (int64_t)seg * p.seg_stride;

  // Keys of the segment.  Entries past its end get the smallest relative key (0) and, by their position, lose
  // every tie against a real entry: they sit at the bottom of the order and k <= n keeps them out.
  constexpr uint32_t kPad = ~0u;   // marks them until then (no key is ~0: the largest is that of +inf)
  uint32_t rel[EPT];
  uint32_t kmin = ~0u, kmax = 0u;
  const bool vec = ((uintptr_t)sc & 15u) == 0;
  ws_clear<W>(sh.bins, tid);
#pragma unroll
  for (int c = 0; c < EPT / 4; ++c) {
    const int t0 = c * (4 * T) + 4 * tid;
    if (vec && (c + 1) * (4 * T) <= n) {             // a full group: no checks per entry
      const f32x4 w = *(const f32x4*)(sc + t0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const uint32_t key = ws_key(w[r]);
        rel[4 * c + r] = key;
        kmin = min(kmin, key);
        kmax = max(kmax, key);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool real = t0 + r < n;
        const uint32_t key = real ? ws_key(sc[t0 + r]) : kPad;
        rel[4 * c + r] = key;
        kmin = min(kmin, key);
        kmax = max(kmax, real ? key : 0u);
      }
    }
  }
  kmin = wave_min_u32(kmin);
  kmax = wave_max_u32(kmax);
  if (lane == 0) { sh.wave_a[wave] = kmin; sh.wave_b[wave] = kmax; }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < W; ++w) { kmin = min(kmin, sh.wave_a[w]); kmax = max(kmax, sh.wave_b[w]); }
  const uint32_t range = kmax - kmin;
  const int bits = range ? 32 - __builtin_clz(range) : 0;
  const int lshift = bits ? 32 - bits : 0;
  const bool padded = n < kMaxLen;
  if (padded && tid == 0) atomicAdd(&sh.bins[0], (uint32_t)(kMaxLen - n));   // the entries past the end, at once
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t r = (rel[e] - kmin) << lshift;
    const bool pad = padded && rel[e] == kPad;
    rel[e] = pad ? 0u : r;
    if (!pad) atomicAdd(&sh.bins[r >> 21], 1u);   // first pass: the leading 11 bits
  }
  __syncthreads();

  // The k-th largest composite T in the order (key, lower token first): selected are the entries >= T.  One pass
  // is enough when the bucket of the k-th is taken whole, or holds at most 64 entries: those are ranked
  // directly, one per lane.  Otherwise further passes fix the threshold key, and a scan ranks its equals.
  uint32_t d, above, cnt;
  ws_find_bin<W>(sh, k, tid, d, above, cnt);
  uint32_t need = k - above;
  uint64_t* sh_sort = (uint64_t*)sh.bins;
  // compaction of the entries that satisfy `pred` into dst
  auto compact = [&](uint64_t* dst, auto pred) {
    const uint32_t mine = ws_count<W, EPT>(rel, tid, pred);
    const uint32_t pos = ws_exclusive<W>(mine, tid, sh);     // (its barriers: every wave has read the histogram)
    ws_scatter<W, EPT>(rel, tid, dst, pos, sh.trash, pred);
  };
  uint64_t thr_c;
  if (cnt == need) {
    thr_c = ws_composite(d << 21, 0u);
  } else if (cnt <= (uint32_t)kWave) {
    compact(sh.cand, [d](uint32_t r, uint32_t) { return (r >> 21) == d; });
    __syncthreads();
    if (wave == 0) {
      // the bucket's entries, one per lane: the one beaten by exactly need - 1 others is the k-th largest
      const uint64_t c = lane < (int)cnt ? sh.cand[lane] : 0ull;
      uint32_t rank = 0;
      for (uint32_t j = 0; j < cnt; ++j) {
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)c, (int)j);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(c >> 32), (int)j);
        rank += (((uint64_t)hi << 32) | lo) > c ? 1u : 0u;
      }
      if (lane < (int)cnt && rank == need - 1u) sh.thr = c;
    }
    __syncthreads();
    thr_c = sh.thr;
  } else {
    uint32_t thr = d << 21;
    bool whole = false;     // the bucket of the threshold is taken whole
    if (bits > 11) whole = ws_pass<1, W, EPT>(rel, tid, sh, thr, need);      // (bits <= 11: that digit is 0 everywhere)
    if (!whole && bits > 22) whole = ws_pass<2, W, EPT>(rel, tid, sh, thr, need);
    if (whole) {
      thr_c = ws_composite(thr, 0u);
    } else {
      // `thr` is now a full key shared by more entries than the `need` still to be taken
      ws_rank_equals<W, EPT>(rel, tid, sh, thr, need);
      __syncthreads();
      thr_c = sh.thr;
    }
  }
  const uint32_t thr_hi = (uint32_t)(thr_c >> 32), thr_lo = (uint32_t)thr_c;
  auto selected = [thr_hi, thr_lo](uint32_t r, uint32_t not_t) { return r > thr_hi || (r == thr_hi && not_t >= thr_lo); };

  if (p.out_idx) {
    compact(sh_sort, selected);
    for (uint32_t r = k + tid; r < (uint32_t)kpad; r += T) sh_sort[r] = 0ull;
    __syncthreads();
    if (!p.unordered) {
      if (ws_max_k(W) >= 2048 && kpad == 2048) {
        ws_sort<ws_max_k(W) >= 2048 ? 2048 : 1024, W>(sh_sort, tid);
      } else {
        switch (kpad) {
          case 1024: ws_sort<1024, W>(sh_sort, tid); break;
          case 512: ws_sort<512, W>(sh_sort, tid); break;
          case 256: ws_sort<256, W>(sh_sort, tid); break;
          case 128: ws_sort<128, W>(sh_sort, tid); break;
          default: ws_sort<64, W>(sh_sort, tid); break;
        }
      }
      __syncthreads();
    }
    // out; the composites carry relative keys: key = (rel >> lshift) + kmin
    // (a modulo by a run-time value is some forty instructions on this hardware: none for one or a power of two of chunks)
    const uint32_t spr = (uint32_t)p.segs_per_row;
    const uint32_t chunk = spr == 1u ? 0u : (spr & (spr - 1u)) == 0u ? (uint32_t)seg & (spr - 1u) : (uint32_t)seg % spr;
    const uint32_t idx_base = p.seg_base_ids ? (uint32_t)(p.seg_base_ids[seg] * p.seg_len) : (uint32_t)(chunk * p.seg_len);
    int32_t* oi = p.out_idx + (int64_t)seg * p.out_stride;
    float* ov = p.out_val ? p.out_val + (int64_t)seg * p.out_stride : nullptr;
    for (uint32_t r = tid; r < k; r += T) {
      const uint64_t c = sh_sort[r];
      oi[r] = (int32_t)(~(uint32_t)c + idx_base);
      if (ov) ov[r] = key_score(((uint32_t)(c >> 32) >> lshift) + kmin);
    }
    if (p.out_expand) {
      int32_t* oe = p.out_expand + (int64_t)seg * p.k * p.expand;
      const uint32_t total = k * (uint32_t)p.expand;
      for (uint32_t e = tid; e < total; e += T) {
        const uint32_t jj = e / (uint32_t)p.expand, ii = e % (uint32_t)p.expand;
        oe[e] = (int32_t)(~(uint32_t)sh_sort[jj] * (uint32_t)p.expand + ii);
      }
    }
  }

  if (p.union_idx && p.union_handoff) {
    // The list only goes to the attention kernels, which take any order and skip -1: sink range [0, lo) and local
    // window [hi, n) first, then a place for each of the k selected tokens in the order of the threads (one scan instead
    // of one per group of four registers), holding -1 when the token lies inside the ranges, where it is listed already.
    const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
    const uint32_t hi = (uint32_t)(n - p.local > (int)lo ? n - p.local : (int)lo);
    const uint32_t edges = lo + ((uint32_t)n - hi);
    const int cap = p.k + p.sink + p.local;
    int32_t* uo = p.union_idx + (int64_t)seg * cap;
    const uint32_t mine = ws_count<W, EPT>(rel, tid, selected);
    uint32_t pos = edges + ws_exclusive<W>(mine, tid, sh);
    const uint32_t not_t0 = ~(uint32_t)(4 * tid);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const uint32_t not_t = not_t0 - ws_token_base(e, W);
      if (selected(rel[e], not_t)) {
        const uint32_t t = ~not_t;
        uo[pos++] = t >= lo && t < hi ? (int32_t)t : -1;
      }
    }
    for (uint32_t i = tid; i < edges; i += T) uo[i] = (int32_t)(i < lo ? i : hi + (i - lo));
    for (uint32_t i = edges + k + tid; i < (uint32_t)cap; i += T) uo[i] = -1;
    if (tid == 0) p.union_count[seg] = (int32_t)(edges + k);
  } else if (p.union_idx) {
    // ascending union with the sink range [0, lo) and the local window [hi, n): the selected tokens between them,
    // in token order (register group, thread, register), then the two ranges, -1 padding and the count
    const uint32_t lo = (uint32_t)(p.sink < n ? p.sink : n);
    const uint32_t hi = (uint32_t)(n - p.local > (int)lo ? n - p.local : (int)lo);
    const int cap = p.k + p.sink + p.local;
    int32_t* uo = p.union_idx + (int64_t)seg * cap;
    const uint32_t not_t0 = ~(uint32_t)(4 * tid);
    uint32_t run_mid = 0;
#pragma unroll
    for (int c = 0; c < EPT / 4; ++c) {
      uint32_t mid[4], mine = 0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const uint32_t not_t = not_t0 - ws_token_base(4 * c + r, W);
        const uint32_t t = ~not_t;
        mid[r] = selected(rel[4 * c + r], not_t) && t >= lo && t < hi ? 1u : 0u;
        mine += mid[r];
      }
      uint32_t total;
      uint32_t at = lo + run_mid + ws_exclusive<W>(mine, tid, sh, &total);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (mid[r]) uo[at++] = (int32_t)(c * (4 * T) + 4 * tid + r);
      }
      run_mid += total;
    }
    for (uint32_t t = tid; t < lo; t += T) uo[t] = (int32_t)t;
    const uint32_t mid_end = lo + run_mid;
    for (int t = (int)hi + tid; t < n; t += T) uo[mid_end + (uint32_t)(t - (int)hi)] = t;
    const uint32_t count = mid_end + (uint32_t)(n - (int)hi);
    for (int i = (int)count + tid; i < cap; i += T) uo[i] = -1;
    if (tid == 0) p.union_count[seg] = (int32_t)count;
  }
}

}  // namespace

int select_wave_max_len() { return kWsMaxLen; }
int select_wave_max_k(int64_t seg_len) { return seg_len > 8 * kWave * 8 ? ws_max_k(16) : ws_max_k(4); }

int launch_select_wave(const SelectParams& p, hipStream_t stream) {
  if (p.seg_len < 1 || p.seg_len > kWsMaxLen || p.k < 1 || p.k > p.seg_len || p.k > select_wave_max_k(p.seg_len) ||
      (!p.out_idx && !p.union_idx) || !p.scores)
    return TKA_EINVAL;
  int kpad = kWave;
  while (kpad < p.k) kpad <<= 1;
  LaunchTimer timer("select_wave", stream);
  const dim3 grid(p.num_segments);
#define TKA_LAUNCH_WS(W, EPT) hipLaunchKernelGGL((select_wave_kernel<W, EPT>), grid, dim3(W * kWave), 0, stream, p, kpad)
  if (p.seg_len <= 2048) TKA_LAUNCH_WS(4, 8);
  else if (p.seg_len <= 4096) TKA_LAUNCH_WS(8, 8);
  else if (p.seg_len <= 8192) TKA_LAUNCH_WS(16, 8);
  else TKA_LAUNCH_WS(16, 16);
#undef TKA_LAUNCH_WS
  return hip_status(hipGetLastError());
}

}  // namespace tka
