// Exact top-k of many short segments: one wavefront per segment, no workgroup barriers.
//
// The operator of the reference selects inside 2048-key chunks, one chunk per (batch entry, head, quarter of
// the sequence) (retrieval_attention.cu:335-354 sorts each chunk whole), so a call has thousands of short
// segments.  A 1024-thread workgroup per segment spends its time in barriers; here a segment belongs to one
// wave, whose 64 lanes hold its 2048 keys in registers (32 each), and a compute unit works on twenty
// segments at a time.
//
//   1. fp32 scores -> order-preserving keys, relative to the smallest key of the segment and shifted so that the
//      largest one fills 32 bits;
//   2. radix select, 11 bits per pass, on (key, 2047 - index): LDS histogram of the wave, suffix scan by DPP,
//      the bin of the k-th largest; passes end as soon as a bucket is taken whole.  Equal keys are told apart
//      by the last pass, whose digit is the index: lower index first;
//   3. the k selected composites are compacted into LDS (the histogram's space) and sorted by the wave with a
//      bitonic network; rank-ordered ids and scores are written.
#include "bitonic.hpp"
#include "kernels.hpp"

namespace tka {

namespace {
constexpr int kWsMaxLen = 2048;             // keys per segment at most
constexpr int kWsEpl = kWsMaxLen / kWave;   // keys per lane
constexpr int kWsBins = 2048;

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
  v = min(v, lane_xor<1>(v));
  v = min(v, lane_xor<2>(v));
  v = min(v, lane_xor<4>(v));
  v = min(v, lane_xor<8>(v));
  v = min(v, lane_xor<16>(v));
  v = min(v, lane_xor<32>(v));
  return v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, lane_xor<1>(v));
  v = max(v, lane_xor<2>(v));
  v = max(v, lane_xor<4>(v));
  v = max(v, lane_xor<8>(v));
  v = max(v, lane_xor<16>(v));
  v = max(v, lane_xor<32>(v));
  return v;
}

// Token of register e of a lane: 256-token groups, four consecutive tokens per lane in each (16-byte loads).
__device__ __forceinline__ int ws_token(int e, int lane) { return (e >> 2) * 256 + 4 * lane + (e & 3); }

// The bin d of the wave's histogram with  count(bins > d) < need <= count(bins >= d);  `above` = count(bins > d),
// `cnt` = its own count.  The histogram must hold at least `need` entries.  Two levels: lane l sums bins
// 32l .. 32l+31 and a suffix scan over the lanes finds the lane that owns d; then the first 32 lanes take one
// bin of that lane each and scan again.
__device__ __forceinline__ void ws_find_bin(const uint32_t* sh, uint32_t need, int lane, uint32_t& d, uint32_t& above, uint32_t& cnt) {
  uint32_t tot = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const u32x4 v = *(const u32x4*)(sh + 32 * lane + 4 * i);
    tot += (v[0] + v[1]) + (v[2] + v[3]);
  }
  const uint32_t inc = wave_inclusive_scan(tot);
  const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
  const uint32_t higher = total - inc;            // entries in the bins of higher lanes
  const int owner = __builtin_ctzll(__ballot(higher < need && need <= higher + tot));
  const uint32_t owner_higher = (uint32_t)__builtin_amdgcn_readlane((int)higher, owner);
  const uint32_t owner_tot = (uint32_t)__builtin_amdgcn_readlane((int)tot, owner);
  const uint32_t v = lane < 32 ? sh[32 * owner + lane] : 0u;
  const uint32_t vinc = wave_inclusive_scan(v);
  const uint32_t vhigher = owner_higher + (owner_tot - vinc);   // entries in bins above bin 32*owner + lane
  const int bin = __builtin_ctzll(__ballot(lane < 32 && vhigher < need && need <= vhigher + v));
  d = 32u * (uint32_t)owner + (uint32_t)bin;
  above = (uint32_t)__builtin_amdgcn_readlane((int)vhigher, bin);
  cnt = (uint32_t)__builtin_amdgcn_readlane((int)v, bin);
}

__device__ __forceinline__ void ws_clear(uint32_t* sh, int lane) {
#pragma unroll
  for (int i = 0; i < 8; ++i) *(u32x4*)(sh + 256 * i + 4 * lane) = u32x4{0u, 0u, 0u, 0u};
}

// One radix pass below the first.  PASS 1, 2: the second and third digit of the relative key (11 and 10 bits)
// among the entries that share the digits found so far; PASS 3: the digit is 2047 - token among the entries
// whose key equals the threshold key.  `thr` is the threshold so far (digits of later passes zero), `need` how
// many entries of the current bucket are still to be taken.  Returns true when the bucket found is taken whole.
template <int PASS>
__device__ __forceinline__ bool ws_pass(const uint32_t (&rel)[kWsEpl], int lane, uint32_t* sh, uint32_t& thr, uint32_t& need,
                                        uint32_t& tok_limit) {
  ws_clear(sh, lane);
  __syncthreads();
#pragma unroll
  for (int e = 0; e < kWsEpl; ++e) {
    bool active;
    uint32_t digit;
    if constexpr (PASS == 1) {
      active = (rel[e] >> 21) == (thr >> 21);
      digit = (rel[e] >> 10) & 2047u;
    } else if constexpr (PASS == 2) {
      active = (rel[e] >> 10) == (thr >> 10);
      digit = rel[e] & 1023u;
    } else {
      active = rel[e] == thr;
      digit = 2047u - (uint32_t)ws_token(e, lane);
    }
    if (active) atomicAdd(&sh[digit], 1u);
  }
  __syncthreads();
  uint32_t d, above, cnt;
  ws_find_bin(sh, need, lane, d, above, cnt);
  __syncthreads();
  need -= above;
  if constexpr (PASS == 1) thr |= d << 10;
  if constexpr (PASS == 2) thr |= d;
  if constexpr (PASS == 3) tok_limit = 2047u - d;
  return cnt == need;
}

// Order-preserving key of a score, as score_key() (NaN lowest, -0 == +0).
__device__ __forceinline__ uint32_t ws_key(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x + 0.0f);
  const uint32_t key = u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
  return x != x ? 0u : key;
}

// Compaction of the entries that satisfy PRED into `dst` (order-preserving composites (rel << 32) | ~token, lane
// after lane).  Straight-line: a count per lane, one scan, and every lane stores all its entries, the ones
// that do not qualify into its own slot of `trash`.
template <typename PRED>
__device__ __forceinline__ void ws_compact(const uint32_t (&rel)[kWsEpl], int lane, uint64_t* dst, uint64_t* trash, PRED pred) {
  const uint32_t not_t0 = ~(uint32_t)(4 * lane);
  uint32_t count[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < kWsEpl; ++e) {
    const uint32_t not_t = not_t0 - (uint32_t)((e >> 2) * 256 + (e & 3));   // ~token
    count[e & 3] += pred(rel[e], not_t) ? 1u : 0u;
  }
  const uint32_t mine = (count[0] + count[1]) + (count[2] + count[3]);
  uint32_t pos = wave_inclusive_scan(mine) - mine;
  uint64_t* own = trash + lane;
#pragma unroll
  for (int e = 0; e < kWsEpl; ++e) {
    const uint32_t not_t = not_t0 - (uint32_t)((e >> 2) * 256 + (e & 3));
    const bool take = pred(rel[e], not_t);
    uint64_t* at = take ? dst + pos : own;
    *at = ((uint64_t)rel[e] << 32) | not_t;
    pos += take ? 1u : 0u;
  }
}

// The selected composites (sh_sort[0 .. 64*E), zero past the k-th) into rank order.  Lane l takes elements
// l*E .. l*E+E-1; the bitonic network runs in registers (strides below E) and through DPP / ds_swizzle /
// ds_bpermute.
template <int E>
__device__ __forceinline__ void ws_sort(uint64_t* sh_sort, int lane) {
  uint64_t v[E];
#pragma unroll
  for (int s = 0; s < E; ++s) v[s] = sh_sort[lane * E + s];
  bitonic_net<64 * E, E, 2, 1>(v, nullptr, lane, true);
  __syncthreads();
#pragma unroll
  for (int s = 0; s < E; ++s) sh_sort[lane * E + s] = v[s];
}

__global__ __launch_bounds__(kWave) void select_wave_kernel(SelectParams p, int kpad) {
  __shared__ __align__(16) uint32_t sh[kWsBins];   // the histogram, then the sort buffer (1024 composites)
  __shared__ uint64_t sh_cand[kWave];              // entries of the threshold bucket when there are few
  __shared__ uint64_t sh_trash[kWave];             // where a lane stores what is not selected
  const int lane = threadIdx.x;
  const int seg = blockIdx.x;
  const int n = (int)p.seg_len;
  const uint32_t k = (uint32_t)p.k;
  const float* sc = p.scores + (int64_t)seg * p.seg_stride;

  // Keys of the segment.  Entries past its end get the smallest relative key (0) and, by their position, lose
  // every tie against a real entry: they sit at the bottom of the order and k <= n keeps them out.
  constexpr uint32_t kPad = ~0u;   // marks them until then (no key is ~0: the largest is that of +inf)
  uint32_t rel[kWsEpl];
  uint32_t kmin = ~0u, kmax = 0u;
  const bool vec = ((uintptr_t)sc & 15u) == 0;
  ws_clear(sh, lane);
#pragma unroll
  for (int c = 0; c < kWsEpl / 4; ++c) {
    const int t0 = c * 256 + 4 * lane;
    if (vec && c * 256 + 256 <= n) {             // a full group: no checks per entry
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
  const uint32_t range = kmax - kmin;
  const int bits = range ? 32 - __builtin_clz(range) : 0;
  const int lshift = bits ? 32 - bits : 0;
  __syncthreads();
  const bool padded = n < kWsMaxLen;
#pragma unroll
  for (int e = 0; e < kWsEpl; ++e) {
    const uint32_t r = (rel[e] - kmin) << lshift;
    rel[e] = padded && rel[e] == kPad ? 0u : r;
    atomicAdd(&sh[rel[e] >> 21], 1u);   // first pass: the leading 11 bits
  }
  __syncthreads();

  // The k-th largest entry in the order (key, lower token first).  One pass is enough when the bucket of the
  // k-th is taken whole, or holds at most 64 entries: those are ranked directly, one per lane.  Otherwise
  // further passes fix the threshold (thr, tok_limit): selected are the entries with
  // (rel, 2047 - token) >= (thr, 2047 - tok_limit).
  uint32_t d, above, cnt;
  ws_find_bin(sh, k, lane, d, above, cnt);
  __syncthreads();
  uint32_t need = k - above;
  uint64_t* sh_sort = (uint64_t*)sh;
  const bool rank_bucket = cnt != need && cnt <= (uint32_t)kWave;
  if (cnt == need) {
    ws_compact(rel, lane, sh_sort, sh_trash, [d](uint32_t r, uint32_t) { return (r >> 21) >= d; });
  } else if (rank_bucket) {
    ws_compact(rel, lane, sh_sort, sh_trash, [d](uint32_t r, uint32_t) { return (r >> 21) > d; });
    ws_compact(rel, lane, sh_cand, sh_trash, [d](uint32_t r, uint32_t) { return (r >> 21) == d; });
  } else {
    uint32_t thr = d << 21, tok_limit = 2047u;
    bool done = false;
    if (bits > 11) done = ws_pass<1>(rel, lane, sh, thr, need, tok_limit);
    if (!done && bits > 22) done = ws_pass<2>(rel, lane, sh, thr, need, tok_limit);
    if (!done) ws_pass<3>(rel, lane, sh, thr, need, tok_limit);
    const uint64_t thr43 = ((uint64_t)thr << 11) | (2047u - tok_limit);
    ws_compact(rel, lane, sh_sort, sh_trash, [thr43](uint32_t r, uint32_t not_t) {
      return (((uint64_t)r << 11) | (not_t & 2047u)) >= thr43;   // (~token & 2047 == 2047 - token)
    });
  }
  for (uint32_t r = k + lane; r < (uint32_t)kpad; r += kWave) sh_sort[r] = 0ull;
  __syncthreads();
  if (rank_bucket) {
    // `cnt` entries of the threshold bucket, one per lane: an entry beaten by fewer than `need` others is in
    const uint64_t c = lane < (int)cnt ? sh_cand[lane] : 0ull;
    uint32_t rank = 0;
    for (uint32_t j = 0; j < cnt; ++j) {
      const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)c, (int)j);
      const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(c >> 32), (int)j);
      rank += (((uint64_t)hi << 32) | lo) > c ? 1u : 0u;
    }
    if (lane < (int)cnt && rank < need) sh_sort[above + rank] = c;
    __syncthreads();
  }

  const uint32_t idx_base = p.seg_base_ids ? (uint32_t)(p.seg_base_ids[seg] * p.seg_len)
                                           : (uint32_t)((seg % p.segs_per_row) * p.seg_len);
  int32_t* oi = p.out_idx + (int64_t)seg * p.out_stride;
  float* ov = p.out_val ? p.out_val + (int64_t)seg * p.out_stride : nullptr;
  if (!p.unordered) {
    switch (kpad) {
      case 1024: ws_sort<16>(sh_sort, lane); break;
      case 512: ws_sort<8>(sh_sort, lane); break;
      case 256: ws_sort<4>(sh_sort, lane); break;
      case 128: ws_sort<2>(sh_sort, lane); break;
      default: ws_sort<1>(sh_sort, lane); break;
    }
    __syncthreads();
  }
  // out; the composites carry relative keys: key = (rel >> lshift) + kmin
  for (uint32_t r = lane; r < k; r += kWave) {
    const uint64_t c = sh_sort[r];
    oi[r] = (int32_t)(~(uint32_t)c + idx_base);
    if (ov) ov[r] = key_score(((uint32_t)(c >> 32) >> lshift) + kmin);
  }
  if (p.out_expand) {
    int32_t* oe = p.out_expand + (int64_t)seg * p.k * p.expand;
    const uint32_t total = k * (uint32_t)p.expand;
    for (uint32_t e = lane; e < total; e += kWave) {
      const uint32_t jj = e / (uint32_t)p.expand, ii = e % (uint32_t)p.expand;
      oe[e] = (int32_t)(~(uint32_t)sh_sort[jj] * (uint32_t)p.expand + ii);
    }
  }
}

}  // namespace

int select_wave_max_len() { return kWsMaxLen; }
int select_wave_max_k() { return kWsBins / 2; }

int launch_select_wave(const SelectParams& p, hipStream_t stream) {
  if (p.seg_len < 1 || p.seg_len > kWsMaxLen || p.k < 1 || p.k > p.seg_len || p.k > kWsBins / 2 || !p.out_idx || !p.scores)
    return TKA_EINVAL;
  int kpad = kWave;
  while (kpad < p.k) kpad <<= 1;
  LaunchTimer timer("select_wave", stream);
  hipLaunchKernelGGL(select_wave_kernel, dim3(p.num_segments), dim3(kWave), 0, stream, p, kpad);
  return hip_status(hipGetLastError());
}

}  // namespace tka
