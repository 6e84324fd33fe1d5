// Shared device helpers for the gfx950 kernels: 16-bit element widening, DPP / ds_swizzle lane
// exchanges for wave64, the order-preserving score key, and host-side launch bookkeeping.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/topk_attn.h"

namespace tka {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kHeadDim = TKA_HEAD_DIM;
constexpr int kWave = 64;
constexpr int kHistBits = 11;
constexpr int kHistBins = 1 << kHistBits;  // first-level selection histogram: top 11 bits of the key
constexpr int kGemvDenseTokensPerWg = 256; // tokens per workgroup of the dense GEMV on large problems
constexpr int kGemvCandTokensPerWg = 512;  // tokens (and threads) per streaming workgroup of the candidate GEMV = slice length
constexpr int64_t kFusedMaxSegLen = 2048;   // segments up to this length are scored and selected by one workgroup in one launch
constexpr int kGemvInlineCentres = 256;     // centroids per head that the GEMV launch of a two-level selection ranks itself
constexpr int64_t kCandMinSegLen = 32768;   // shorter segments never take the candidate mode
constexpr int64_t kCandMinRows = 1 << 20;   // ... nor do segments below 65536 tokens unless the call has this many rows
constexpr int kCandHead = 32;               // first candidates of a slice, kept in a compact array of their own (see GemvParams::cand_head)
constexpr int kGemvMaxSamples = 8192;      // most samples per segment of the candidate-mode threshold estimate
constexpr uint32_t kTauHasCut = 0x40000000u; // bit of the epoch half of a threshold word: a token cut among equal keys goes with it
constexpr int kTauSpinLimit = 1 << 16;     // polls of a streaming workgroup for its threshold before it gives up
// Count field (10 bits) of a candidate slice whose workgroup never saw its threshold: no real slice holds more than
// 512 candidates, so the selection kernel cannot take it for a count, and it redoes the segment from the keys.
constexpr uint32_t kSliceGaveUp = 1023u;

// Common-cut route (a few segments of middling length: gemv_cut_kernel + select_rank_kernel)
constexpr int kCutTokensPerWg = 256;       // tokens (and threads) per workgroup of the GEMV = slice length
constexpr int kCutHead = 64;               // entries of a slice that the ranking kernel reads in its first round trip
constexpr int kCutMaxSlices = 256;         // slices per segment: segments of up to 65536 tokens
constexpr int kCutMaxK = 2048;             // largest k
constexpr int kCutMaxCandidates = 8192;    // candidates of one segment that the ranking kernel holds
constexpr int kCutMaxExtras = 6144;        // of them, entries beyond the first kCutHead of their slices
constexpr int kCutSamplesOnce = 256;        // sample rows of a segment where one workgroup scores them for all (256 or 512)
constexpr uint32_t kCutGaveUp = 0xffffffffu; // slice count of a workgroup that never saw its segment's cut
constexpr int64_t kCutMaxRows = 1572864;   // rows of a call (all segments) up to which the route is taken
constexpr int kCutParts = 8;                // ranking workgroups per segment, each with its own range of the order

// ---- lane exchanges ---------------------------------------------------------------------------

// DPP move: returns the value of the lane selected by CTRL inside the 16-lane row.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, false);
}

// Sum over the 16 lanes of a DPP row; every lane ends with the same value.  row_ror by 8, 4, 2, 1
// pairs each lane with its xor-8, xor-4, xor-2, xor-1 partner's partial (the partials have period 8,
// 4, 2 after each step), so the tree is the butterfly of gemv_topk.cu:325-328 bit for bit.
__device__ __forceinline__ float row16_sum(float p) {
  p = p + dpp_f32<0x128>(p);
  p = p + dpp_f32<0x124>(p);
  p = p + dpp_f32<0x122>(p);
  p = p + dpp_f32<0x121>(p);
  return p;
}

// Value held by lane (lane ^ M) of the wave, M a power of two.
//   M = 1, 2  : DPP quad_perm          M = 8 : DPP row_ror:8
//   M = 4, 16 : ds_swizzle bit mode    M = 32: ds_bpermute
template <int M>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v) {
  if constexpr (M == 1) {
    return dpp_u32<0xB1>(v);  // quad_perm [1,0,3,2]
  } else if constexpr (M == 2) {
    return dpp_u32<0x4E>(v);  // quad_perm [2,3,0,1]
  } else if constexpr (M == 8) {
    return dpp_u32<0x128>(v);  // row_ror:8
  } else if constexpr (M == 4 || M == 16) {
    return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (M << 10) | 0x1f);
  } else {
    static_assert(M == 32, "lane_xor: unsupported distance");
    int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    return (uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, (int)v);
  }
}

template <int M>
__device__ __forceinline__ uint64_t lane_xor64(uint64_t v) {
  uint32_t lo = lane_xor<M>((uint32_t)v);
  uint32_t hi = lane_xor<M>((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// Inclusive prefix sum over the 64 lanes of the wave: four DPP row shifts, then the row totals are carried
// forward with row_bcast:15 (rows 1, 3) and row_bcast:31 (rows 2, 3).  Lanes without a source add 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_add_u32(uint32_t v) {
  return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  v = dpp_add_u32<0x111, 0xf>(v);   // row_shr:1
  v = dpp_add_u32<0x112, 0xf>(v);   // row_shr:2
  v = dpp_add_u32<0x114, 0xf>(v);   // row_shr:4
  v = dpp_add_u32<0x118, 0xf>(v);   // row_shr:8
  v = dpp_add_u32<0x142, 0xa>(v);   // row_bcast:15 into rows 1 and 3
  v = dpp_add_u32<0x143, 0xc>(v);   // row_bcast:31 into rows 2 and 3
  return v;
}

// Largest and smallest value of the wave, valid in lane 63 only: two steps inside the quads, the two mirrors of a DPP
// row, and the row results carried forward as in the scan - six DPP operands and no trip through the LDS crossbar
// (lane_xor takes one for distances 4, 16 and 32).  A lane without a source keeps its own value.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_self(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ uint32_t wave_max_in_last_lane(uint32_t v) {
  v = max(v, dpp_or_self<0xB1, 0xf>(v));    // quad_perm [1,0,3,2]
  v = max(v, dpp_or_self<0x4E, 0xf>(v));    // quad_perm [2,3,0,1]
  v = max(v, dpp_or_self<0x141, 0xf>(v));   // row_half_mirror
  v = max(v, dpp_or_self<0x140, 0xf>(v));   // row_mirror
  v = max(v, dpp_or_self<0x142, 0xa>(v));   // row_bcast:15 into rows 1 and 3
  v = max(v, dpp_or_self<0x143, 0xc>(v));   // row_bcast:31 into rows 2 and 3
  return v;
}
__device__ __forceinline__ uint32_t wave_min_in_last_lane(uint32_t v) { return ~wave_max_in_last_lane(~v); }

__device__ __forceinline__ int lane_id() {
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// ---- 16-bit elements --------------------------------------------------------------------------

template <int DT>
struct Elem;

template <>
struct Elem<TKA_F16> {
  // widen element `i` (0..7) of a 16-byte packet
  static __device__ __forceinline__ float get(const u32x4& v, int i) {
    uint32_t w = v[i >> 1];
    uint16_t h = (i & 1) ? (uint16_t)(w >> 16) : (uint16_t)w;
    return (float)__builtin_bit_cast(_Float16, h);
  }
  static __device__ __forceinline__ float widen(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
  static __device__ __forceinline__ uint16_t narrow(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
};

template <>
struct Elem<TKA_BF16> {
  static __device__ __forceinline__ float get(const u32x4& v, int i) {
    uint32_t w = v[i >> 1];
    return __builtin_bit_cast(float, (i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  static __device__ __forceinline__ float widen(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
  static __device__ __forceinline__ uint16_t narrow(float f) {  // round to nearest even
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  }
};

// ---- canonical row score (gemv_topk.cu:303-332) ------------------------------------------------

// Group query of this lane in fp32: ((q0 + q1) + q2) + ... in ascending head order, dims 8j..8j+7.
// Groups are 1, 2, 4 or 8 heads; up to PAR heads of a group are asked for together (one round trip, not one per head;
// PAR bounds the registers in flight for kernels that have few).
template <int DT, int G, int PAR>
__device__ __forceinline__ void sum_group_query(const uint16_t* qb, float (&qf)[8]) {
  constexpr int P = G < PAR ? G : PAR;
#pragma unroll
  for (int g0 = 0; g0 < G; g0 += P) {
    u32x4 w[P];
#pragma unroll
    for (int g = 0; g < P; ++g) w[g] = *(const u32x4*)(qb + (int64_t)(g0 + g) * kHeadDim);
#pragma unroll
    for (int g = 0; g < P; ++g)
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[i] = (g0 + g == 0) ? Elem<DT>::get(w[g], i) : qf[i] + Elem<DT>::get(w[g], i);
    if (P < G && PAR >= 2) __builtin_amdgcn_sched_barrier(0);   // (batch after batch: scheduled together they would all be in flight after all)
  }
}
template <int DT, int PAR = 8>
__device__ __forceinline__ void load_group_query(const void* q, int64_t q_stride_b, int b, int h, int group, int j, float (&qf)[8]) {
  const uint16_t* qb = (const uint16_t*)q + (int64_t)b * q_stride_b + (int64_t)h * group * kHeadDim + 8 * j;
  if (group == 1) sum_group_query<DT, 1, PAR>(qb, qf);
  else if (group == 2) sum_group_query<DT, 2, PAR>(qb, qf);
  else if (group == 4) sum_group_query<DT, 4, PAR>(qb, qf);
  else sum_group_query<DT, 8, PAR>(qb, qf);
}

// Canonical score of the row in `kv` for the lane's 8 dims: fma chain, DPP butterfly, one multiply.
template <int DT>
__device__ __forceinline__ float row_score(const float (&qf)[8], const u32x4& kv, float scale) {
  float acc = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) acc = __builtin_fmaf(qf[i], Elem<DT>::get(kv, i), acc);
  return row16_sum(acc) * scale;
}

// ---- score key --------------------------------------------------------------------------------

// Order-preserving fp32 -> uint32 (bigger score, bigger key); -0.0 == +0.0; NaN is the lowest key.
__device__ __forceinline__ uint32_t score_key(float x) {
  if (x != x) return 0u;
  uint32_t u = __builtin_bit_cast(uint32_t, x + 0.0f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_score(uint32_t key) {
  uint32_t u = (key & 0x80000000u) ? (key & 0x7fffffffu) : ~key;
  return __builtin_bit_cast(float, u);
}
// 64-bit composite: all elements distinct, larger = earlier in (score desc, index asc) order.
__device__ __forceinline__ uint64_t composite(uint32_t key, uint32_t idx) { return ((uint64_t)key << 32) | (uint32_t)~idx; }

// ---- sampled thresholds -------------------------------------------------------------------------

__device__ __forceinline__ uint32_t mix32(uint32_t x) {  // integer hash for the sample jitter
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// Token of sample i of a segment: one per stride, at a hashed offset inside the stride so that periodic data
// cannot alias with the sampling.
__device__ __forceinline__ int64_t sample_token(int seg, int i, int64_t stride) {
  // (hash scaled to [0, stride) by a multiply-high: the hardware has no integer division)
  return (int64_t)i * stride + (int64_t)__umulhi(mix32((uint32_t)seg * 0x9e3779b9u + (uint32_t)i), (uint32_t)stride);
}

// The same for the common-cut route, whose kernels are a few microseconds long and pay for every instruction: the
// offset inside the stride is the fractional part of a multiple of the golden ratio (a sequence that fills the stride
// evenly), shifted per segment - three instructions instead of the hash's ten.
__device__ __forceinline__ int64_t cut_sample_token(int seg, int i, int64_t stride) {
  return (int64_t)i * stride + (int64_t)__umulhi(((uint32_t)i + (uint32_t)seg * 0x85ebca6bu) * 0x9e3779b9u, (uint32_t)stride);
}

// ---- block-wide threshold search (1024 threads, 2048 bins) --------------------------------------

// Finds the bin d with  count(bins > d) < need <= count(bins >= d)  in sh_hist[2048]; every one of the 1024
// threads of the block must call it.  Results: sh_res[0] = d, sh_res[1] = count(bins > d), sh_res[2] = sh_hist[d].
// sh_res is left untouched when the histogram holds fewer than `need` elements.
__device__ __forceinline__ void find_threshold_bin_1024(const uint32_t* sh_hist, uint32_t need, uint32_t* sh_wtot, uint32_t* sh_res) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const uint32_t h0 = sh_hist[2 * tid], h1 = sh_hist[2 * tid + 1];
  const uint32_t mine = h0 + h1;
  const uint32_t inc = wave_inclusive_scan(mine);
  const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
  const uint32_t v = wave_total - inc + mine;  // suffix sum over lanes >= lane
  if (lane == 0) sh_wtot[wave] = v;
  __syncthreads();
  // the totals of the waves above: one read and a sum across sixteen lanes instead of a loop of up to fifteen reads
  uint32_t above = lane > wave && lane < 16 ? sh_wtot[lane] : 0u;
  above += lane_xor<1>(above);
  above += lane_xor<2>(above);
  above += lane_xor<4>(above);
  above += lane_xor<8>(above);
  above = (uint32_t)__builtin_amdgcn_readfirstlane((int)above);
  const uint32_t ge0 = above + v;   // count(bins >= 2*tid)
  const uint32_t ge1 = ge0 - h0;    // count(bins >= 2*tid+1)
  const uint32_t gt1 = ge1 - h1;    // count(bins >  2*tid+1)
  if (ge1 >= need && gt1 < need) { sh_res[0] = 2 * tid + 1; sh_res[1] = gt1; sh_res[2] = h1; }
  if (ge0 >= need && ge1 < need) { sh_res[0] = 2 * tid;     sh_res[1] = ge1; sh_res[2] = h0; }
  __syncthreads();
}

// ---- host-side launch bookkeeping -------------------------------------------------------------

// Records an event pair around a launch when profiling is on (see tka_profile_enable).
struct LaunchTimer {
  LaunchTimer(const char* name, hipStream_t stream);
  ~LaunchTimer();
  const char* name_;
  hipStream_t stream_;
  void* slot_;
};

inline int hip_status(hipError_t e) { return e == hipSuccess ? TKA_OK : TKA_EHIP; }

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace tka
