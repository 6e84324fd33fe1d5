// Log-sum-exp combine of the split-K partials of one output row, as a device function: the combine kernel
// (attention.hip) and the combine launch of the decode step that also redoes flagged segments (topk_select.hip) share it.
#pragma once
#include "kernels.hpp"

namespace tka {

// One workgroup of kCombineThreads threads per output row.  The split maxima and sums go to LDS first (one
// coalesced read), the weights 2^(m_s-M) are computed once, then 32 groups of 32 lanes (4 dims per lane,
// 16-byte loads) add up the accumulators of every 32nd split and a last pass folds the 32 groups.
constexpr int kCombineThreads = 1024;
constexpr int kCombineLanes = kHeadDim / 4;                      // 32 lanes cover one accumulator row
constexpr int kCombineGroups = kCombineThreads / kCombineLanes;  // 32 splits in flight

// LDS of lse_combine_row, carved from a buffer of the caller (which may hold other things at other times)
struct CombineLds {
  float w[TKA_MAX_SPLITS];                     // m_s, then the weight of split s
  float red[kCombineThreads / kWave];
  f32x4 o[kCombineGroups][kCombineLanes];
  float stat[2];                               // M, L
};

template <int ODT>
__device__ __forceinline__ void lse_combine_row(const CombineParams& p, int row, CombineLds& sh) {
  float (&sh_w)[TKA_MAX_SPLITS] = sh.w;
  float (&sh_red)[kCombineThreads / kWave] = sh.red;
  f32x4 (&sh_o)[kCombineGroups][kCombineLanes] = sh.o;
  float (&sh_stat)[2] = sh.stat;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int S = p.num_splits;
  const float* pm = p.part_m + (int64_t)row * S;
  const float* pl = p.part_l + (int64_t)row * S;
  const f32x4* pa = (const f32x4*)(p.part_acc + (int64_t)row * S * kHeadDim);

  // accumulators: group g takes splits g, g+32, ...; the first four of them are requested before anything else,
  // so that their round trip to memory runs beside that of the maxima and sums
  const int g = tid / kCombineLanes, dl = tid % kCombineLanes;
  const f32x4 zero4 = (f32x4){0.f, 0.f, 0.f, 0.f};
  f32x4 a0[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int s = g + u * kCombineGroups;
    a0[u] = s < S ? pa[(int64_t)s * kCombineLanes + dl] : zero4;
  }

  // M = max over non-empty splits
  float ms = -INFINITY, ls = 0.0f;
  if (tid < S) {
    ls = pl[tid];
    ms = ls > 0.0f ? pm[tid] : -INFINITY;
  }
  float mx = ms;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
  if (lane == 0) sh_red[wave] = mx;
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < kCombineThreads / kWave; ++w) M = fmaxf(M, sh_red[w]);
  // weights and L
  const float wgt = (ms != -INFINITY) ? __builtin_amdgcn_exp2f(ms - M) : 0.0f;
  if (tid < S) sh_w[tid] = wgt;
  float lsum = ls * wgt;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) lsum += __shfl_xor(lsum, d, 64);
  __syncthreads();  // sh_red read by everyone, sh_w written
  if (lane == 0) sh_red[wave] = lsum;
  __syncthreads();
  if (tid == 0) {
    float L = 0.0f;
    for (int w = 0; w < kCombineThreads / kWave; ++w) L += sh_red[w];
    sh_stat[0] = M;
    sh_stat[1] = L;
  }
  f32x4 o = zero4;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int s = g + u * kCombineGroups;
    const float w = s < S ? sh_w[s] : 0.0f;
    if (w != 0.0f) o += a0[u] * w;   // the accumulator of an empty split is never looked at
  }
  // beyond 128 splits: four per trip, loads first (a load behind the weight test would make every trip a memory
  // round trip)
  for (int s0 = g + 4 * kCombineGroups; s0 < S; s0 += 4 * kCombineGroups) {
    f32x4 a[4];
    float w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = s0 + u * kCombineGroups;
      w[u] = s < S ? sh_w[s] : 0.0f;
      a[u] = s < S ? pa[(int64_t)s * kCombineLanes + dl] : zero4;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (w[u] != 0.0f) o += a[u] * w[u];
  }
  sh_o[g][dl] = o;
  __syncthreads();
  if (tid >= kHeadDim) return;
  const float L = sh_stat[1];
  float acc = 0.0f;
  const float* so = (const float*)sh_o;
#pragma unroll 8
  for (int gg = 0; gg < kCombineGroups; ++gg) acc += so[gg * kHeadDim + tid];
  const float r = L > 0.0f ? acc / L : 0.0f;
  const int bb = row / p.rows_per_batch, hh = row % p.rows_per_batch;
  uint16_t* out = (uint16_t*)p.out + (int64_t)bb * p.out_stride_b + (int64_t)hh * kHeadDim;
  out[tid] = Elem<ODT>::narrow(r);
  if (p.out_lse && tid == 0) p.out_lse[row] = L > 0.0f ? (sh_stat[0] + __builtin_log2f(L)) * 0.69314718055994531f : -INFINITY;
}

}  // namespace tka
