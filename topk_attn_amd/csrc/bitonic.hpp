// Bitonic sort of up to 8192 64-bit composites in LDS by a block of 1024 threads, descending.
#pragma once
#include "common.hpp"

namespace tka {

constexpr int kSortThreads = 1024;

// ---- bitonic sort of 1024*E composites, descending --------------------------------------------

// One compare-exchange stage whose partner sits M lanes away.  keep_max is the same for every element of
// the thread (the stride and the merge size are multiples of E).  Composites are distinct (equal only
// among the zero padding), so "partner greater" decides both directions with one 64-bit compare.
template <int M, int E>
__device__ __forceinline__ void stage_lanes(uint64_t (&v)[E], bool keep_max) {
#pragma unroll
  for (int s = 0; s < E; ++s) {
    const uint64_t o = lane_xor64<M>(v[s]);
    const bool take = (o > v[s]) == keep_max;
    v[s] = take ? o : v[s];
  }
}

// One compare-exchange stage inside the thread (STRIDE < E).
template <int STRIDE, int E>
__device__ __forceinline__ void stage_regs(uint64_t (&v)[E], int first, int size) {
  if constexpr (STRIDE < E) {
#pragma unroll
    for (int s = 0; s < E; ++s) {
      if ((s & STRIDE) == 0) {
        const bool desc = ((first + s) & size) == 0;
        const uint64_t a = v[s], b = v[s ^ STRIDE];
        const bool sw = (b > a) == desc;
        v[s] = sw ? b : a;
        v[s ^ STRIDE] = sw ? a : b;
      }
    }
  }
}

// Bitonic sort, descending, of N composites held by the first N/E threads of the block (thread t holds
// elements t*E .. t*E+E-1).  The network is unrolled at compile time: strides inside a thread are
// register compare-exchanges, strides inside a wave use DPP / ds_swizzle / ds_bpermute, and only strides
// of 64*E and more go through LDS (`sh`, N entries) with block barriers, which every thread must reach.
template <int N, int E, int SIZE, int STRIDE>
__device__ __forceinline__ void bitonic_net(uint64_t (&v)[E], uint64_t* sh, int tid, bool active) {
  if constexpr (SIZE <= N) {
    const int e0 = tid * E;
    if constexpr (STRIDE >= 64 * E) {
      __syncthreads();
      if (active) {
#pragma unroll
        for (int s = 0; s < E; ++s) sh[e0 + s] = v[s];
      }
      __syncthreads();
      if (active) {
        const bool keep_max = ((e0 & STRIDE) == 0) == ((e0 & SIZE) == 0);
#pragma unroll
        for (int s = 0; s < E; ++s) {
          const uint64_t o = sh[(e0 + s) ^ STRIDE];
          const bool take = (o > v[s]) == keep_max;
          v[s] = take ? o : v[s];
        }
      }
    } else if constexpr (STRIDE >= E) {
      if (active) {
        const bool keep_max = ((e0 & STRIDE) == 0) == ((e0 & SIZE) == 0);
        stage_lanes<STRIDE / E, E>(v, keep_max);
      }
    } else {
      if (active) stage_regs<STRIDE, E>(v, e0, SIZE);
    }
    if constexpr (STRIDE > 1)
      bitonic_net<N, E, SIZE, STRIDE / 2>(v, sh, tid, active);
    else
      bitonic_net<N, E, SIZE * 2, SIZE>(v, sh, tid, active);
  }
}

// One element per thread up to 1024 (many waves hide the cross-lane latency), then 2, 4, 8 per thread.
template <int N>
__device__ __noinline__ void sort_lds_desc_n(uint64_t* sh_sort, uint64_t* sh_xchg) {
  constexpr int E = N > kSortThreads ? N / kSortThreads : 1;
  constexpr int NT = N / E;
  uint64_t v[E];
  const int tid = threadIdx.x;
  const bool active = tid < NT;
  if (active) {
#pragma unroll
    for (int s = 0; s < E; ++s) v[s] = sh_sort[tid * E + s];
  }
  bitonic_net<N, E, 2, 1>(v, sh_xchg, tid, active);
  __syncthreads();
  if (active) {
#pragma unroll
    for (int s = 0; s < E; ++s) sh_sort[tid * E + s] = v[s];
  }
  __syncthreads();
}

// Sorts sh_sort[0 .. kpad) descending; kpad is a power of two between 64 and 8192.
__device__ inline void sort_lds_desc(uint64_t* sh_sort, uint64_t* sh_xchg, int kpad) {
  switch (kpad) {
    case 64: sort_lds_desc_n<64>(sh_sort, sh_xchg); break;
    case 128: sort_lds_desc_n<128>(sh_sort, sh_xchg); break;
    case 256: sort_lds_desc_n<256>(sh_sort, sh_xchg); break;
    case 512: sort_lds_desc_n<512>(sh_sort, sh_xchg); break;
    case 1024: sort_lds_desc_n<1024>(sh_sort, sh_xchg); break;
    case 2048: sort_lds_desc_n<2048>(sh_sort, sh_xchg); break;
    case 4096: sort_lds_desc_n<4096>(sh_sort, sh_xchg); break;
    default: sort_lds_desc_n<8192>(sh_sort, sh_xchg); break;
  }
}

}  // namespace tka
