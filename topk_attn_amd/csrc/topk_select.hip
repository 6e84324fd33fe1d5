// Stage 1, selection phase: exact top-k of fp32 scores per segment, ties to the lower index, output in
// rank order.  Replaces the full cub::BlockRadixSort of the reference (gemv_topk.cu:353-378) with a
// radix SELECT followed by a sort of the k survivors only.
//
// Every element is ranked by the 64-bit composite (score key << 32) | ~index, so all elements are
// distinct and "top k" is unique: score descending, index ascending.
//
//   1. first-level histogram of the top 11 key bits (by the GEMV kernel, or select_hist_kernel);
//   2. filter: each workgroup finds the threshold bin b1 from the histogram, keeps its slice of the
//      scores in registers, and appends composites with bin > b1 to the "sure" list and bin == b1 to
//      the "maybe" list (one global reservation per workgroup and list);
//   3. finalize (next kernel, one workgroup per segment): refines the threshold inside the maybe
//      list with further 11-bit radix passes (stops as soon as a bucket is taken whole), gathers
//      the k survivors in LDS, sorts them with a bitonic network (registers, DPP / ds_swizzle across
//      lanes, LDS across waves) and writes indices and values.
//
// No workgroup ever waits for another: the hand-off between 2 and 3 is the kernel boundary (a
// device-scope fence per workgroup would write back the whole L2 of its XCD each time).
// Traffic: 4 B read per score plus 8 B written and read per sure/maybe element; scores come from L2 /
// Infinity Cache when the GEMV has just written them.
#include "kernels.hpp"

namespace tka {

namespace {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / kWave;
constexpr int kSelMaxPerThread = 16;  // scores per thread held in registers by the filter

// ---- block-wide helpers (1024 threads, 2048 bins) ---------------------------------------------

// Finds the bin d with  count(bins > d) < need <= count(bins >= d)  in sh_hist[2048].
// Results in sh_res[0] = d, sh_res[1] = count(bins > d), sh_res[2] = sh_hist[d].
__device__ void find_threshold_bin(const uint32_t* sh_hist, uint32_t need, uint32_t* sh_wtot, uint32_t* sh_res) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const uint32_t h0 = sh_hist[2 * tid], h1 = sh_hist[2 * tid + 1];
  uint32_t v = h0 + h1;  // suffix sum over lanes >= lane
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    uint32_t t = __shfl_down(v, d, 64);
    if (lane + d < 64) v += t;
  }
  if (lane == 0) sh_wtot[wave] = v;
  __syncthreads();
  uint32_t above = 0;
  for (int w = wave + 1; w < kSelWaves; ++w) above += sh_wtot[w];
  const uint32_t ge0 = above + v;   // count(bins >= 2*tid)
  const uint32_t ge1 = ge0 - h0;    // count(bins >= 2*tid+1)
  const uint32_t gt1 = ge1 - h1;    // count(bins >  2*tid+1)
  if (ge1 >= need && gt1 < need) { sh_res[0] = 2 * tid + 1; sh_res[1] = gt1; sh_res[2] = h1; }
  if (ge0 >= need && ge1 < need) { sh_res[0] = 2 * tid;     sh_res[1] = ge1; sh_res[2] = h0; }
  __syncthreads();
}

// ---- bitonic sort of 1024*E composites, descending --------------------------------------------

template <int M>
__device__ __forceinline__ void cx_lane(uint64_t& v, bool keep_max) {
  uint64_t o = lane_xor64<M>(v);
  bool take = keep_max ? (o > v) : (o < v);
  v = take ? o : v;
}

template <int STRIDE, int E>
__device__ __forceinline__ void cx_regs(uint64_t (&v)[E], int size) {
  if constexpr (STRIDE < E) {
#pragma unroll
    for (int s = 0; s < E; ++s) {
      if ((s & STRIDE) == 0) {
        int e = threadIdx.x * E + s;
        bool desc = (e & size) == 0;
        uint64_t a = v[s], b = v[s ^ STRIDE];
        bool sw = desc ? (b > a) : (b < a);
        v[s] = sw ? b : a;
        v[s ^ STRIDE] = sw ? a : b;
      }
    }
  }
}

// Thread t holds elements t*E .. t*E+E-1.  sh is scratch for the cross-wave strides (1024*E entries).
template <int E>
__device__ void bitonic_sort_desc(uint64_t (&v)[E], uint64_t* sh) {
  const int tid = threadIdx.x;
  constexpr int N = kSelThreads * E;
  for (int size = 2; size <= N; size <<= 1) {
    for (int stride = size >> 1; stride >= 1; stride >>= 1) {
      if (stride >= 64 * E) {
        // partner in another wave: exchange through LDS
        __syncthreads();
#pragma unroll
        for (int s = 0; s < E; ++s) sh[tid * E + s] = v[s];
        __syncthreads();
#pragma unroll
        for (int s = 0; s < E; ++s) {
          int e = tid * E + s;
          uint64_t o = sh[e ^ stride];
          bool keep_max = ((e & stride) == 0) == ((e & size) == 0);
          bool take = keep_max ? (o > v[s]) : (o < v[s]);
          v[s] = take ? o : v[s];
        }
      } else if (stride >= E) {
        const int m = stride / E;  // lane distance
#pragma unroll
        for (int s = 0; s < E; ++s) {
          int e = tid * E + s;
          bool keep_max = ((e & stride) == 0) == ((e & size) == 0);
          switch (m) {
            case 1: cx_lane<1>(v[s], keep_max); break;
            case 2: cx_lane<2>(v[s], keep_max); break;
            case 4: cx_lane<4>(v[s], keep_max); break;
            case 8: cx_lane<8>(v[s], keep_max); break;
            case 16: cx_lane<16>(v[s], keep_max); break;
            default: cx_lane<32>(v[s], keep_max); break;
          }
        }
      } else {
        // both elements in this thread (stride is 1, 2 or 4; compile-time register indices)
        switch (stride) {
          case 1: cx_regs<1, E>(v, size); break;
          case 2: cx_regs<2, E>(v, size); break;
          default: cx_regs<4, E>(v, size); break;
        }
      }
    }
  }
}

template <int E>
__device__ void sort_lds_desc(uint64_t* sh_sort, uint64_t* sh_xchg) {
  uint64_t v[E];
  const int tid = threadIdx.x;
#pragma unroll
  for (int s = 0; s < E; ++s) v[s] = sh_sort[tid * E + s];
  bitonic_sort_desc<E>(v, sh_xchg);
  __syncthreads();
#pragma unroll
  for (int s = 0; s < E; ++s) sh_sort[tid * E + s] = v[s];
  __syncthreads();
}

// ---- kernels ----------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void zero_u32_kernel(uint32_t* p, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// First-level histogram when the scores do not come from the GEMV kernel.
__global__ __launch_bounds__(kSelThreads) void select_hist_kernel(SelectParams p) {
  __shared__ uint32_t sh_hist[kHistBins];
  const int tid = threadIdx.x;
  const int seg = blockIdx.y;
  for (int i = tid; i < kHistBins; i += kSelThreads) sh_hist[i] = 0;
  __syncthreads();
  const float* sc = p.scores + (int64_t)seg * p.seg_stride;
  const int64_t begin = (int64_t)blockIdx.x * p.part_len;
  int64_t end = begin + p.part_len;
  if (end > p.seg_len) end = p.seg_len;
  for (int64_t i = begin + tid; i < end; i += kSelThreads) atomicAdd(&sh_hist[score_key(sc[i]) >> (32 - kHistBits)], 1u);
  __syncthreads();
  uint32_t* gh = p.hist + (int64_t)seg * kHistBins;
  for (int i = tid; i < kHistBins; i += kSelThreads) {
    uint32_t c = sh_hist[i];
    if (c) atomicAdd(&gh[i], c);
  }
}

__global__ __launch_bounds__(kSelThreads) void select_filter_kernel(SelectParams p) {
  __shared__ uint32_t sh_hist[kHistBins];
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];
  __shared__ uint32_t sh_cnt[2];    // workgroup totals: sure, maybe
  __shared__ uint32_t sh_base[2];   // global reservation bases

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int seg = blockIdx.y;
  const uint32_t k = (uint32_t)p.k;

  // ---- 1. threshold bin from the first-level histogram
  const uint32_t* gh = p.hist + (int64_t)seg * kHistBins;
  sh_hist[2 * tid] = gh[2 * tid];
  sh_hist[2 * tid + 1] = gh[2 * tid + 1];
  if (tid < 2) sh_cnt[tid] = 0;
  __syncthreads();
  find_threshold_bin(sh_hist, k, sh_wtot, sh_res);
  const uint32_t b1 = sh_res[0];

  // ---- 2. filter this workgroup's slice (kept in registers between count and write)
  const float* sc = p.scores + (int64_t)seg * p.seg_stride;
  const int64_t begin = (int64_t)blockIdx.x * p.part_len;
  uint32_t keys[kSelMaxPerThread];
  uint32_t my_sure = 0, my_maybe = 0;
  const int iters = p.part_len / kSelThreads;
#pragma unroll
  for (int it = 0; it < kSelMaxPerThread; ++it) {
    keys[it] = 0;
    if (it < iters) {
      int64_t i = begin + (int64_t)it * kSelThreads + tid;
      if (i < p.seg_len) {
        uint32_t key = score_key(sc[i]);
        uint32_t bin = key >> (32 - kHistBits);
        keys[it] = key;
        my_sure += bin > b1;
        my_maybe += bin == b1;
      } else {
        keys[it] = 0;  // bin 0 <= b1; excluded below by the bounds test
      }
    }
  }
  // wave-level exclusive prefix of the per-thread counts, wave totals reserved in LDS
  uint32_t ps = my_sure, pm = my_maybe;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    uint32_t ts = __shfl_up(ps, d, 64), tm = __shfl_up(pm, d, 64);
    if (lane >= d) { ps += ts; pm += tm; }
  }
  uint32_t wbase_s = 0, wbase_m = 0;
  if (lane == 63) {
    wbase_s = atomicAdd(&sh_cnt[0], ps);
    wbase_m = atomicAdd(&sh_cnt[1], pm);
  }
  wbase_s = __shfl(wbase_s, 63, 64);
  wbase_m = __shfl(wbase_m, 63, 64);
  __syncthreads();
  uint32_t* ctr = p.counters + (int64_t)seg * 4;
  if (tid == 0) {
    sh_base[0] = sh_cnt[0] ? atomicAdd(&ctr[0], sh_cnt[0]) : 0u;
    sh_base[1] = sh_cnt[1] ? atomicAdd(&ctr[1], sh_cnt[1]) : 0u;
  }
  __syncthreads();
  {
    uint64_t* sure = p.sure + (int64_t)seg * p.k;
    uint64_t* maybe = p.maybe + (int64_t)seg * p.seg_len;
    uint32_t slot_s = sh_base[0] + wbase_s + (ps - my_sure);
    uint32_t slot_m = sh_base[1] + wbase_m + (pm - my_maybe);
#pragma unroll
    for (int it = 0; it < kSelMaxPerThread; ++it) {
      if (it < iters) {
        int64_t i = begin + (int64_t)it * kSelThreads + tid;
        if (i < p.seg_len) {
          uint32_t bin = keys[it] >> (32 - kHistBits);
          uint64_t c = composite(keys[it], (uint32_t)i);
          if (bin > b1) sure[slot_s++] = c;
          else if (bin == b1) maybe[slot_m++] = c;
        }
      }
    }
  }

}

// Dynamic LDS layout of select_finalize_kernel: [0, 8 KB) histogram; then kpad composites (sort
// buffer); then kpad composites (cross-wave exchange buffer).
__global__ __launch_bounds__(kSelThreads) void select_finalize_kernel(SelectParams p, int kpad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint32_t* sh_hist = (uint32_t*)smem;
  uint64_t* sh_sort = (uint64_t*)(smem + kHistBins * sizeof(uint32_t));
  uint64_t* sh_xchg = sh_sort + kpad;
  __shared__ uint32_t sh_wtot[kSelWaves];
  __shared__ uint32_t sh_res[4];
  __shared__ uint32_t sh_cnt[2];

  const int tid = threadIdx.x;
  const int seg = blockIdx.x;
  const uint32_t k = (uint32_t)p.k;
  const uint32_t* ctr = p.counters + (int64_t)seg * 4;
  const uint32_t n_sure = ctr[0];
  const uint32_t n_maybe = ctr[1];

  // threshold bin again (cheap) — the maybe list holds exactly the elements of bin b1
  {
    const uint32_t* gh = p.hist + (int64_t)seg * kHistBins;
    sh_hist[2 * tid] = gh[2 * tid];
    sh_hist[2 * tid + 1] = gh[2 * tid + 1];
    __syncthreads();
    find_threshold_bin(sh_hist, k, sh_wtot, sh_res);
  }
  const uint32_t b1 = sh_res[0];
  const uint64_t* sure = p.sure + (int64_t)seg * p.k;
  const uint64_t* maybe = p.maybe + (int64_t)seg * p.seg_len;

  // Refine: composites of the maybe list share their top 11 bits (= b1).  Take `need` of them.
  uint32_t need = k - n_sure;           // >= 1 by construction of b1
  uint64_t prefix = b1;                 // value of the bits fixed so far
  int fixed = kHistBits;                // number of top bits fixed
  uint64_t threshold = 0;               // selected maybe elements: composite >= threshold
  bool done = (need == n_maybe);        // whole bin taken
  if (done) threshold = (uint64_t)b1 << (64 - kHistBits);
  while (!done) {
    const int bits = (64 - fixed) >= kHistBits ? kHistBits : (64 - fixed);
    const int shift = 64 - fixed - bits;
    __syncthreads();
    sh_hist[2 * tid] = 0;
    sh_hist[2 * tid + 1] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < n_maybe; i += kSelThreads) {
      uint64_t c = maybe[i];
      if ((c >> (64 - fixed)) == prefix) atomicAdd(&sh_hist[(uint32_t)(c >> shift) & ((1u << bits) - 1u)], 1u);
    }
    __syncthreads();
    find_threshold_bin(sh_hist, need, sh_wtot, sh_res);
    const uint32_t d = sh_res[0], gt = sh_res[1], cnt = sh_res[2];
    need -= gt;
    prefix = (prefix << bits) | d;
    fixed += bits;
    if (cnt == need || fixed == 64) {
      threshold = fixed == 64 ? prefix : (prefix << (64 - fixed));
      done = true;
    }
  }

  // Gather the k survivors (order irrelevant), pad with 0 (below every real composite).
  __syncthreads();
  for (int i = tid; i < kpad; i += kSelThreads) sh_sort[i] = 0;
  if (tid < 2) sh_cnt[tid] = 0;
  __syncthreads();
  for (uint32_t i = tid; i < n_sure; i += kSelThreads) sh_sort[i] = sure[i];
  for (uint32_t i = tid; i < n_maybe; i += kSelThreads) {
    uint64_t c = maybe[i];
    if (c >= threshold) {
      uint32_t slot = atomicAdd(&sh_cnt[0], 1u);
      if (n_sure + slot < k) sh_sort[n_sure + slot] = c;
    }
  }
  __syncthreads();

  switch (kpad / kSelThreads) {
    case 1: sort_lds_desc<1>(sh_sort, sh_xchg); break;
    case 2: sort_lds_desc<2>(sh_sort, sh_xchg); break;
    case 4: sort_lds_desc<4>(sh_sort, sh_xchg); break;
    default: sort_lds_desc<8>(sh_sort, sh_xchg); break;
  }

  const uint32_t idx_base = p.seg_base_ids ? (uint32_t)(p.seg_base_ids[seg] * p.seg_len)
                                           : (uint32_t)((seg % p.segs_per_row) * p.seg_len);
  int32_t* oi = p.out_idx + (int64_t)seg * p.out_stride;
  float* ov = p.out_val ? p.out_val + (int64_t)seg * p.out_stride : nullptr;
  for (uint32_t r = tid; r < k; r += kSelThreads) {
    uint64_t c = sh_sort[r];
    oi[r] = (int32_t)(~(uint32_t)c + idx_base);
    if (ov) ov[r] = key_score((uint32_t)(c >> 32));
  }
  if (p.out_expand) {
    int32_t* oe = p.out_expand + (int64_t)seg * p.k * p.expand;
    const uint32_t total = k * (uint32_t)p.expand;
    for (uint32_t e = tid; e < total; e += kSelThreads) {
      uint32_t jj = e / (uint32_t)p.expand, ii = e % (uint32_t)p.expand;
      oe[e] = (int32_t)(~(uint32_t)sh_sort[jj] * (uint32_t)p.expand + ii);
    }
  }
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
  switch (kpad / kSelThreads) {
    case 1: sort_lds_desc<1>(sh_sort, sh_xchg); break;
    case 2: sort_lds_desc<2>(sh_sort, sh_xchg); break;
    case 4: sort_lds_desc<4>(sh_sort, sh_xchg); break;
    default: sort_lds_desc<8>(sh_sort, sh_xchg); break;
  }
  // count distinct non-zero entries; entry i is kept when it differs from entry i-1
  int32_t* out = p.out_idx + (int64_t)seg * (p.k + p.sink + p.local);
  const int cap = p.k + p.sink + p.local;
  // positions: a prefix count of "kept" flags.  kpad <= 8192: each thread scans its contiguous run.
  const int per = kpad / kSelThreads;
  uint32_t mine = 0;
  for (int s = 0; s < per; ++s) {
    int i = tid * per + s;
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
  int kpad = kSelThreads;
  while (kpad < k) kpad <<= 1;
  return kpad;
}

}  // namespace

size_t select_workspace_bytes(int num_segments, int64_t seg_len, int k) {
  size_t b = 0;
  b += align_up((size_t)num_segments * kHistBins * sizeof(uint32_t), 256);
  b += align_up((size_t)num_segments * 4 * sizeof(uint32_t), 256);
  b += align_up((size_t)num_segments * (size_t)k * sizeof(uint64_t), 256);
  b += align_up((size_t)num_segments * (size_t)seg_len * sizeof(uint64_t), 256);
  return b;
}

void select_carve(void* ws, int num_segments, int64_t seg_len, int k, SelectParams* p) {
  unsigned char* c = (unsigned char*)ws;
  p->hist = (uint32_t*)c;
  c += align_up((size_t)num_segments * kHistBins * sizeof(uint32_t), 256);
  p->counters = (uint32_t*)c;
  c += align_up((size_t)num_segments * 4 * sizeof(uint32_t), 256);
  p->sure = (uint64_t*)c;
  c += align_up((size_t)num_segments * (size_t)k * sizeof(uint64_t), 256);
  p->maybe = (uint64_t*)c;
}

// Slice size per workgroup: a multiple of 1024 up to 16384, small enough that a segment is spread
// over several CUs when there are few segments.
void select_plan(int64_t seg_len, int num_segments, SelectParams* p) {
  int per_thread = kSelMaxPerThread;
  while (per_thread > 1) {
    int64_t parts = (seg_len + (int64_t)per_thread * kSelThreads - 1) / ((int64_t)per_thread * kSelThreads);
    if (parts * num_segments >= 256) break;
    per_thread >>= 1;
  }
  p->part_len = per_thread * kSelThreads;
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
  select_hist_kernel<<<dim3((unsigned)p.parts, (unsigned)p.num_segments), kSelThreads, 0, stream>>>(p);
  return hip_status(hipGetLastError());
}

int launch_select(const SelectParams& p, hipStream_t stream) {
  const int kpad = kpad_for(p.k);
  const size_t lds = kHistBins * sizeof(uint32_t) + 2 * (size_t)kpad * sizeof(uint64_t);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)select_finalize_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512);
    if (e != hipSuccess) return TKA_EHIP;
    attr_set = true;
  }
  {
    LaunchTimer timer("select_filter", stream);
    select_filter_kernel<<<dim3((unsigned)p.parts, (unsigned)p.num_segments), kSelThreads, 0, stream>>>(p);
    if (hipGetLastError() != hipSuccess) return TKA_EHIP;
  }
  LaunchTimer timer("select_finalize", stream);
  select_finalize_kernel<<<(unsigned)p.num_segments, kSelThreads, lds, stream>>>(p, kpad);
  return hip_status(hipGetLastError());
}

int launch_index_union(const UnionParams& p, hipStream_t stream) {
  const int kpad = kpad_for(p.k);
  const size_t lds = 2 * (size_t)kpad * sizeof(uint64_t);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)index_union_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512);
    if (e != hipSuccess) return TKA_EHIP;
    attr_set = true;
  }
  LaunchTimer timer("index_union", stream);
  index_union_kernel<<<(unsigned)p.num_segments, kSelThreads, lds, stream>>>(p, kpad);
  return hip_status(hipGetLastError());
}

}  // namespace tka
