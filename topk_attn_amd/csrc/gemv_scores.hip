// Stage 1, GEMV phase: stream the key rows of one KV head once and produce fp32 scores in the canonical
// 16-lane order (gemv_topk.cu:303-332 of the reference).
//
// Mapping (wave64): 16 lanes x 16 B cover one 256-byte head row, so one global_load_dwordx4 brings four
// rows per wave; each lane keeps its 8 query dims in registers for the whole kernel; the 16-lane reduce is
// four DPP row rotations (no LDS).  Eight loads are in flight per lane.  HBM-bound: 256 B read per row.
//
// What the kernel WRITES decides how close it gets to the streaming rate.  Measured on MI355X (2.1 GB of
// keys): no writes 306 us; 4 B of score per row (1.6 % of the bytes) +45 us; 2 B per row +35 us; the
// histogram flush (150 memory-side atomics per 256-token workgroup) +40 us; the same stores into a buffer
// that stays in L2 +2 us.  The cost follows the volume that reaches HBM.  Hence two kernels:
//   dense      every score is stored and a first-level histogram is flushed (short segments and callers that
//              want all scores);
//   candidate  a threshold tau per segment comes from an order statistic of a strided sample of the segment,
//              chosen so that about 2k tokens pass; only tokens at or above it (key > tau, or key == tau and
//              token <= a cut that heavy ties make finite) are stored, in index order, in the workgroup's own
//              slice (the count rides in the first entry: one partial line per workgroup).  The selection
//              kernel checks that at least k tokens passed and otherwise redoes the segment from the keys, so
//              the result is exact whatever the data.
//              The sampling runs inside the same launch: the first workgroups of the grid score the samples,
//              the last of them to finish publishes the threshold, and the streaming workgroups need it only
//              when their rows are scored and wait (bounded) for it then.
#include "kernels.hpp"

namespace tka {

namespace {

constexpr int kGemvThreads = 256;
constexpr int kGemvUnroll = 8;                                         // loads in flight per lane
constexpr int kGemvRowsPerIter = (kGemvThreads / 16) * kGemvUnroll;    // 128 tokens per WG iteration
constexpr int kEarlySlices = 3;        // slices of a streaming workgroup that starts before the threshold is published
constexpr int kCandThreads = kGemvCandTokensPerWg;                     // candidate kernel: one thread per token of the slice
constexpr int kCandWaves = kCandThreads / kWave;
constexpr int kCandRowsPerIter = (kCandThreads / 16) * kGemvUnroll;    // 256 tokens per WG iteration

template <int DT>
__global__ __launch_bounds__(kGemvThreads) void gemv_scores_kernel(GemvParams p) {
  __shared__ uint32_t sh_hist[kHistBins];

  const int tid = threadIdx.x;
  const int j = tid & 15;            // lane inside the row: dims 8j..8j+7
  const int rg = tid >> 4;           // row group 0..15 inside the workgroup
  // (p.interleave_segs: the grid's x counts the heads and its y the places inside a head, see launch_gemv_scores)
  const int h = p.interleave_segs ? blockIdx.x : blockIdx.y;
  const int b = blockIdx.z;
  const uint32_t place = p.interleave_segs ? blockIdx.y : blockIdx.x;
  const int chunk = place / p.wgs_per_chunk;
  const int wg_in_chunk = place % p.wgs_per_chunk;
  const int64_t seg = ((int64_t)b * p.num_kv_heads + h) * p.num_chunks + chunk;
  const int64_t t_begin = (int64_t)wg_in_chunk * p.tokens_per_wg;
  int64_t t_end = t_begin + p.tokens_per_wg;
  if (t_end > p.chunk_len) t_end = p.chunk_len;

  const bool do_hist = p.hist != nullptr;
  if (do_hist) {
    for (int i = tid; i < kHistBins; i += kGemvThreads) sh_hist[i] = 0;
  }
  __syncthreads();

  // (without a centre stage the query is asked for behind the first rows, see below)
  float qf[8];
  if (p.centers) load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf);

  // tokens are counted inside the chunk; the chunk starts at chunk*chunk_len, or at the start of the
  // cluster chosen for this (head, rank) in two-level selection
  int64_t chunk_base;
  if (p.centers) {
    // Centre stage inline: every workgroup scores the (few) centroids of its head in the same order as any
    // other row, ranks them by (key descending, id ascending) and takes the one of rank `chunk`.  It costs a
    // round trip to memory at the head of the workgroup and saves a launch.
    __shared__ uint32_t sh_ckey[kGemvInlineCentres];
    __shared__ int sh_cid;
    const uint16_t* cbase = (const uint16_t*)p.centers + ((int64_t)b * p.num_kv_heads + h) * p.num_centers * kHeadDim + 8 * j;
    for (int c0 = 0; c0 < p.num_centers; c0 += kGemvRowsPerIter) {
      u32x4 cv[kGemvUnroll];
#pragma unroll
      for (int u = 0; u < kGemvUnroll; ++u) {
        const int c = c0 + rg * kGemvUnroll + u;
        cv[u] = *(const u32x4*)(cbase + (int64_t)(c < p.num_centers ? c : p.num_centers - 1) * kHeadDim);
      }
      float mine = 0.0f;
#pragma unroll
      for (int u = 0; u < kGemvUnroll; ++u) {
        const float s = row_score<DT>(qf, cv[u], p.scale);
        if (j == u) mine = s;
      }
      const int c = c0 + rg * kGemvUnroll + j;
      if (j < kGemvUnroll && c < p.num_centers) sh_ckey[c] = score_key(mine);
    }
    __syncthreads();
    if (tid < p.num_centers) {
      const uint32_t my = sh_ckey[tid];
      int ahead = 0;
      for (int i = 0; i < p.num_centers; ++i) {
        const uint32_t other = sh_ckey[i];
        ahead += (other > my || (other == my && i < tid)) ? 1 : 0;
      }
      if (ahead == chunk) sh_cid = tid;
    }
    __syncthreads();
    const int cid = sh_cid;
    if (wg_in_chunk == 0 && tid == 0) p.cluster_ids_out[seg] = cid;
    chunk_base = (int64_t)cid * p.chunk_len;
  } else {
    chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
  }

  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  float* sc_out = p.scores + seg * p.chunk_len;

  // row group rg owns 8 consecutive tokens per iteration: load u brings token base + rg*8 + u.  The first rows are
  // asked for before the query: its conversion waits for it, and that wait would otherwise stand in front of the
  // row loads (a round trip to memory that short launches feel).
  u32x4 kv[kGemvUnroll];
#pragma unroll
  for (int u = 0; u < kGemvUnroll; ++u) {
    int64_t t = t_begin + rg * kGemvUnroll + u;
    int64_t tc = t < t_end ? t : t_end - 1;
    kv[u] = __builtin_nontemporal_load((const u32x4*)(kbase + tc * p.key_stride_n));
  }
  __builtin_amdgcn_sched_barrier(0);
  if (!p.centers) load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf);
  for (int64_t base = t_begin; base < t_end; base += kGemvRowsPerIter) {
    if (base != t_begin) {
#pragma unroll
      for (int u = 0; u < kGemvUnroll; ++u) {
        int64_t t = base + rg * kGemvUnroll + u;
        int64_t tc = t < t_end ? t : t_end - 1;
        kv[u] = __builtin_nontemporal_load((const u32x4*)(kbase + tc * p.key_stride_n));
      }
    }
    float mine = 0.0f;
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const float s = row_score<DT>(qf, kv[u], p.scale);
      if (j == u) mine = s;
    }
    // lane j < 8 of row group rg now holds the score of token base + rg*8 + j
    const int64_t t = base + rg * kGemvUnroll + j;
    if (j < kGemvUnroll && t < t_end) {
      sc_out[t] = mine;
      if (do_hist) atomicAdd(&sh_hist[score_key(mine) >> (32 - kHistBits)], 1u);
    }
  }

  if (do_hist) {
    __syncthreads();
    uint32_t* gh = p.hist + seg * kHistBins;
    for (int i = tid; i < kHistBins; i += kGemvThreads) {
      uint32_t c = sh_hist[i];
      if (c) atomicAdd(&gh[i], c);
    }
  }
}

// ---- one key stream for a batch of queries ------------------------------------------------------------

// Value of lane (lane ^ 4) of the 16-lane row: row_half_mirror (lane ^ 7) then quad_perm [3,2,1,0] (lane ^ 3).
__device__ __forceinline__ float row_xor4(float x) { return dpp_f32<0x1B>(dpp_f32<0x141>(x)); }

// The 16-lane sums of BQ partial products per lane, in the canonical tree (xor 8, 4, 2, 1), as a reduce-scatter:
// at each level a lane keeps the half of its values whose query index has the lane's bit set (or clear) and hands
// the other half to its partner, so the adds are the ones of row16_sum (addition commutes) at about a third of
// the instructions.  Lane j returns the sum of query j / (16 / BQ).
template <int BQ>
__device__ __forceinline__ float row16_reduce_scatter(const float (&acc)[BQ], int j) {
  const bool b3 = (j & 8) != 0, b2 = (j & 4) != 0, b1 = (j & 2) != 0;
  float r;
  if constexpr (BQ == 8) {
    float r1[4], r2[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) r1[i] = (b3 ? acc[i + 4] : acc[i]) + dpp_f32<0x128>(b3 ? acc[i] : acc[i + 4]);
#pragma unroll
    for (int i = 0; i < 2; ++i) r2[i] = (b2 ? r1[i + 2] : r1[i]) + row_xor4(b2 ? r1[i] : r1[i + 2]);
    r = (b1 ? r2[1] : r2[0]) + dpp_f32<0x4E>(b1 ? r2[0] : r2[1]);
  } else if constexpr (BQ == 4) {
    float r1[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) r1[i] = (b3 ? acc[i + 2] : acc[i]) + dpp_f32<0x128>(b3 ? acc[i] : acc[i + 2]);
    r = (b2 ? r1[1] : r1[0]) + row_xor4(b2 ? r1[0] : r1[1]);
    r = r + dpp_f32<0x4E>(r);
  } else {
    static_assert(BQ == 2, "row16_reduce_scatter: 2, 4 or 8 queries");
    r = (b3 ? acc[1] : acc[0]) + dpp_f32<0x128>(b3 ? acc[0] : acc[1]);
    r = r + row_xor4(r);
    r = r + dpp_f32<0x4E>(r);
  }
  return r + dpp_f32<0xB1>(r);
}

// Keys shared by every batch entry (key_stride_b == 0: the operator of the reference holds one KV cache for
// the whole batch, retrieval_attention.cu:681-683): a workgroup scores its rows for BQ batch entries at once,
// so the keys are read once per BQ entries instead of once per entry.  Each score is the canonical one
// (fma chain over the lane's 8 dims, the 16-lane tree, one multiply) of its (entry, row).  16 row groups of
// 16 lanes, 8 rows in flight per group; after the reduce-scatter lane j holds the scores of entry
// j / (16 / BQ) for the 8 rows and stores BQ / 2 of them.
// PACKED (fp16, one query head per KV head): the queries stay in their 16-bit form, four registers per entry,
// and the widening is part of the multiply-add instruction.
// Grid: 1-D over (head, row tile, batch tile), batch tile fastest, dealt so that the tiles that share rows run
// on the same XCD (same L2) at about the same time.
template <int DT, int BQ, bool PACKED>
__global__ __launch_bounds__(kGemvThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void gemv_scores_shared_kernel(
    GemvParams p, int row_tiles, int batch_tiles) {
  constexpr int LPQ = 16 / BQ;       // lanes that end up with the same entry
  constexpr int RPL = 8 / LPQ;       // rows each of them stores
  const int tid = threadIdx.x;
  const int j = tid & 15, rg = tid >> 4;
  uint32_t id = blockIdx.x;
  if (gridDim.x % 8 == 0) id = (id % 8) * (gridDim.x / 8) + id / 8;
  const int bt = (int)(id % (uint32_t)batch_tiles);
  const int tile = (int)((id / (uint32_t)batch_tiles) % (uint32_t)row_tiles);
  const int h = (int)(id / ((uint32_t)batch_tiles * (uint32_t)row_tiles));
  const int b0 = bt * BQ;
  const int64_t n = p.chunk_len * p.num_chunks;
  const int64_t t_begin = (int64_t)tile * p.tokens_per_wg;
  int64_t t_end = t_begin + p.tokens_per_wg;
  if (t_end > n) t_end = n;

  float qf[PACKED ? 1 : BQ][8];
  u32x4 qp[PACKED ? BQ : 1];
#pragma unroll
  for (int q = 0; q < BQ; ++q) {
    const int b = b0 + q < p.batch ? b0 + q : p.batch - 1;
    if constexpr (PACKED)
      qp[q] = *(const u32x4*)((const uint16_t*)p.q + (int64_t)b * p.q_stride_b + (int64_t)h * kHeadDim + 8 * j);
    else
      load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf[q]);
  }
  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)h * p.key_stride_h + 8 * j;
  const int my_b = b0 + j / LPQ;
  const int my_row0 = (j % LPQ) * RPL;
  float* my_out = p.scores + ((int64_t)(my_b < p.batch ? my_b : 0) * p.num_kv_heads + h) * n;

  for (int64_t base = t_begin; base < t_end; base += kGemvRowsPerIter) {
    u32x4 kv[kGemvUnroll];
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const int64_t t = base + rg * kGemvUnroll + u;
      const int64_t tc = t < t_end ? t : t_end - 1;
      kv[u] = *(const u32x4*)(kbase + tc * p.key_stride_n);
    }
    float mine[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) mine[i] = 0.0f;
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      float acc[BQ];
#pragma unroll
      for (int q = 0; q < BQ; ++q) {
        acc[q] = 0.0f;
        if constexpr (PACKED) {
          // (the empty asm keeps the compiler from widening all queries to fp32 ahead of the loop, which
          // would take 8 registers per entry instead of 4)
          asm volatile("" : "+v"(qp[q]));
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[q] = __builtin_fmaf(Elem<DT>::get(qp[q], i), Elem<DT>::get(kv[u], i), acc[q]);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[q] = __builtin_fmaf(qf[q][i], Elem<DT>::get(kv[u], i), acc[q]);
        }
      }
      const float s = row16_reduce_scatter<BQ>(acc, j) * p.scale;
      if (u / RPL * RPL == my_row0) mine[u % RPL] = s;
      // one row at a time: its BQ independent chains are parallelism enough, and interleaving the rows costs
      // more registers than the file has for four waves
      __builtin_amdgcn_sched_barrier(0);
    }
    const int64_t t0 = base + rg * kGemvUnroll + my_row0;
    if (my_b < p.batch) {
#pragma unroll
      for (int i = 0; i < RPL; ++i)
        if (t0 + i < t_end) my_out[t0 + i] = mine[i];
    }
  }
}

// ---- candidate mode -----------------------------------------------------------------------------

// Sampling workgroup: scores 256 of the segment's p.num_samples sample tokens (one round of
// loads) and stores their keys in the segment's pool.  The workgroup that arrives last (epoch-valued arrival
// flags, so that the workspace needs no clearing) takes the p.sample_rank-th largest key of the whole pool and
// publishes it as the segment's threshold word, (epoch << 32) | key (and, in front of it, the token cut among
// the keys equal to it).  The sample is spread evenly over the segment, so about sample_rank/num_samples of the
// segment's tokens lie at or above that threshold wherever the large scores sit.
// Ordering between workgroups: the keys are agent-scope atomic stores, their completion and a barrier precede
// the workgroup's arrival flag; the last workgroup reads the pool with agent-scope atomic loads after it has
// seen every flag.
// sh: 2048 + 16 words.
template <int DT>
__device__ __forceinline__ void sample_role(const GemvParams& p, int seg, int part, uint32_t* sh) {
  uint32_t* sh_hist = sh;                   // 2048 bins
  uint32_t* sh_wtot = sh_hist + kHistBins;  // 8 wave totals, then [8] bin, [9] count above it, [10] "last" flag, [11] count in the bin, [12..14] tie scan
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int j = tid & 15, rg = tid >> 4;
  const int chunk = seg % p.num_chunks, bh = seg / p.num_chunks;
  const int h = bh % p.num_kv_heads, b = bh / p.num_kv_heads;
  const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
  float qf[8];
  load_group_query<DT, 1>(p.q, p.q_stride_b, b, h, p.group, j, qf);
  const int64_t stride = p.chunk_len / p.num_samples;
  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  uint32_t* pool = p.sample_pool + (int64_t)seg * p.num_samples;
  {
    const int first = part * kCandRowsPerIter + rg * kGemvUnroll;
    u32x4 kv[kGemvUnroll];
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u)
      kv[u] = *(const u32x4*)(kbase + sample_token(seg, first + u, stride) * p.key_stride_n);
    float mine = 0.0f;
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const float sc = row_score<DT>(qf, kv[u], p.scale);
      if (j == u) mine = sc;
    }
    if (j < kGemvUnroll) __hip_atomic_store(pool + first + j, score_key(mine), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // The keys went out as agent-scope atomic stores (performed at the point of coherence); what the counter
  // update needs is that they have completed, not a write-back of the L2 (an agent-scope release fence walks
  // the whole L2 every time a wave executes it: 4096 of them cost 150 us here).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's key stores have completed
  __syncthreads();
  if (wave == 0) {
    // Arrival flags, one word per sampling workgroup (a shared counter costs 0.4 us per arrival: the adds to
    // one word are served one after the other).  Set my flag, wait until it has completed, read all flags:
    // of two workgroups that finish together at least the one whose flag completed later sees both, so
    // somebody always sees all of them; if two do, both publish the same threshold.
    const int parts = p.num_samples / kCandRowsPerIter;   // <= 64
    uint32_t* flags = p.sample_flags + (int64_t)seg * (kGemvMaxSamples / kCandRowsPerIter);
    if (lane == 0) __hip_atomic_store(flags + part, p.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint32_t f = lane < parts ? __hip_atomic_load(flags + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : p.epoch;
    const bool all = __ballot(f == p.epoch) == ~0ull;
    if (lane == 0) sh_wtot[10] = all ? 1u : 0u;
  }
  __syncthreads();
  if (sh_wtot[10] == 0u) return;

  // sample_rank-th largest key of the pool, to its top 22 bits (the threshold only has to lie at or below that
  // order statistic): two 11-bit radix passes, thread t owns bins 4t .. 4t+3
  // the pool once into registers, all loads in flight together (one at a time they cost 2-3 us each)
  constexpr int kPerThread = kGemvMaxSamples / kCandThreads;
  constexpr int kBinsPerThread = kHistBins / kCandThreads;
  uint32_t keys[kPerThread];
#pragma unroll
  for (int u = 0; u < kPerThread; ++u) {
    const int i = u * kCandThreads + tid;
    keys[u] = i < p.num_samples ? __hip_atomic_load(pool + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
  }
  // One radix pass over the pooled keys: histogram of digit (key >> shift) & mask among the keys whose bits above the
  // digit equal `match`; finds the bin of the need-th largest.  sh_wtot[8] = bin, [9] = keys above it, [11] = keys in it.
  auto radix_pass = [&](int shift, uint32_t mask, int match_shift, uint32_t match, uint32_t need) {
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kBinsPerThread; ++e) sh_hist[kBinsPerThread * tid + e] = 0;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) {
      const uint32_t key = keys[u];
      if (u * kCandThreads + tid < p.num_samples && (match_shift >= 32 || (key >> match_shift) == match))
        atomicAdd(&sh_hist[(key >> shift) & mask], 1u);
    }
    __syncthreads();
    uint32_t h[kBinsPerThread], mine = 0;
#pragma unroll
    for (int e = 0; e < kBinsPerThread; ++e) {
      h[e] = sh_hist[kBinsPerThread * tid + e];
      mine += h[e];
    }
    uint32_t ge = mine;   // count in the bins of threads >= tid, first inside the wave
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const uint32_t t = __shfl_down(ge, d, 64);
      if (lane + d < 64) ge += t;
    }
    if (lane == 0) sh_wtot[wave] = ge;
    __syncthreads();
    for (int w = wave + 1; w < kCandWaves; ++w) ge += sh_wtot[w];
    if (ge >= need && ge - mine < need) {   // the bin sits among this thread's four: walk them from the top
      uint32_t above = ge - mine;
      int bin = 0;
      uint32_t in_bin = 0;
      bool found = false;
#pragma unroll
      for (int e = kBinsPerThread - 1; e >= 0; --e) {
        if (!found && above + h[e] >= need) { bin = kBinsPerThread * tid + e; in_bin = h[e]; found = true; }
        if (!found) above += h[e];
      }
      sh_wtot[8] = (uint32_t)bin;
      sh_wtot[9] = above;
      sh_wtot[11] = in_bin;
    }
    __syncthreads();
  };
  uint32_t need = (uint32_t)p.sample_rank;
  radix_pass(32 - kHistBits, kHistBins - 1, 32, 0u, need);
  uint32_t prefix = sh_wtot[8];
  need -= sh_wtot[9];
  radix_pass(32 - 2 * kHistBits, kHistBins - 1, 32 - kHistBits, prefix, need);
  prefix = (prefix << kHistBits) | sh_wtot[8];
  need -= sh_wtot[9];
  uint32_t tau = prefix << (32 - 2 * kHistBits);
  uint32_t cut = 0x7fffffffu;                 // tokens of the threshold key that pass: all
  // The threshold so far admits every key that shares the 22 leading bits of the order statistic.  When many
  // samples do (heavy ties: quantised or constant scores), that is far more tokens than planned, so the order
  // statistic is taken in the full order instead: the key to its last bit, and among the samples that hold that
  // key the need-th in token order, whose token becomes the cut.  The candidates (key > tau, or key == tau and
  // token <= cut) are still an upper set of the order (score descending, token ascending): if at least k pass
  // they contain the top k, whatever the data, and their number again concentrates around n R / S.
  constexpr uint32_t kTieSlack = 4;           // samples at the threshold beyond the need-th that are let pass as they are
  if (sh_wtot[11] - need > kTieSlack) {
    radix_pass(0, (1u << (32 - 2 * kHistBits)) - 1u, 32 - 2 * kHistBits, prefix, need);
    tau |= sh_wtot[8];
    need -= sh_wtot[9];
    if (sh_wtot[11] - need > kTieSlack) {
      // samples with key == tau in sample order (u, thread): counts per (u, wave), one scan, the need-th one
      __syncthreads();
#pragma unroll
      for (int u = 0; u < kPerThread; ++u) {
        const bool eq = u * kCandThreads + tid < p.num_samples && keys[u] == tau;
        const unsigned long long m = __ballot(eq);
        if (lane == 0) sh_hist[u * kCandWaves + wave] = (uint32_t)__popcll(m);
      }
      __syncthreads();
      if (wave == 0) {
        constexpr int kCells = kPerThread * kCandWaves;   // 128: two per lane, in order
        const uint32_t c0 = sh_hist[2 * lane], c1 = sh_hist[2 * lane + 1];
        const uint32_t inc = wave_inclusive_scan(c0 + c1);
        const uint32_t before0 = inc - (c0 + c1), before1 = before0 + c0;
        static_assert(kCells == 2 * kWave, "two cells per lane");
        if (before0 < need && need <= before0 + c0) { sh_wtot[12] = 2 * lane; sh_wtot[13] = need - before0; }
        if (before1 < need && need <= before1 + c1) { sh_wtot[12] = 2 * lane + 1; sh_wtot[13] = need - before1; }
      }
      __syncthreads();
      const int cell = (int)sh_wtot[12];
      const uint32_t nth = sh_wtot[13];              // 1-based position inside the cell's wave
#pragma unroll
      for (int u = 0; u < kPerThread; ++u) {
        if (u == cell / kCandWaves && wave == cell % kCandWaves) {
          const bool eq = u * kCandThreads + tid < p.num_samples && keys[u] == tau;
          const unsigned long long m = __ballot(eq);
          const uint32_t rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
          if (eq && rank + 1u == nth) sh_wtot[14] = (uint32_t)sample_token(seg, u * kCandThreads + tid, stride);
        }
      }
      __syncthreads();
      cut = sh_wtot[14];
    }
  }
  if (p.withhold_mod > 0 && seg % p.withhold_mod == p.withhold_rem) {
    // testing: this segment's threshold is withheld, so that streaming workgroups run into the end of their
    // bounded wait.  Mode 0: for good.  Mode 1: until one of them has given up (it leaves the call's epoch in the
    // segment's flag word), or this wait, bounded like theirs, runs out.
    if (p.withhold_mode == 0) return;
    if (tid == 0) {
      const uint32_t* flag = p.seg_flags + seg;
      for (int spin = 0; spin < kTauSpinLimit && __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != p.epoch; ++spin)
        __builtin_amdgcn_s_sleep(16);
    }
  }
  if (tid == 0) {
    // A cut (rare: heavy ties) goes out first, and once it has completed, the word the streaming workgroups wait
    // for; bit 30 of the word's epoch half says that there is a cut to fetch.
    const bool has_cut = cut != 0x7fffffffu;
    if (has_cut) {
      __hip_atomic_store(p.tau_words + 2 * seg + 1, (uint64_t)cut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __hip_atomic_store(p.tau_words + 2 * seg, ((uint64_t)(p.epoch | (has_cut ? kTauHasCut : 0u)) << 32) | tau, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Scores of one slice (up to 512 tokens from sbase on) as keys into LDS: lane j < 8 of row group rg writes the
// key of token it*256 + rg*8 + j to keys_out[it*256].  FULL: the slice has all 512 tokens; the eight rows of
// a lane then differ by a uniform offset and one lane offset serves all loads.  Otherwise rows past the end
// are clamped to the last one, lane by lane.
template <int DT, bool FULL>
__device__ __forceinline__ void stream_slice(const unsigned char* sbase, uint32_t row_bytes, int n_local, const float (&qf)[8],
                                             float scale, uint32_t* keys_out) {
  const int j = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const uint32_t voff = (uint32_t)(rg * kGemvUnroll) * row_bytes + 16u * (uint32_t)j;
  for (int it = 0; it < kCandThreads / kCandRowsPerIter; ++it) {
    u32x4 kv[kGemvUnroll];
    if constexpr (FULL) {
      const unsigned char* ibase = sbase + (uint64_t)(it * kCandRowsPerIter) * row_bytes;   // uniform
#pragma unroll
      for (int u = 0; u < kGemvUnroll; ++u)
        kv[u] = __builtin_nontemporal_load((const u32x4*)(ibase + (uint64_t)u * row_bytes + voff));
    } else {
#pragma unroll
      for (int u = 0; u < kGemvUnroll; ++u) {
        int lt = it * kCandRowsPerIter + rg * kGemvUnroll + u;
        lt = lt < n_local ? lt : n_local - 1;
        kv[u] = __builtin_nontemporal_load((const u32x4*)(sbase + ((uint32_t)lt * row_bytes + 16u * (uint32_t)j)));
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // all eight loads go out before the first score is computed
    float mine = 0.0f;
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const float sc = row_score<DT>(qf, kv[u], scale);
      if (j == u) mine = sc;
    }
    if (j < kGemvUnroll) keys_out[it * kCandRowsPerIter] = score_key(mine);
  }
}

// Grid: p.sample_wgs sampling workgroups first (so that they are resident before any workgroup that waits for
// them), then the streaming workgroups.  Slices (512 tokens) are numbered segment-major (or, with
// ROUND, in units that go round the segments, see launch_gemv_candidates).  The first
// p.early_wgs streaming workgroups take kEarlySlices consecutive slices each, all later ones a single slice:
// the workgroups that start together with the sampling would otherwise sit idle on their CU until the
// thresholds arrive; with more rows to stream they reach that point when the thresholds are there.
template <int DT, bool ROUND>
__global__ __launch_bounds__(kCandThreads) __attribute__((amdgpu_waves_per_eu(8, 8))) void gemv_candidates_kernel(GemvParams p) {
  __shared__ uint32_t sh[kHistBins + 16];   // streaming: keys of kEarlySlices * 512 tokens + wave counts; sampling: histogram
  static_assert(kEarlySlices * kCandThreads <= kHistBins, "LDS of the streaming role");
  const int tid = threadIdx.x;
  if ((int)blockIdx.x < p.sample_wgs) {
    __builtin_amdgcn_s_setprio(3);   // everyone else waits for these few waves
    const int parts = p.num_samples / kCandRowsPerIter;
    sample_role<DT>(p, (int)blockIdx.x / parts, (int)blockIdx.x % parts, sh);
    return;
  }
  uint32_t* sh_key = sh;                               // keys of this workgroup's tokens, slice after slice
  uint32_t* sh_wcnt = sh + kEarlySlices * kCandThreads; // candidates per wave
  __shared__ uint32_t sh_tau[3];                        // the segment's threshold key, whether it has arrived, its token cut

  const int j = tid & 15;            // lane inside the row: dims 8j..8j+7
  const int rg = tid >> 4;           // row group 0..15 inside the workgroup
  const int lane = tid & 63, wave = tid >> 6;
  // (slices and segments are counted in 32 bits - the launcher checks that the grid fits - because a 64-bit division is
  // a hundred scalar instructions, and a workgroup asks for its first row only behind them)
  const uint32_t w = blockIdx.x - (uint32_t)p.sample_wgs;
  int num_slices = w < (uint32_t)p.early_wgs ? kEarlySlices : 1;
  const uint32_t first_slice = w < (uint32_t)p.early_wgs ? w * kEarlySlices : (uint32_t)p.early_wgs * kEarlySlices + (w - (uint32_t)p.early_wgs);

  int64_t first_seg;
  int first_wg;
  if (ROUND) {
    // slices numbered in units of kEarlySlices consecutive slices of one segment, the units segment after segment and
    // then on through the tokens: unit u = slices kEarlySlices (u / segs) ... of segment u % segs (a segment's last
    // unit may be short: the numbers behind its end name no slice)
    const uint32_t segs = (uint32_t)(p.batch * p.num_kv_heads * p.num_chunks);
    const uint32_t u = first_slice / (uint32_t)kEarlySlices, r = first_slice - u * (uint32_t)kEarlySlices;
    const uint32_t t = u / segs;
    first_seg = (int64_t)(u - t * segs);
    first_wg = (int)(t * (uint32_t)kEarlySlices + r);
    const int left = p.wgs_per_chunk - first_wg;
    if (left <= 0) return;
    num_slices = num_slices < left ? num_slices : left;
  } else {
    first_seg = (int64_t)(first_slice / (uint32_t)p.wgs_per_chunk);
    first_wg = (int)(first_slice % (uint32_t)p.wgs_per_chunk);
  }

  // A workgroup that starts after the first wave of them finds its threshold published: it asks for the word
  // now, so that the answer travels beside the rows instead of costing a round trip of its own behind them
  // (a request issued at the end queues behind the loads of the other workgroups of the CU).
  uint64_t early_word = 0;
  if (num_slices == 1 && tid == 0) early_word = __hip_atomic_load(p.tau_words + 2 * first_seg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  const uint32_t row_bytes = (uint32_t)p.key_stride_n * 2u;
  {
    int64_t seg = first_seg;
    int wg_in_chunk = first_wg;
    for (int s = 0; s < num_slices; ++s) {
      const uint32_t chunk = (uint32_t)seg % (uint32_t)p.num_chunks, bh = (uint32_t)seg / (uint32_t)p.num_chunks;
      const int h = (int)(bh % (uint32_t)p.num_kv_heads), b = (int)(bh / (uint32_t)p.num_kv_heads);
      const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
      const int64_t t_begin = (int64_t)wg_in_chunk * kCandThreads;
      const int n_local = (int)(p.chunk_len - t_begin < kCandThreads ? p.chunk_len - t_begin : kCandThreads);
      float qf[8];
      load_group_query<DT, 1>(p.q, p.q_stride_b, b, h, p.group, j, qf);   // (one head at a time: the kernel has 64 registers per lane, and its workgroups overlap each other's waits)
      // uniform base of the slice + 32-bit lane offsets: one address register per load
      const unsigned char* sbase = (const unsigned char*)p.keys +
                                   2 * ((int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h + (chunk_base + t_begin) * p.key_stride_n);
      uint32_t* keys_out = sh_key + s * kCandThreads + rg * kGemvUnroll + j;
      if (n_local == kCandThreads)
        stream_slice<DT, true>(sbase, row_bytes, n_local, qf, p.scale, keys_out);
      else
        stream_slice<DT, false>(sbase, row_bytes, n_local, qf, p.scale, keys_out);
      if (++wg_in_chunk == p.wgs_per_chunk) { wg_in_chunk = 0; ++seg; }
    }
  }
  __syncthreads();

  uint32_t tau = 0, cut = 0;
  bool tau_ready = false;
  int64_t tau_seg = first_seg, seg = first_seg;
  int wg_in_chunk = first_wg;
  for (int s = 0; s < num_slices; ++s) {
    const int64_t t_begin = (int64_t)wg_in_chunk * kCandThreads;
    int64_t t_end = t_begin + kCandThreads;
    if (t_end > p.chunk_len) t_end = p.chunk_len;
    // Threshold of the slice's segment: one lane fetches the word and hands it on through LDS (every wave
    // asking for itself makes a hot spot of the few words).  A bounded wait: a workgroup that never sees its
    // threshold stores no candidates and marks its slice (kSliceGaveUp in the count field); the selection kernel
    // redoes a segment that holds such a slice from the keys, however many candidates the other slices hold.
    if (s == 0 || seg != tau_seg) {
      tau_seg = seg;
      if (s) __syncthreads();   // the previous slice's threshold has been read
      if (tid == 0) {
        const uint64_t* word = p.tau_words + 2 * seg;
        uint64_t v = early_word;
        for (int spin = 0; ((uint32_t)(v >> 32) & ~kTauHasCut) != p.epoch && spin < p.tau_spin_limit; ++spin) {
          if (spin) __builtin_amdgcn_s_sleep(16);
          v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        early_word = 0;
        __atomic_signal_fence(__ATOMIC_SEQ_CST);   // (the cut below is asked for behind the word that announces it: program order, which the compiler must keep)
        const uint32_t ep = (uint32_t)(v >> 32);
        sh_tau[0] = (uint32_t)v;
        sh_tau[1] = (ep & ~kTauHasCut) == p.epoch ? 1u : 0u;
        // (a cut was written, and had completed, before the word that announces it)
        sh_tau[2] = (ep & kTauHasCut) ? (uint32_t)__hip_atomic_load(word + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0x7fffffffu;
      }
      __syncthreads();
      tau = sh_tau[0];
      tau_ready = sh_tau[1] != 0u;
      cut = sh_tau[2];
    }

    // thread t owns token t_begin + t: candidates in index order into the slice.
    // Slice format: word = key << 32 | count << 9 | token - first token of the slice; only entry 0 carries
    // the count (0 .. 512).  Entries 0 .. 31 go to the slice's 256 bytes of the dense head array, further
    // ones (rare) to the slice's place in the wide array: the stores of a launch then touch a few megabytes
    // of whole lines, which stay in the L2 until the kernel ends, instead of one partial line per 4 KB.
    const uint32_t key = sh_key[s * kCandThreads + tid];
    // at or above the threshold in the order (score descending, token ascending)
    const bool pass = tau_ready && t_begin + tid < t_end && (key > tau || (key == tau && (uint32_t)(t_begin + tid) <= cut));
    const unsigned long long mask = __ballot(pass);
    if (s) __syncthreads();   // the previous slice's counts have been read
    if (lane == 0) sh_wcnt[wave] = (uint32_t)__popcll(mask);
    __syncthreads();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int v = 0; v < kCandWaves; ++v) {
      const uint32_t c = sh_wcnt[v];
      before += v < wave ? c : 0u;
      total += c;
    }
    uint64_t* slice = p.cand + seg * p.cand_seg_stride + (int64_t)wg_in_chunk * kCandThreads;
    uint64_t* head = p.cand_head + (seg * p.wgs_per_chunk + wg_in_chunk) * kCandHead;
    if (pass) {
      // (stored through to memory: a plain store leaves a dirty line in this XCD's L2 to be written back when the kernel
      // ends, and the launch measured 1.6 us longer with it, 317.3 against 315.7 us for 2 GiB of keys)
      const uint32_t pos = before + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
      __hip_atomic_store((pos < (uint32_t)kCandHead ? head : slice) + pos, ((uint64_t)key << 32) | (pos == 0 ? total << 9 : 0u) | (uint32_t)tid,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (tid == 0 && total == 0) head[0] = tau_ready ? 0ull : (uint64_t)(kSliceGaveUp << 9);
    if (tid == 0 && !tau_ready) __hip_atomic_store(p.seg_flags + seg, p.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (++wg_in_chunk == p.wgs_per_chunk) { wg_in_chunk = 0; ++seg; }
  }
}

// ---- candidate mode over keys that the batch shares ---------------------------------------------------

// Keys shared by every batch entry (key_stride_b == 0) on long segments: a streaming workgroup scores its slice for a
// tile of BQ batch entries at once, so the keys are streamed once per tile instead of once per entry (the batch
// loop of retrieval_attention.cu:654-896 over one cache, :681-683, at the lengths of the candidate route).  Every
// score is the canonical one of its (entry, row): fma chain over the lane's 8 dims and the 16-lane tree as a
// reduce-scatter (row16_reduce_scatter), one multiply.  Thresholds, slices and flags are those of the segment
// (entry, head), exactly as the one-entry kernel leaves them: the selection behind it does not know the difference.
// The kernel is bound by the vector units, not by memory (B x 128 multiply-adds per row and their 16-lane sums, with
// the packed two-per-instruction form of the fp32 multiply-add not used here): batch 8 over 8 heads x 131072 tokens
// takes 84 us where the one-entry kernel takes 311 for the same scores.
// One slice per workgroup, slices numbered (head, batch tile)-major (workgroups that take several slices each at the
// front of the grid, as the one-entry kernel has them, cost 3 us here).  Sampling workgroups: sample_role, one
// segment each.
template <int DT, int BQ>
__global__ __launch_bounds__(kCandThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemv_candidates_shared_kernel(GemvParams p, int batch_tiles) {
  constexpr int LPQ = 16 / BQ;       // lanes of a row that end up with the same entry
  constexpr int RPL = 8 / LPQ;       // rows of a round each of them keeps
  // streaming: keys of the slice for BQ entries, then wave counts and thresholds; sampling: histogram
  constexpr int kWords = BQ * kCandThreads + BQ * kCandWaves + 4 * BQ;
  __shared__ uint32_t sh[kWords > kHistBins + 16 ? kWords : kHistBins + 16];
  __shared__ __attribute__((aligned(16))) float sh_q[BQ * kHeadDim];   // group queries of the tile's entries
  const int tid = threadIdx.x;
  if ((int)blockIdx.x < p.sample_wgs) {
    __builtin_amdgcn_s_setprio(3);   // everyone else waits for these few waves
    const int parts = p.num_samples / kCandRowsPerIter;
    sample_role<DT>(p, (int)blockIdx.x / parts, (int)blockIdx.x % parts, sh);
    return;
  }
  uint32_t* sh_key = sh;                          // [entry][token]
  uint32_t* sh_wcnt = sh + BQ * kCandThreads;     // [entry][wave]
  uint32_t* sh_tau = sh_wcnt + BQ * kCandWaves;   // [entry]: threshold key, arrived, cut

  const int j = tid & 15, rg = tid >> 4;
  const int lane = tid & 63, wave = tid >> 6;
  const uint32_t slice_no = blockIdx.x - (uint32_t)p.sample_wgs;
  const uint32_t vseg = slice_no / (uint32_t)p.wgs_per_chunk;
  const int wg_in_chunk = (int)(slice_no % (uint32_t)p.wgs_per_chunk);
  const int h = (int)(vseg / (uint32_t)batch_tiles), b0 = (int)(vseg % (uint32_t)batch_tiles) * BQ;
  const int64_t t_begin = (int64_t)wg_in_chunk * kCandThreads;
  const int n_local = (int)(p.chunk_len - t_begin < kCandThreads ? p.chunk_len - t_begin : kCandThreads);
  const uint32_t row_bytes = (uint32_t)p.key_stride_n * 2u;
  const int my_q = j / LPQ, my_row0 = (j % LPQ) * RPL;

  // ---- the rows of the first round are asked for before anything else: they travel beside the queries
  const unsigned char* sbase = (const unsigned char*)p.keys + 2 * ((int64_t)h * p.key_stride_h + t_begin * p.key_stride_n);
  u32x4 kv[kGemvUnroll];
  auto ask = [&](int it, int first) {   // four rows of round `it`
#pragma unroll
    for (int u = first; u < first + 4; ++u) {
      int lt = it * kCandRowsPerIter + rg * kGemvUnroll + u;
      lt = lt < n_local ? lt : n_local - 1;
      kv[u] = __builtin_nontemporal_load((const u32x4*)(sbase + ((uint32_t)lt * row_bytes + 16u * (uint32_t)j)));
    }
  };
  ask(0, 0);
  ask(0, 4);

  // ---- the group queries of the tile's entries, summed once for the workgroup: every one of its 32 row groups needs all
  // of them, and each lane summing its own (BQ entries x G heads: 32 loads, 256 widenings and 192 adds at G = 4) was a
  // fifth of the kernel's instructions.  Thread x: two dims of one entry, heads added in ascending order in fp32
  // (sum_group_query's order).
  for (int x = tid; x < BQ * (kHeadDim / 2); x += kCandThreads) {
    const int e = x / (kHeadDim / 2), d = x % (kHeadDim / 2) * 2;
    const int b = b0 + e < p.batch ? b0 + e : p.batch - 1;
    const uint16_t* qb = (const uint16_t*)p.q + (int64_t)b * p.q_stride_b + (int64_t)h * p.group * kHeadDim + d;
    uint32_t w[8];
#pragma unroll
    for (int g = 0; g < 8; ++g) w[g] = g < p.group ? *(const uint32_t*)(qb + g * kHeadDim) : 0u;
    float s0 = Elem<DT>::widen((uint16_t)w[0]), s1 = Elem<DT>::widen((uint16_t)(w[0] >> 16));
#pragma unroll
    for (int g = 1; g < 8; ++g)
      if (g < p.group) {
        s0 = s0 + Elem<DT>::widen((uint16_t)w[g]);
        s1 = s1 + Elem<DT>::widen((uint16_t)(w[g] >> 16));
      }
    sh_q[e * kHeadDim + d] = s0;
    sh_q[e * kHeadDim + d + 1] = s1;
  }
  __syncthreads();

  // ---- scores of the slice for the BQ entries of the tile, as keys into LDS.  Four rows are computed while the next four
  // are on their way (the kernel is bound by the vector units; with all eight rows of a round asked for and then awaited
  // together its four waves per SIMD did not cover the wait).
  {
    float qf[BQ][8];
#pragma unroll
    for (int q = 0; q < BQ; ++q) {
      const f32x4 lo = *(const f32x4*)(sh_q + q * kHeadDim + 8 * j), hi = *(const f32x4*)(sh_q + q * kHeadDim + 8 * j + 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        qf[q][i] = lo[i];
        qf[q][4 + i] = hi[i];
      }
    }
    constexpr int kRounds = kCandThreads / kCandRowsPerIter;
#pragma unroll
    for (int it = 0; it < kRounds; ++it) {
      float mine[RPL];
#pragma unroll
      for (int i = 0; i < RPL; ++i) mine[i] = 0.0f;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int u = 4 * half; u < 4 * half + 4; ++u) {
          float acc[BQ];
#pragma unroll
          for (int q = 0; q < BQ; ++q) {
            acc[q] = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[q] = __builtin_fmaf(qf[q][i], Elem<DT>::get(kv[u], i), acc[q]);
          }
          const float sc = row16_reduce_scatter<BQ>(acc, j) * p.scale;
          if (u / RPL * RPL == my_row0) mine[u % RPL] = sc;
          __builtin_amdgcn_sched_barrier(0);   // one row at a time (see gemv_scores_shared_kernel)
        }
        if (it + 1 < kRounds) ask(it + 1, 4 * half);   // (their registers are free now)
        __builtin_amdgcn_sched_barrier(0);
      }
      uint32_t* dst = sh_key + my_q * kCandThreads + it * kCandRowsPerIter + rg * kGemvUnroll + my_row0;
#pragma unroll
      for (int i = 0; i < RPL; ++i) dst[i] = score_key(mine[i]);
    }
  }
  // thresholds of the tile's segments: BQ lanes poll one word each (bounded, see gemv_candidates_kernel)
  if (tid < BQ && b0 + tid < p.batch) {
    const int64_t seg = (int64_t)(b0 + tid) * p.num_kv_heads + h;
    const uint64_t* word = p.tau_words + 2 * seg;
    uint64_t v = 0;
    for (int spin = 0; ((uint32_t)(v >> 32) & ~kTauHasCut) != p.epoch && spin < p.tau_spin_limit; ++spin) {
      if (spin) __builtin_amdgcn_s_sleep(16);
      v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __atomic_signal_fence(__ATOMIC_SEQ_CST);   // (the cut below is asked for behind the word that announces it)
    const uint32_t ep = (uint32_t)(v >> 32);
    sh_tau[4 * tid] = (uint32_t)v;
    sh_tau[4 * tid + 1] = (ep & ~kTauHasCut) == p.epoch ? 1u : 0u;
    sh_tau[4 * tid + 2] = (ep & kTauHasCut) ? (uint32_t)__hip_atomic_load(word + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0x7fffffffu;
  }
  __syncthreads();

  // ---- candidates of every entry: thread t owns token t of the slice
  int64_t t_end = t_begin + kCandThreads;
  if (t_end > p.chunk_len) t_end = p.chunk_len;
  unsigned long long mask[BQ];
#pragma unroll
  for (int q = 0; q < BQ; ++q) {
    const uint32_t key = sh_key[q * kCandThreads + tid];
    const uint32_t tau = sh_tau[4 * q], cut = sh_tau[4 * q + 2];
    const bool pass = b0 + q < p.batch && sh_tau[4 * q + 1] != 0u && t_begin + tid < t_end &&
                      (key > tau || (key == tau && (uint32_t)(t_begin + tid) <= cut));
    mask[q] = __ballot(pass);
    if (lane == 0) sh_wcnt[q * kCandWaves + wave] = (uint32_t)__popcll(mask[q]);
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < BQ; ++q) {
    if (b0 + q >= p.batch) continue;
    const int64_t seg = (int64_t)(b0 + q) * p.num_kv_heads + h;
    const bool tau_ready = sh_tau[4 * q + 1] != 0u;
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int v = 0; v < kCandWaves; ++v) {
      const uint32_t c = sh_wcnt[q * kCandWaves + v];
      before += v < wave ? c : 0u;
      total += c;
    }
    uint64_t* slice = p.cand + seg * p.cand_seg_stride + (int64_t)wg_in_chunk * kCandThreads;
    uint64_t* head = p.cand_head + (seg * p.wgs_per_chunk + wg_in_chunk) * kCandHead;
    if (mask[q] >> lane & 1ull) {
      const uint32_t key = sh_key[q * kCandThreads + tid];
      const uint32_t pos = before + (uint32_t)__popcll(mask[q] & ((1ull << lane) - 1ull));
      __hip_atomic_store((pos < (uint32_t)kCandHead ? head : slice) + pos, ((uint64_t)key << 32) | (pos == 0 ? total << 9 : 0u) | (uint32_t)tid,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (tid == 0 && total == 0) head[0] = tau_ready ? 0ull : (uint64_t)(kSliceGaveUp << 9);
    if (tid == 0 && !tau_ready) __hip_atomic_store(p.seg_flags + seg, p.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace

int launch_gemv_scores(const GemvParams& p0, int dtype, hipStream_t stream) {
  GemvParams p = p0;
  const int64_t places = (int64_t)p.num_chunks * p.wgs_per_chunk;
  // Which workgroups run together: those of consecutive tokens of one head (x counts the places inside a head), or those of
  // the same tokens of all heads (x counts the heads).  Where a head's rows lie a multiple of 4 KB apart (16, 32 KV heads in
  // a cache laid out [token][head][128]) the first crowds a few memory channels: 2 x 16 heads x 131072 tokens 252 -> 188 us,
  // 16 x 65536 71 -> 49, 4 x 16 x 16384 57 -> 44, 32 x 131072 196 -> 189.  Calls of up to a million rows gain as well
  // (8 x 32768 tokens 17.7 -> 15.4 us, 8 x 8 x 16384 46.0 -> 44.5); large ones of other strides lose 2-3 % (4 x 8 x 131072:
  // 189 against 183 us) and keep the first.
  const int64_t row_bytes = p.key_stride_n * 2, rows = (int64_t)p.batch * p.num_kv_heads * p.num_chunks * p.chunk_len;
  p.interleave_segs = places <= 65535 && p.num_kv_heads > 1 &&
                      (row_bytes % 4096 == 0 || (rows <= (1 << 20) && (p.num_kv_heads & (p.num_kv_heads - 1)) == 0)) ? 1 : 0;
  dim3 grid((unsigned)places, (unsigned)p.num_kv_heads, (unsigned)p.batch);
  if (p.interleave_segs) grid = dim3((unsigned)p.num_kv_heads, (unsigned)places, (unsigned)p.batch);
  LaunchTimer timer("gemv_scores", stream);
  if (dtype == TKA_F16)
    gemv_scores_kernel<TKA_F16><<<grid, kGemvThreads, 0, stream>>>(p);
  else
    gemv_scores_kernel<TKA_BF16><<<grid, kGemvThreads, 0, stream>>>(p);
  return hip_status(hipGetLastError());
}

// Shared keys (key_stride_b == 0), plain scores [batch][head][seq_len] (no histogram, no cluster bases).
int launch_gemv_scores_shared(const GemvParams& p0, int dtype, hipStream_t stream) {
  if (p0.key_stride_b != 0 || p0.cluster_ids || !p0.scores) return TKA_EINVAL;
  GemvParams p = p0;
  const int64_t n = p.chunk_len * p.num_chunks;
  p.tokens_per_wg = kGemvRowsPerIter;   // one round of loads per workgroup: measured 10-20 % quicker than two
  // fp16 queries of single heads stay packed: 8 entries per pass fit the registers; otherwise 4 (fp32 queries)
  const bool packed = dtype == TKA_F16 && p.group == 1;
  const int bq = packed && p.batch >= 5 ? 8 : p.batch >= 3 ? 4 : 2;
  const int64_t row_tiles = (n + p.tokens_per_wg - 1) / p.tokens_per_wg;
  const int64_t batch_tiles = (p.batch + bq - 1) / bq;
  const int64_t wgs = row_tiles * batch_tiles * p.num_kv_heads;
  if (wgs > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  LaunchTimer timer("gemv_scores_shared", stream);
#define TKA_LAUNCH_SHARED(DT, BQ, PACKED) \
  gemv_scores_shared_kernel<DT, BQ, PACKED><<<(unsigned)wgs, kGemvThreads, 0, stream>>>(p, (int)row_tiles, (int)batch_tiles)
  if (packed) {
    if (bq == 8) TKA_LAUNCH_SHARED(TKA_F16, 8, true);
    else if (bq == 4) TKA_LAUNCH_SHARED(TKA_F16, 4, true);
    else TKA_LAUNCH_SHARED(TKA_F16, 2, true);
  } else if (dtype == TKA_F16) {
    if (bq == 4) TKA_LAUNCH_SHARED(TKA_F16, 4, false);
    else TKA_LAUNCH_SHARED(TKA_F16, 2, false);
  } else {
    if (bq == 4) TKA_LAUNCH_SHARED(TKA_BF16, 4, false);
    else TKA_LAUNCH_SHARED(TKA_BF16, 2, false);
  }
#undef TKA_LAUNCH_SHARED
  return hip_status(hipGetLastError());
}

// Streaming workgroups of the candidate kernel that the current device holds at once: 8 waves per SIMD, 4 SIMDs per
// CU, 8 waves per workgroup = 4 per CU (1024 on the 256 CUs of MI355X).  Asked for once.
static int64_t resident_streaming_wgs() {
  static const int64_t n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
    return (int64_t)4 * cus;
  }();
  return n;
}

// Candidate mode: sampling workgroups (256 samples each) at the front of the grid, then the streaming ones.
int launch_gemv_candidates(const GemvParams& p0, int dtype, hipStream_t stream) {
  GemvParams p = p0;
  const int64_t segs = (int64_t)p.batch * p.num_kv_heads * p.num_chunks;
  if (p.tokens_per_wg != kCandThreads || p.num_samples < kCandRowsPerIter || p.num_samples % kCandRowsPerIter ||
      p.num_samples > kGemvMaxSamples || p.sample_rank < 1 || p.sample_rank > p.num_samples)
    return TKA_EINVAL;
  p.sample_wgs = (int)(segs * (p.num_samples / kCandRowsPerIter));
  // early workgroups: as many as the GPU holds at once
  // Rows of one head 4 KB apart (sixteen KV heads in a cache laid out [token][head][128]): the workgroups that run
  // together, all on the same few heads, crowd the same memory channels - 4.7 instead of 6.3 TB/s.  Then the slices are
  // taken in units of kEarlySlices of one segment, segment after segment, and on through the tokens (per launch, 131072
  // tokens: 16 heads 115 -> 89 us, 2 x 16 226 -> 169, 4 x 16 432 -> 329).  Other strides keep the segment-by-segment
  // order, which is 0.5-2 % quicker for them (8 x 8 heads: 325.7 against 328.6 us).
  p.interleave_segs = p.key_stride_n * 2 == 4096 ? 1 : 0;
  const int64_t slices = p.interleave_segs ? segs * ((p.wgs_per_chunk + kEarlySlices - 1) / kEarlySlices) * kEarlySlices : segs * p.wgs_per_chunk;
  int64_t early = resident_streaming_wgs();
  if (early > slices / (2 * kEarlySlices)) early = slices / (2 * kEarlySlices);
  p.early_wgs = (int)early;
  if (slices > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  const int64_t wgs = p.sample_wgs + early + (slices - early * kEarlySlices);
  if (wgs > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  LaunchTimer timer("gemv_candidates", stream);
  if (dtype == TKA_F16) {
    if (p.interleave_segs) gemv_candidates_kernel<TKA_F16, true><<<(unsigned)wgs, kCandThreads, 0, stream>>>(p);
    else gemv_candidates_kernel<TKA_F16, false><<<(unsigned)wgs, kCandThreads, 0, stream>>>(p);
  } else {
    if (p.interleave_segs) gemv_candidates_kernel<TKA_BF16, true><<<(unsigned)wgs, kCandThreads, 0, stream>>>(p);
    else gemv_candidates_kernel<TKA_BF16, false><<<(unsigned)wgs, kCandThreads, 0, stream>>>(p);
  }
  return hip_status(hipGetLastError());
}

// Candidate mode over keys shared by the batch (key_stride_b == 0): the keys are streamed once per tile of batch entries.
int launch_gemv_candidates_shared(const GemvParams& p0, int dtype, hipStream_t stream) {
  GemvParams p = p0;
  if (p.key_stride_b != 0 || p.cluster_ids || p.num_chunks != 1 || p.tokens_per_wg != kCandThreads || p.num_samples < kCandRowsPerIter ||
      p.num_samples % kCandRowsPerIter || p.num_samples > kGemvMaxSamples || p.sample_rank < 1 || p.sample_rank > p.num_samples)
    return TKA_EINVAL;
  const int64_t segs = (int64_t)p.batch * p.num_kv_heads;
  p.sample_wgs = (int)(segs * (p.num_samples / kCandRowsPerIter));
  const int bq = p.batch >= 5 ? 8 : (p.batch >= 3 ? 4 : 2);
  const int batch_tiles = (p.batch + bq - 1) / bq;
  const int64_t slices = (int64_t)p.num_kv_heads * batch_tiles * p.wgs_per_chunk;
  p.early_wgs = 0;
  const int64_t wgs = p.sample_wgs + slices;
  if (wgs > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  LaunchTimer timer("gemv_candidates_shared", stream);
#define TKA_LAUNCH_CAND_SHARED(DT, BQ) gemv_candidates_shared_kernel<DT, BQ><<<(unsigned)wgs, kCandThreads, 0, stream>>>(p, batch_tiles)
  if (dtype == TKA_F16) {
    if (bq == 8) TKA_LAUNCH_CAND_SHARED(TKA_F16, 8);
    else if (bq == 4) TKA_LAUNCH_CAND_SHARED(TKA_F16, 4);
    else TKA_LAUNCH_CAND_SHARED(TKA_F16, 2);
  } else {
    if (bq == 8) TKA_LAUNCH_CAND_SHARED(TKA_BF16, 8);
    else if (bq == 4) TKA_LAUNCH_CAND_SHARED(TKA_BF16, 4);
    else TKA_LAUNCH_CAND_SHARED(TKA_BF16, 2);
  }
#undef TKA_LAUNCH_CAND_SHARED
  return hip_status(hipGetLastError());
}

// Tokens per workgroup.  Short runs win: with 256 tokens (64 KB of keys) per workgroup the streaming rate
// measured on MI355X is about 5% above that of 2048-token runs.  Problems of up to a million rows (256 MB of
// keys) take 128, one round of loads per workgroup: more workgroups than fit at once, so loads and arithmetic
// of different workgroups overlap (262144 rows: 15.1 instead of 17.1 us).
int gemv_tokens_per_wg(int64_t total_rows, int64_t chunk_len) {
  (void)chunk_len;
  return total_rows <= (1 << 20) ? 128 : kGemvDenseTokensPerWg;
}

// Candidate-mode plan for one segment length and k: samples per segment and the rank of the order statistic
// that becomes the threshold, or 0 samples when pruning does not pay (short segments, k a large share of the
// segment, more candidates than the selection kernel holds).
// With S samples spread evenly over the n tokens and m = k*S/n, the rank is R = m + 6*sqrt(m) + 2.  The share of
// tokens at or above the R-th largest sample concentrates around R/S with relative deviation 1/sqrt(R), so
// "fewer than k pass" (the segment is then redone from the keys) lies more than four deviations out, and about
// n*R/S candidates are stored.
void gemv_candidate_plan(int64_t chunk_len, int64_t total_rows, int k, int max_candidates, int* num_samples, int* sample_rank) {
  *num_samples = 0;
  *sample_rank = 0;
  if (chunk_len < kCandMinSegLen || (int64_t)k * 16 > chunk_len) return;
  // between 32768 and 65536 tokens the sampling at the head of the launch only pays on large calls (8 x 8 segments of
  // 32768: 120 instead of 134 us per decode step; 2 x 8 segments: 58 instead of 56)
  if (chunk_len < 2 * kCandMinSegLen && total_rows < kCandMinRows) return;
  // more samples on long segments keep the candidate count near k
  const int s = chunk_len >= 1048576 ? kGemvMaxSamples : (chunk_len >= 524288 ? kGemvMaxSamples / 2 : kGemvMaxSamples / 4);
  const double m = (double)k * s / (double)chunk_len;
  double root = 0.0;
  while ((root + 1.0) * (root + 1.0) <= m) root += 1.0;   // floor(sqrt(m))
  const int r = (int)(m + 6.0 * (root + 1.0) + 2.0);
  const double expected = (double)chunk_len * r / s;
  if (expected * 1.5 > (double)max_candidates) return;
  *num_samples = s;
  *sample_rank = r;
}

}  // namespace tka
