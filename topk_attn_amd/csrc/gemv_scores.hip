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
// that stays in L2 +2 us.  The cost follows the volume that reaches HBM.  Hence two modes:
//   dense      every score is stored and a first-level histogram is flushed (short segments, the fallback,
//              and callers that want all scores);
//   candidate  a threshold tau per segment is known beforehand (sample_tau_kernel: an order statistic of a
//              strided sample of the segment, chosen so that about 2k tokens pass); only tokens with
//              key >= tau are stored, in index order, in the workgroup's own slice (the count rides in the
//              first entry: one partial line per workgroup).  The selection kernel checks that at least k
//              tokens passed and otherwise flags the segment for the fallback kernel, so the result is
//              exact whatever the data.
#include "kernels.hpp"

namespace tka {

namespace {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;
constexpr int kGemvUnroll = 8;                                         // loads in flight per lane
constexpr int kGemvRowsPerIter = (kGemvThreads / 16) * kGemvUnroll;    // 128 tokens per WG iteration
constexpr int kCandMaxIters = kGemvCandTokensPerWg / kGemvRowsPerIter; // iterations of a candidate-mode workgroup
constexpr int kCandSubLists = kCandMaxIters * kGemvWaves;
constexpr int kTauSplit = 4;   // sample workgroups (and thresholds) per segment

template <int DT, bool CAND>
__global__ __launch_bounds__(kGemvThreads) void gemv_scores_kernel(GemvParams p) {
  __shared__ uint32_t sh_hist[CAND ? 1 : kHistBins];
  __shared__ uint64_t sh_cand[CAND ? kCandSubLists : 1][32];   // per (iteration, wave): ascending index
  __shared__ uint32_t sh_ccnt[kCandSubLists];

  const int tid = threadIdx.x;
  const int j = tid & 15;            // lane inside the row: dims 8j..8j+7
  const int rg = tid >> 4;           // row group 0..15 inside the workgroup
  const int h = blockIdx.y;
  const int b = blockIdx.z;
  const int chunk = blockIdx.x / p.wgs_per_chunk;
  const int wg_in_chunk = blockIdx.x % p.wgs_per_chunk;
  const int64_t seg = ((int64_t)b * p.num_kv_heads + h) * p.num_chunks + chunk;
  // tokens are counted inside the chunk; the chunk starts at chunk*chunk_len, or at the start of the
  // cluster chosen for this (head, rank) in two-level selection
  const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;
  const int64_t t_begin = (int64_t)wg_in_chunk * p.tokens_per_wg;
  int64_t t_end = t_begin + p.tokens_per_wg;
  if (t_end > p.chunk_len) t_end = p.chunk_len;

  const bool do_hist = !CAND && p.hist != nullptr;
  if (do_hist) {
    for (int i = tid; i < kHistBins; i += kGemvThreads) sh_hist[i] = 0;
  }
  if (CAND && tid < kCandSubLists) sh_ccnt[tid] = 0;
  __syncthreads();

  float qf[8];
  load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf);

  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  float* sc_out = CAND ? nullptr : p.scores + seg * p.chunk_len;
  uint32_t tau = 0u;
  if (CAND) {   // lowest of the quarter thresholds: every quarter then passes at least its own share
    tau = ~0u;
#pragma unroll
    for (int w = 0; w < kTauSplit; ++w) tau = min(tau, p.tau_key[seg * kTauSplit + w]);
  }

  int it = 0;
  for (int64_t base = t_begin; base < t_end; base += kGemvRowsPerIter, ++it) {
    // row group rg owns 8 consecutive tokens per iteration: load u brings token base + rg*8 + u
    u32x4 kv[kGemvUnroll];
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      int64_t t = base + rg * kGemvUnroll + u;
      int64_t tc = t < t_end ? t : t_end - 1;
      kv[u] = __builtin_nontemporal_load((const u32x4*)(kbase + tc * p.key_stride_n));
    }
    float mine = 0.0f;
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const float s = row_score<DT>(qf, kv[u], p.scale);
      if (j == u) mine = s;
    }
    // lane j < 8 of row group rg now holds the score of token base + rg*8 + j: a wave covers 32
    // consecutive tokens, in lane order
    const int64_t t = base + rg * kGemvUnroll + j;
    const bool owner = j < kGemvUnroll && t < t_end;
    const uint32_t key = score_key(mine);
    if (CAND) {
      const bool pass = owner && key >= tau;
      const unsigned long long mask = __ballot(pass);
      const int lane = tid & 63, wave = tid >> 6;
      if (pass) sh_cand[it * kGemvWaves + wave][__popcll(mask & ((1ull << lane) - 1ull))] = composite(key, (uint32_t)t);
      if (lane == 0) sh_ccnt[it * kGemvWaves + wave] = (uint32_t)__popcll(mask);
    } else if (owner) {
      sc_out[t] = mine;
      if (do_hist) atomicAdd(&sh_hist[key >> (32 - kHistBits)], 1u);
    }
  }

  if (CAND) {
    // (iteration, wave) sub-lists are in token order one after the other: concatenate them into the slice
    __syncthreads();
    const int sub = tid >> 5, r = tid & 31;   // 8 sub-lists x 32 slots = 256 threads
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int s = 0; s < kCandSubLists; ++s) {
      const uint32_t c = sh_ccnt[s];
      before += s < sub ? c : 0u;
      total += c;
    }
    // Slice format: word = key << 32 | count << 8 | token - first token of the slice; only slot 0 carries the
    // count (0 .. 256), so a workgroup with few candidates writes a single line and nothing else
    uint64_t* slice = p.cand + seg * p.cand_seg_stride + (int64_t)wg_in_chunk * p.tokens_per_wg;
    if (sub < kCandSubLists && (uint32_t)r < sh_ccnt[sub]) {
      const uint64_t c = sh_cand[sub][r];
      const uint32_t pos = before + r;
      const uint32_t rel = ~(uint32_t)c - (uint32_t)t_begin;
      slice[pos] = (c & 0xffffffff00000000ull) | (pos == 0 ? total << 8 : 0u) | rel;
    }
    if (tid == 0 && total == 0) slice[0] = 0ull;
    return;
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

// ---- pilot: threshold of the candidate mode -----------------------------------------------------

constexpr int kTauThreads = 1024;
constexpr int kTauRowGroups = kTauThreads / 16;
constexpr int kTauUnroll = 8;            // rows per row group and round: 512 samples per round

__device__ __forceinline__ uint32_t mix32(uint32_t x) {  // integer hash for the sample jitter
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// kTauSplit workgroups per segment (a single CU cannot pull its share of rows fast enough): each scores
// num_samples tokens of its quarter of the segment (one per stride, at a hashed offset inside the stride so
// that periodic data cannot alias with the sampling) and takes the sample_rank-th largest key by radix select
// in LDS -> tau_key[segment][quarter].  About sample_rank/num_samples of the quarter's tokens lie at or above
// that key wherever the large scores sit in the segment; the GEMV uses the lowest of the four, so that the
// number of tokens that pass is at least the sum of the four shares.
template <int DT>
__global__ __launch_bounds__(kTauThreads) void sample_tau_kernel(GemvParams p, int num_samples, int sample_rank) {
  __shared__ uint32_t sh_keys[kGemvMaxSamples];
  __shared__ uint32_t sh_hist[kHistBins];
  __shared__ uint32_t sh_wtot[kTauThreads / kWave];
  __shared__ uint32_t sh_res[4];

  const int tid = threadIdx.x;
  const int j = tid & 15, rg = tid >> 4;
  const int seg = blockIdx.y;
  const int quarter = blockIdx.x;
  const int chunk = seg % p.num_chunks, bh = seg / p.num_chunks;
  const int h = bh % p.num_kv_heads, b = bh / p.num_kv_heads;
  const int64_t chunk_base = p.cluster_ids ? (int64_t)p.cluster_ids[seg] * p.chunk_len : (int64_t)chunk * p.chunk_len;

  float qf[8];
  load_group_query<DT>(p.q, p.q_stride_b, b, h, p.group, j, qf);
  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)b * p.key_stride_b + (int64_t)h * p.key_stride_h +
                          chunk_base * p.key_stride_n + 8 * j;
  const int64_t quarter_len = p.chunk_len / kTauSplit;
  const int64_t stride = quarter_len / num_samples;
  kbase += (int64_t)quarter * quarter_len * p.key_stride_n;

  // kTauUnroll rows in flight per row group: the kernel is one latency chain per batch of loads
  for (int base = 0; base < num_samples; base += kTauRowGroups * kTauUnroll) {
    u32x4 kv[kTauUnroll];
#pragma unroll
    for (int u = 0; u < kTauUnroll; ++u) {
      const int i = base + rg * kTauUnroll + u;                        // sample number (num_samples is a multiple of 512)
      const int64_t t = (int64_t)i * stride + (int64_t)(mix32(((uint32_t)seg * kTauSplit + quarter) * 0x9e3779b9u + (uint32_t)i) % (uint32_t)stride);
      kv[u] = *(const u32x4*)(kbase + t * p.key_stride_n);
    }
    float mine = 0.0f;
#pragma unroll
    for (int u = 0; u < kTauUnroll; ++u) {
      const float s = row_score<DT>(qf, kv[u], p.scale);
      if (j == u) mine = s;
    }
    if (j < kTauUnroll) sh_keys[base + rg * kTauUnroll + j] = score_key(mine);
  }

  // sample_rank-th largest of sh_keys[0 .. num_samples), resolved to its top 22 bits: the threshold only has
  // to lie at or below that order statistic, so the low 10 bits are left at zero
  uint32_t need = (uint32_t)sample_rank, prefix = 0;
  int fixed = 0;
  while (fixed < 2 * kHistBits) {
    const int bits = kHistBits;
    const int shift = 32 - fixed - bits;
    __syncthreads();
    sh_hist[2 * tid] = 0;
    sh_hist[2 * tid + 1] = 0;
    __syncthreads();
    for (int i = tid; i < num_samples; i += kTauThreads) {
      const uint32_t key = sh_keys[i];
      if (fixed == 0 || (key >> (32 - fixed)) == prefix) atomicAdd(&sh_hist[(key >> shift) & ((1u << bits) - 1u)], 1u);
    }
    __syncthreads();
    find_threshold_bin_1024(sh_hist, need, sh_wtot, sh_res);
    need -= sh_res[1];
    prefix = (prefix << bits) | sh_res[0];
    fixed += bits;
  }
  prefix <<= (32 - fixed);
  if (tid == 0) p.tau_key_out[seg * kTauSplit + quarter] = prefix;
}

}  // namespace

int launch_gemv_scores(const GemvParams& p, int dtype, hipStream_t stream) {
  dim3 grid((unsigned)(p.num_chunks * p.wgs_per_chunk), (unsigned)p.num_kv_heads, (unsigned)p.batch);
  const bool cand = p.cand != nullptr;
  LaunchTimer timer(cand ? "gemv_scores_cand" : "gemv_scores", stream);
  if (dtype == TKA_F16) {
    if (cand) gemv_scores_kernel<TKA_F16, true><<<grid, kGemvThreads, 0, stream>>>(p);
    else gemv_scores_kernel<TKA_F16, false><<<grid, kGemvThreads, 0, stream>>>(p);
  } else {
    if (cand) gemv_scores_kernel<TKA_BF16, true><<<grid, kGemvThreads, 0, stream>>>(p);
    else gemv_scores_kernel<TKA_BF16, false><<<grid, kGemvThreads, 0, stream>>>(p);
  }
  return hip_status(hipGetLastError());
}

int launch_sample_tau(const GemvParams& p, int dtype, int num_samples, int sample_rank, hipStream_t stream) {
  const dim3 segs(kTauSplit, (unsigned)(p.batch * p.num_kv_heads * p.num_chunks));
  LaunchTimer timer("sample_tau", stream);
  if (dtype == TKA_F16)
    sample_tau_kernel<TKA_F16><<<segs, kTauThreads, 0, stream>>>(p, num_samples, sample_rank);
  else
    sample_tau_kernel<TKA_BF16><<<segs, kTauThreads, 0, stream>>>(p, num_samples, sample_rank);
  return hip_status(hipGetLastError());
}

// Tokens per workgroup.  Short runs win: with 256 tokens (64 KB of keys) per workgroup the streaming rate
// measured on MI355X is about 5% above that of 2048-token runs.  Tiny problems take 128 so that every CU
// gets a workgroup.
int gemv_tokens_per_wg(int64_t total_rows, int64_t chunk_len) {
  (void)chunk_len;
  return total_rows <= 65536 ? 128 : kGemvCandTokensPerWg;
}

// Candidate-mode plan for one segment length and k: samples per sampling workgroup and the rank of the order
// statistic each of them takes as its threshold, or 0 samples when pruning does not pay (short segments, k a
// large share of the segment, more candidates than the selection kernel holds).
// With S = kTauSplit * s samples in all and m = k*S/n, R = m + 6*sqrt(m) + 2 is the total rank: the share of
// tokens that pass concentrates around R/S with relative deviation 1/sqrt(R), which puts "fewer than k pass"
// (the segment is then redone densely) four to five deviations out.  Taking the lowest of the four
// thresholds passes about a quarter more than R/S.
void gemv_candidate_plan(int64_t chunk_len, int k, int max_candidates, int* num_samples, int* sample_rank) {
  *num_samples = 0;
  *sample_rank = 0;
  if (chunk_len < 65536 || (int64_t)k * 16 > chunk_len) return;
  const int rounds = chunk_len >= 1048576 ? 4 : (chunk_len >= 524288 ? 2 : 1);   // more samples on long segments keep the candidate share near k/n
  const int s = kTauRowGroups * kTauUnroll * rounds;
  const double S = (double)s * kTauSplit;
  const double m = (double)k * S / (double)chunk_len;
  double root = 0.0;
  while ((root + 1.0) * (root + 1.0) <= m) root += 1.0;   // floor(sqrt(m))
  const int r = ((int)(m + 6.0 * (root + 1.0) + 2.0) + kTauSplit - 1) / kTauSplit;
  const double expected = (double)chunk_len * r / s * 1.25;
  if (expected * 1.3 > (double)max_candidates) return;
  *num_samples = s;
  *sample_rank = r;
}

}  // namespace tka
