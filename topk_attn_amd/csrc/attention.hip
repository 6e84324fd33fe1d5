// Stages 2 and 3: split-K decode attention over a token list (dense range, gathered index list, or an
// index list with caller-supplied logits) and the log-sum-exp combine.
//
// attn_partial_kernel — one workgroup per (split, KV head, batch entry), 4 waves.  A 16-lane row group
// owns one token at a time (4 or 8 tokens in flight): 16 B of the K row and 16 B of the V row per lane, scores for the G query
// heads of the group by fma chain + DPP row reduce, online softmax in the exp2 domain
// (baseline_1.cu:406-468 of the reference), fp32 accumulators of 8 output dims per lane and head.
// The 16 row-group states of the workgroup are merged through LDS and written as one fp32
// (m, l, acc[128]) partial per query head; nothing is atomically added and nothing needs pre-zeroing.
//
// lse_combine_kernel — out = sum_s acc_s 2^(m_s-M) / sum_s l_s 2^(m_s-M), written once
// (replaces the DSM ring reduce + half atomicAdd of flash_decoding.cu:325-387).
#include "kernels.hpp"
#include "lse_combine.hpp"

namespace tka {

namespace {

constexpr int kAttnThreads = 256;
constexpr int kAttnRowGroups = kAttnThreads / 16;  // 16 tokens per load slot of the workgroup

enum { MODE_DENSE = 0, MODE_INDEXED = 1, MODE_LOGIT = 2 };

// Tokens per row group per step: K and V rows of U tokens are in flight together (2*U 16-byte loads per
// lane).  Large groups keep fewer in flight to stay inside the register file.
template <int G>
struct AttnUnroll {
  static constexpr int value = G <= 4 ? 8 : 4;
};

template <int DT, int G, int MODE>
__global__ __launch_bounds__(kAttnThreads) void attn_partial_kernel(AttnParams p) {
  constexpr int U = AttnUnroll<G>::value;
  constexpr int kStep = kAttnRowGroups * U;  // positions per workgroup step
  __shared__ float sh_acc[kAttnRowGroups][kHeadDim];
  __shared__ float sh_m[kAttnRowGroups];
  __shared__ float sh_l[kAttnRowGroups];

  const int tid = threadIdx.x;
  const int j = tid & 15;
  const int rg = tid >> 4;
  const int split = MODE == MODE_DENSE && p.head_fastest ? blockIdx.y : blockIdx.x;   // (see launch_attn_partial)
  const int h = MODE == MODE_DENSE && p.head_fastest ? blockIdx.x : blockIdx.y;
  const int b = blockIdx.z;
  const int64_t seg = (int64_t)b * p.num_kv_heads + h;

  int64_t count = p.seq_len;
  if (MODE != MODE_DENSE) {
    count = p.kv_count ? p.kv_count[seg] : p.idx_len;
    if (count > p.idx_len) count = p.idx_len;
    if (count < 0) count = 0;
  }
  const int64_t begin = (int64_t)split * p.tokens_per_split;
  int64_t end = begin + p.tokens_per_split;
  if (end > count) end = count;

  const int32_t* idx = MODE != MODE_DENSE ? p.kv_idx + seg * p.idx_len : nullptr;
  const float* logit = MODE == MODE_LOGIT ? p.kv_logit + seg * p.idx_len : nullptr;

  float qf[G][8];
  if (MODE != MODE_LOGIT) {
    const uint16_t* qb = (const uint16_t*)p.q + (int64_t)b * p.q_stride_b + (int64_t)h * G * kHeadDim + 8 * j;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      u32x4 v = *(const u32x4*)(qb + g * kHeadDim);
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[g][i] = Elem<DT>::get(v, i);
    }
  }

  const int64_t head_off = (int64_t)b * p.kv_stride_b + (int64_t)h * p.kv_stride_h + 8 * j;
  const uint16_t* kbase = (const uint16_t*)p.keys + head_off;
  const uint16_t* vbase = (const uint16_t*)p.values + head_off;

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
  }

  // token ids (and supplied logits) of one step; fetched one step ahead so that the row loads of a step
  // do not wait for an index load
  int32_t nid[U];
  float nlg[U];
  auto fetch_ids = [&](int64_t base) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t pos = base + rg * U + u;
      const int64_t pc = pos < end ? pos : (end > 0 ? end - 1 : 0);
      nid[u] = MODE == MODE_DENSE ? 0 : (base < end ? idx[pc] : 0);
      nlg[u] = MODE == MODE_LOGIT ? (base < end ? logit[pc] : 0.0f) : 0.0f;
    }
  };
  fetch_ids(begin);

  for (int64_t base = begin; base < end; base += kStep) {
    int64_t tok[U];
    bool valid[U];
    float lg[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t pos = base + rg * U + u;
      valid[u] = pos < end;
      tok[u] = MODE == MODE_DENSE ? (valid[u] ? pos : end - 1) : (int64_t)nid[u];
      lg[u] = nlg[u];
      if (MODE != MODE_DENSE && (tok[u] < 0 || tok[u] >= p.seq_len)) {  // skip ids outside the cache
        valid[u] = false;                                                // (retrieval_attention.cu:1325)
        tok[u] = 0;
      }
    }
    u32x4 kv[U], vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // whole 256-byte rows per request: the streaming hint suits the dense scan, gathered rows run faster without
      const u32x4* ksrc = (const u32x4*)(kbase + tok[u] * p.kv_stride_n);
      const u32x4* vsrc = (const u32x4*)(vbase + tok[u] * p.kv_stride_n);
      if (MODE != MODE_LOGIT) kv[u] = MODE == MODE_DENSE ? __builtin_nontemporal_load(ksrc) : *ksrc;
      vv[u] = MODE == MODE_DENSE ? __builtin_nontemporal_load(vsrc) : *vsrc;
    }
    if (MODE != MODE_DENSE) fetch_ids(base + kStep);
    if (MODE != MODE_DENSE) {
      // A skipped id had row 0 loaded in its place (and a position past the end of the list the last row): its
      // weight is 0, but 0 * inf would still poison the sum, so such a V row is cleared.  Wave-uniform test:
      // steps made of valid ids only pay one ballot.
      bool skipped = false;
#pragma unroll
      for (int u = 0; u < U; ++u) skipped |= !valid[u];
      if (__ballot(skipped) != 0ull) {
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (!valid[u]) vv[u] = (u32x4){0u, 0u, 0u, 0u};
      }
    }
    float x[G][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float s;
        if (MODE == MODE_LOGIT) {
          s = lg[u] * p.scale_log2e;
        } else {
          float a = 0.0f;
#pragma unroll
          for (int i = 0; i < 8; ++i) a = __builtin_fmaf(qf[g][i], Elem<DT>::get(kv[u], i), a);
          s = row16_sum(a) * p.scale_log2e;
        }
        x[g][u] = valid[u] ? s : -INFINITY;
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mx = m[g];
#pragma unroll
      for (int u = 0; u < U; ++u) mx = fmaxf(mx, x[g][u]);
      if (mx == -INFINITY) continue;  // nothing valid so far
      const float alpha = __builtin_amdgcn_exp2f(m[g] - mx);  // m = -inf -> 0
      m[g] = mx;
      l[g] *= alpha;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[g][i] *= alpha;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float pu = __builtin_amdgcn_exp2f(x[g][u] - mx);  // invalid -> 0
        l[g] += pu;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = __builtin_fmaf(pu, Elem<DT>::get(vv[u], i), acc[g][i]);
      }
    }
  }

  // merge the 16 row-group states, one query head at a time
  const int64_t row0 = ((int64_t)b * p.num_kv_heads + h) * G;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) sh_acc[rg][8 * j + i] = acc[g][i];
    if (j == 0) { sh_m[rg] = m[g]; sh_l[rg] = l[g]; }
    __syncthreads();
    if (tid < kHeadDim) {
      float M = -INFINITY;
#pragma unroll
      for (int r = 0; r < kAttnRowGroups; ++r) M = fmaxf(M, sh_m[r]);
      float L = 0.0f, o = 0.0f;
      if (M != -INFINITY) {
#pragma unroll
        for (int r = 0; r < kAttnRowGroups; ++r) {
          const float w = __builtin_amdgcn_exp2f(sh_m[r] - M);
          L += sh_l[r] * w;
          o += sh_acc[r][tid] * w;
        }
      }
      if (p.out) {
        // the only split of its row: what the combine would compute from this one partial (weight 2^0)
        const float r = L > 0.0f ? o / L : 0.0f;
        uint16_t* out = (uint16_t*)p.out + (int64_t)b * p.out_stride_b + ((int64_t)h * G + g) * kHeadDim;
        out[tid] = p.out_dtype == TKA_F16 ? Elem<TKA_F16>::narrow(r) : Elem<TKA_BF16>::narrow(r);
        if (p.out_lse && tid == 0)
          p.out_lse[row0 + g] = L > 0.0f ? (M + __builtin_log2f(L)) * 0.69314718055994531f : -INFINITY;
      } else {
        const int64_t slot = (row0 + g) * p.num_splits + split;
        p.part_acc[slot * kHeadDim + tid] = o;
        if (tid == 0) { p.part_m[slot] = M; p.part_l[slot] = L; }
      }
    }
  }
}

// lse_combine_kernel: one workgroup per output row (lse_combine.hpp).
template <int ODT>
__global__ __launch_bounds__(kCombineThreads) void lse_combine_kernel(CombineParams p) {
  __shared__ CombineLds sh;
  lse_combine_row<ODT>(p, (int)blockIdx.x, sh);
}

template <int DT, int MODE>
int launch_partial_g(const AttnParams& p, dim3 grid, hipStream_t stream) {
  switch (p.group) {
    case 1: attn_partial_kernel<DT, 1, MODE><<<grid, kAttnThreads, 0, stream>>>(p); break;
    case 2: attn_partial_kernel<DT, 2, MODE><<<grid, kAttnThreads, 0, stream>>>(p); break;
    case 4: attn_partial_kernel<DT, 4, MODE><<<grid, kAttnThreads, 0, stream>>>(p); break;
    case 8: attn_partial_kernel<DT, 8, MODE><<<grid, kAttnThreads, 0, stream>>>(p); break;
    default: return TKA_EUNSUPPORTED;
  }
  return hip_status(hipGetLastError());
}

template <int DT>
int launch_partial_dt(const AttnParams& p, dim3 grid, hipStream_t stream) {
  if (p.kv_logit) {
    if (p.group != 1) return TKA_EUNSUPPORTED;
    attn_partial_kernel<DT, 1, MODE_LOGIT><<<grid, kAttnThreads, 0, stream>>>(p);
    return hip_status(hipGetLastError());
  }
  if (p.kv_idx) return launch_partial_g<DT, MODE_INDEXED>(p, grid, stream);
  return launch_partial_g<DT, MODE_DENSE>(p, grid, stream);
}

}  // namespace

int launch_attn_partial(const AttnParams& p0, int dtype, hipStream_t stream) {
  AttnParams p = p0;
  // The dense scan where a head's rows lie a multiple of 4 KB apart (16 or 32 KV heads in a cache laid out
  // [token][head][128]): the heads in the grid's x, so that the workgroups that run together take the same tokens of all heads
  // instead of long runs of a few heads, which crowd the same memory channels (one query head per KV head: 2 x 16 heads x
  // 131072 tokens 375 -> 345 us, 32 heads 417 -> 361, 16 x 65536 115 -> 95).  Other strides lose 1-5 % that way and keep
  // the splits in x (4 x 8 x 131072: 335 against 330).
  p.head_fastest = !p.kv_idx && !p.kv_logit && p.num_splits <= 65535 && (p.kv_stride_n * 2) % 4096 == 0 ? 1 : 0;
  dim3 grid((unsigned)p.num_splits, (unsigned)p.num_kv_heads, (unsigned)p.batch);
  if (p.head_fastest) grid = dim3((unsigned)p.num_kv_heads, (unsigned)p.num_splits, (unsigned)p.batch);
  LaunchTimer timer(p.kv_logit ? "attn_partial_logit" : (p.kv_idx ? "attn_partial_indexed" : "attn_partial_dense"), stream);
  return dtype == TKA_F16 ? launch_partial_dt<TKA_F16>(p, grid, stream) : launch_partial_dt<TKA_BF16>(p, grid, stream);
}

int launch_lse_combine(const CombineParams& p, hipStream_t stream) {
  LaunchTimer timer("lse_combine", stream);
  if (p.out_dtype == TKA_F16)
    lse_combine_kernel<TKA_F16><<<(unsigned)p.rows, kCombineThreads, 0, stream>>>(p);
  else
    lse_combine_kernel<TKA_BF16><<<(unsigned)p.rows, kCombineThreads, 0, stream>>>(p);
  return hip_status(hipGetLastError());
}

}  // namespace tka
