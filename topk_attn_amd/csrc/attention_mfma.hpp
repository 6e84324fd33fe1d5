// Tile loop of the matrix-core decode attention (grouped queries, G = 2, 4 or 8 query heads per KV head), shared by the
// kernel that reads its token list from memory (attention_mfma.hip) and the one that selects the tokens itself
// (attention_select.hip).  See attention_mfma.hip for the operand layout.
#pragma once
#include "kernels.hpp"

namespace tka {
namespace mfma_attn {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kTile = 32;               // tokens per wave tile
constexpr int kStep = kWaves * kTile;   // positions per workgroup step

template <int DT>
struct Mfma;
template <>
struct Mfma<TKA_F16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    const f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
};
template <>
struct Mfma<TKA_BF16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& a, const u32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    return (uint32_t)Elem<TKA_BF16>::narrow(lo) | ((uint32_t)Elem<TKA_BF16>::narrow(hi) << 16);
  }
};

// token of contraction slot (quarter j, s) inside a 32-token tile
__device__ __forceinline__ int slot_token(int j, int s) { return s < 4 ? 4 * j + s : 16 + 4 * j + (s - 4); }

// Attention of one workgroup (kThreads threads) over the positions [begin, end) of a token list (`idx`, in memory or in
// LDS; INDEXED = false: the positions are the tokens) for the G query heads of KV head h of batch entry b; writes the
// fp32 partial (m, l, acc[128]) of every head to slot `split` of its row.  Every thread of the workgroup must call it.
// LDS of attend(): written only behind its tile loop, so the caller may have used the memory for something else before.
template <int G>
struct AttendLds {
  float acc[kWaves][G][kHeadDim];
  float m[kWaves][G];
  float l[kWaves][G];
};

template <int DT, int G, bool INDEXED>
__device__ __forceinline__ void attend(const AttnParams& p, const int32_t* idx, int64_t begin, int64_t end, int b, int h, int split,
                                       AttendLds<G>& sh) {
  float (&sh_acc)[kWaves][G][kHeadDim] = sh.acc;
  float (&sh_m)[kWaves][G] = sh.m;
  float (&sh_l)[kWaves][G] = sh.l;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int n = lane & 15;   // token row (scores) / query head (softmax) / output dim block (values)
  const int j = lane >> 4;   // quarter: 8 contraction elements of every 32
  // Q^T fragments: head n (zero for the padding heads), dims 32*kb + 8j .. +7
  u32x4 qfrag[4];
  {
    const uint16_t* qb = (const uint16_t*)p.q + (int64_t)b * p.q_stride_b + ((int64_t)h * G + (n < G ? n : 0)) * kHeadDim + 8 * j;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      u32x4 v = *(const u32x4*)(qb + 32 * kb);
      if (n >= G) v = (u32x4){0u, 0u, 0u, 0u};
      qfrag[kb] = v;
    }
  }

  const int64_t head_off = (int64_t)b * p.kv_stride_b + (int64_t)h * p.kv_stride_h;
  const uint16_t* kbase = (const uint16_t*)p.keys + head_off + 8 * j;    // + token*stride + 32*kb
  const uint16_t* vbase = (const uint16_t*)p.values + head_off + 8 * n;  // + token*stride

  float m_run = -INFINITY, l_run = 0.0f;   // head n; l_run is this quarter's share of the sum
  f32x4 acc[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int64_t tile = begin + wave * kTile; tile < end; tile += kStep) {
    // ---- token ids: rows n and 16+n for the score tiles, the eight slot tokens of quarter j for V
    int64_t tk[2];
    bool okk[2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int64_t pos = tile + 16 * x + n;
      okk[x] = pos < end;
      const int64_t pc = okk[x] ? pos : end - 1;
      int64_t t = INDEXED ? (int64_t)idx[pc] : pc;
      if (INDEXED && (t < 0 || t >= p.seq_len)) { okk[x] = false; t = 0; }  // ids outside the cache are skipped
      tk[x] = t;
    }
    int64_t tv[8];
    bool okv[8];
    bool skipped = false;   // an id outside the cache among this lane's slots
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int64_t pos = tile + slot_token(j, s);
      okv[s] = pos < end;
      const int64_t pc = okv[s] ? pos : end - 1;
      int64_t t = INDEXED ? (int64_t)idx[pc] : pc;
      if (INDEXED && (t < 0 || t >= p.seq_len)) { okv[s] = false; t = 0; skipped = true; }
      tv[s] = t;
    }
    // ---- loads: 8 x 16 B of K (2 tiles x 4 k-blocks), 8 x 16 B of V (8 rows).  A K request covers half a line
    // per row (the other k-block of the pair asks for the other half): with the non-temporal hint the line
    // was fetched twice (dense c3: 87 -> 80 us without it).  V requests cover whole rows; streaming them with
    // the hint is right for the dense scan, while the gathered rows of the indexed form run faster without.
    u32x4 kf[2][4], vr[8];
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
        kf[x][kb] = *(const u32x4*)(kbase + tk[x] * p.kv_stride_n + 32 * kb);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const u32x4* src = (const u32x4*)(vbase + tv[s] * p.kv_stride_n);
      vr[s] = INDEXED ? *src : __builtin_nontemporal_load(src);
    }

    // ---- scores: S[token][head] for the two 16-token tiles
    f32x4 sc[2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      f32x4 d = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) d = Mfma<DT>::run(kf[x][kb], qfrag[kb], d);
      sc[x] = d;
    }
    // lane (head n, quarter j) holds tokens 4j+i (tile 0) and 16+4j+i (tile 1): slot s = 4x + i.
    // Validity of those tokens is okv[s] (same tokens as this quarter's V rows).
    float xs[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) xs[s] = okv[s] ? sc[s >> 2][s & 3] * p.scale_log2e : -INFINITY;
    float tmax = xs[0];
#pragma unroll
    for (int s = 1; s < 8; ++s) tmax = fmaxf(tmax, xs[s]);
    tmax = fmaxf(tmax, __builtin_bit_cast(float, lane_xor<16>(__builtin_bit_cast(uint32_t, tmax))));
    tmax = fmaxf(tmax, __builtin_bit_cast(float, lane_xor<32>(__builtin_bit_cast(uint32_t, tmax))));
    const float m_new = fmaxf(m_run, tmax);
    const bool any = m_new != -INFINITY;
    const float alpha = any ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;  // m_run = -inf -> 0
    float ps[8], psum = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      ps[s] = any ? __builtin_amdgcn_exp2f(xs[s] - m_new) : 0.0f;  // masked -> 0
      psum += ps[s];
    }
    m_run = m_new;
    l_run = l_run * alpha + psum;
    u32x4 pfrag;
#pragma unroll
    for (int w = 0; w < 4; ++w) pfrag[w] = Mfma<DT>::pack(ps[2 * w], ps[2 * w + 1]);
    // bf16 keeps 8 bits of a weight: the rest goes through the matrix cores as a second operand (the products are
    // exact, the sum is fp32), so that a short list of tokens is weighted as precisely as the fp32 sum l above
    u32x4 pfrag_lo;
    if constexpr (DT == TKA_BF16) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float r0 = ps[2 * w] - Elem<DT>::widen((uint16_t)pfrag[w]), r1 = ps[2 * w + 1] - Elem<DT>::widen((uint16_t)(pfrag[w] >> 16));
        pfrag_lo[w] = Mfma<DT>::pack(r0, r1);
      }
    }

    // ---- rescale the accumulators: element i belongs to head 4j+i, whose alpha sits in lane 4j+i
    float ah[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) ah[i] = __shfl(alpha, 4 * j + i, 64);
#pragma unroll
    for (int c = 0; c < 8; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[c][i] *= ah[i];

    // ---- V rows of masked tokens (past the end of the list, or ids outside the cache, whose slot loaded row 0
    // instead) must not reach the product (0 * inf).  Wave-uniform test: full tiles of valid ids skip the selects.
    if (tile + kTile > end || (INDEXED && __ballot(skipped) != 0ull)) {
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (!okv[s]) vr[s] = (u32x4){0u, 0u, 0u, 0u};
    }
    // ---- values: O[head][8n+c] += sum over slots P[head][slot] * V[slot token][8n+c]
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      u32x4 vt;
      const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int w = 0; w < 4; ++w) vt[w] = __builtin_amdgcn_perm(vr[2 * w + 1][c >> 1], vr[2 * w][c >> 1], sel);
      acc[c] = Mfma<DT>::run(pfrag, vt, acc[c]);
      if constexpr (DT == TKA_BF16) acc[c] = Mfma<DT>::run(pfrag_lo, vt, acc[c]);
    }
    (void)okk;
  }

  // ---- per-wave result -> LDS: sum l over the quarters; acc element (c, i) is O[head 4j+i][8n+c]
  float l_tot = l_run;
  l_tot += __builtin_bit_cast(float, lane_xor<16>(__builtin_bit_cast(uint32_t, l_tot)));
  l_tot += __builtin_bit_cast(float, lane_xor<32>(__builtin_bit_cast(uint32_t, l_tot)));
  if (j == 0 && n < G) { sh_m[wave][n] = m_run; sh_l[wave][n] = l_tot; }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int head = 4 * j + i;
    if (head < G) {
#pragma unroll
      for (int c = 0; c < 8; ++c) sh_acc[wave][head][8 * n + c] = acc[c][i];
    }
  }
  __syncthreads();
  const int64_t row0 = ((int64_t)b * p.num_kv_heads + h) * G;
  for (int o = tid; o < G * kHeadDim; o += kThreads) {
    const int g = o / kHeadDim, d = o % kHeadDim;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) M = fmaxf(M, sh_m[w][g]);
    float L = 0.0f, out = 0.0f;
    if (M != -INFINITY) {
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const float wgt = __builtin_amdgcn_exp2f(sh_m[w][g] - M);  // empty wave: exp2(-inf) = 0
        L += sh_l[w][g] * wgt;
        out += sh_acc[w][g][d] * wgt;
      }
    }
    const int64_t slot = (row0 + g) * p.num_splits + split;
    p.part_acc[slot * kHeadDim + d] = out;
    if (d == 0) { p.part_m[slot] = M; p.part_l[slot] = L; }
  }
}

}  // namespace mfma_attn
}  // namespace tka
