// Scores of a batch of queries over ONE key cache on the matrix cores - the "skinny GEMM" form of the batch
// pipeline of the reference's operator (retrieval_attention.cu:654-896: one cluster per head loops over the
// batch entries; here one pass over the keys of a head serves up to 32 entries).
//
//     S[token][entry] = sum_d K[token][head][d] * q[entry][head][d]          (then one multiply by `scale`)
//
// as v_mfma_f32_16x16x32: A = 16 key rows (lane = row, 16 bytes of it per 32-wide block of d), B = the queries
// of 16 batch entries (kept in registers for the whole kernel), four MFMAs per 16 x 16 tile of scores, fp32
// accumulation inside the matrix unit.  Products of 16-bit inputs are exact in fp32; the ORDER in which the
// unit adds the 128 of them is not the 16-lane order of gemv_scores.hip, so these scores agree with the
// canonical ones to a few units in the last place, not bit for bit - which is why this kernel is opt-in
// (tka_gemv_topk_args.score_mode) and the selection that follows it is exact on the scores it produced.
// The VALU kernel needs B * 128 multiply-adds per row and lane group and is bound by them from about 16
// entries on; this one is bound by the key stream and the score stores.
//
// Workgroup: 4 waves, 256 rows per step; a wave takes 64 rows as four 16-row tiles, 16 loads of 16 bytes in
// flight per lane.  Lane (n, j) of a tile ends with the scores of rows 4j .. 4j+3 for entry n: one 16-byte store.
// Measured on MI355X (the operator's shape: 8192 keys x 32 heads, 67 MB, resident in the Infinity Cache): 15.9 us
// at 4 entries, 18.0 at 16, 22.6 at 32 (the canonical kernel: 14.7, 27.9, 49.4); at 32 entries the launch moves
// 67 MB of keys and 34 MB of scores.  Two or one tile per wave and step, and 512 to 2048 rows per workgroup,
// were all slower (24.9 - 30.0 us at 32 entries).
#include "kernels.hpp"

namespace tka {

namespace {

constexpr int kMfmaThreads = 256;
constexpr int kMfmaRowsPerWave = 64;
constexpr int kMfmaRowsPerStep = (kMfmaThreads / kWave) * kMfmaRowsPerWave;   // 256

template <int DT>
__device__ __forceinline__ f32x4 mfma_16x16x32(const u32x4& a, const u32x4& b, const f32x4& c) {
  if constexpr (DT == TKA_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// NB: 16-entry batch tiles per workgroup (1 or 2).  Grid: 1-D over (head, row tile, batch tile), batch tile fastest.
template <int DT, int NB>
__global__ __launch_bounds__(kMfmaThreads) void gemv_scores_mfma_kernel(GemvParams p, int row_tiles, int batch_tiles) {
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int n = lane & 15;   // key row of the tile (A), batch entry of the tile (B, result)
  const int j = lane >> 4;   // 8 of every 32 values of d (A, B); rows 4j .. 4j+3 (result)
  uint32_t id = blockIdx.x;
  if (gridDim.x % 8 == 0) id = (id % 8) * (gridDim.x / 8) + id / 8;   // neighbours in the grid share rows: same XCD
  const int bt = (int)(id % (uint32_t)batch_tiles);
  const int tile = (int)((id / (uint32_t)batch_tiles) % (uint32_t)row_tiles);
  const int h = (int)(id / ((uint32_t)batch_tiles * (uint32_t)row_tiles));
  const int b0 = bt * 16 * NB;
  const int64_t n_rows = p.chunk_len * p.num_chunks;
  const int64_t t_begin = (int64_t)tile * p.tokens_per_wg;
  int64_t t_end = t_begin + p.tokens_per_wg;
  if (t_end > n_rows) t_end = n_rows;

  // B operand: entry b0 + 16 nb + n, values d = 32 kb + 8 j .. + 7 (zero for entries beyond the batch)
  u32x4 qfrag[NB][4];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int b = b0 + 16 * nb + n;
    const uint16_t* qb = (const uint16_t*)p.q + (int64_t)(b < p.batch ? b : 0) * p.q_stride_b + (int64_t)h * kHeadDim + 8 * j;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      u32x4 v = *(const u32x4*)(qb + 32 * kb);
      if (b >= p.batch) v = (u32x4){0u, 0u, 0u, 0u};
      qfrag[nb][kb] = v;
    }
  }
  const uint16_t* kbase = (const uint16_t*)p.keys + (int64_t)h * p.key_stride_h + 8 * j;
  const bool vec_ok = (n_rows & 3) == 0 && (((uintptr_t)p.scores) & 15u) == 0;

  for (int64_t base = t_begin + wave * kMfmaRowsPerWave; base < t_end; base += kMfmaRowsPerStep) {
    u32x4 kf[4][4];   // [16-row tile][32-wide block of d]
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int64_t t = base + 16 * x + n;
      const uint16_t* row = kbase + (t < t_end ? t : t_end - 1) * p.key_stride_n;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) kf[x][kb] = *(const u32x4*)(row + 32 * kb);
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) acc = mfma_16x16x32<DT>(kf[x][kb], qfrag[nb][kb], acc);
        // acc[i] = score of row base + 16x + 4j + i for entry b0 + 16nb + n
        const int b = b0 + 16 * nb + n;
        const int64_t t0 = base + 16 * x + 4 * j;
        if (b < p.batch && t0 < t_end) {
          float* out = p.scores + ((int64_t)b * p.num_kv_heads + h) * n_rows + t0;
          if (vec_ok && t0 + 3 < t_end) {
            *(f32x4*)out = acc * p.scale;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (t0 + i < t_end) out[i] = acc[i] * p.scale;
          }
        }
      }
    }
  }
}

}  // namespace

// Keys shared by the batch (key_stride_b == 0), one query head per KV head, plain scores [batch][head][rows].
int launch_gemv_scores_mfma(const GemvParams& p0, int dtype, hipStream_t stream) {
  if (p0.key_stride_b != 0 || p0.cluster_ids || !p0.scores || p0.group != 1) return TKA_EINVAL;
  GemvParams p = p0;
  const int64_t n_rows = p.chunk_len * p.num_chunks;
  p.tokens_per_wg = kMfmaRowsPerStep;
  const int nb = p.batch > 16 ? 2 : 1;
  const int64_t row_tiles = (n_rows + p.tokens_per_wg - 1) / p.tokens_per_wg;
  const int64_t batch_tiles = (p.batch + 16 * nb - 1) / (16 * nb);
  const int64_t wgs = row_tiles * batch_tiles * p.num_kv_heads;
  if (wgs > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  LaunchTimer timer("gemv_scores_mfma", stream);
#define TKA_LAUNCH_MFMA(DT, NB) \
  gemv_scores_mfma_kernel<DT, NB><<<(unsigned)wgs, kMfmaThreads, 0, stream>>>(p, (int)row_tiles, (int)batch_tiles)
  if (dtype == TKA_F16) {
    if (nb == 2) TKA_LAUNCH_MFMA(TKA_F16, 2);
    else TKA_LAUNCH_MFMA(TKA_F16, 1);
  } else {
    if (nb == 2) TKA_LAUNCH_MFMA(TKA_BF16, 2);
    else TKA_LAUNCH_MFMA(TKA_BF16, 1);
  }
#undef TKA_LAUNCH_MFMA
  return hip_status(hipGetLastError());
}

}  // namespace tka
