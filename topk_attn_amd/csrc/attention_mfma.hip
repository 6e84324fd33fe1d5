// Split-K decode attention for grouped queries (G = 2, 4 or 8 query heads per KV head) on the matrix
// cores.  With a group the score computation is a small dense contraction [tokens x 128] . [128 x G] and
// the value product [G x tokens] . [tokens x 128]; both run as v_mfma_f32_16x16x32 with the query heads
// padded to 16.  Everything else (online softmax in the exp2 domain, baseline_1.cu:406-468 of the
// reference) is VALU work, and the kernel stays bound by the K and V streams.
//
// One workgroup per (split, KV head, batch entry), 4 waves; a wave owns tiles of 32 tokens.
//   scores   A = K rows of 16 tokens (lane = token, 16 B of the row per k-block), B = Q^T; two tiles give
//            lane (head n, quarter j) the logits of tokens 4j..4j+3 and 16+4j..16+4j+3 of the tile;
//   softmax  running max / sum per head, replicated over the four quarters;
//   values   A = P, taken straight from the score registers: contraction slot (j, s) means token
//            4j+s (s < 4) or 16+4j+s-4, so no cross-lane movement; B = V, loaded as full 256-byte rows
//            (lane = 8 output dims of 8 tokens) and transposed inside the lane with byte permutes;
//   output   eight accumulators of 4 registers: O[head 4j+i][dim 8n+c].
#include "attention_mfma.hpp"

namespace tka {

namespace {

using namespace mfma_attn;

// STAGED (indexed form, splits of up to kStagedIds tokens): the split's ids go to LDS in one coalesced trip before the
// first tile, so that a tile's row requests do not wait for a load of their ids first (a tile then costs one round trip
// to memory instead of two: c4's gathered attention 20.4 -> 18.6 us).
constexpr int kStagedIds = 2048;

template <int DT, int G, bool INDEXED, bool STAGED>
__global__ __launch_bounds__(kThreads) void attn_mfma_kernel(AttnParams p) {
  const int split = p.head_fastest ? blockIdx.y : blockIdx.x;
  const int h = p.head_fastest ? blockIdx.x : blockIdx.y;
  const int b = blockIdx.z;
  const int64_t seg = (int64_t)b * p.num_kv_heads + h;
  int64_t count = p.seq_len;
  if (INDEXED) {
    count = p.kv_count ? p.kv_count[seg] : p.idx_len;
    if (count > p.idx_len) count = p.idx_len;
    if (count < 0) count = 0;
  }
  const int64_t begin = (int64_t)split * p.tokens_per_split;
  int64_t end = begin + p.tokens_per_split;
  if (end > count) end = count;
  __shared__ AttendLds<G> sh;
  if constexpr (INDEXED && STAGED) {
    __shared__ int32_t sh_ids[kStagedIds];
    const int32_t* idx = p.kv_idx + seg * p.idx_len + begin;
    const int n = end > begin ? (int)(end - begin) : 0;
    for (int i = threadIdx.x; i < n; i += kThreads) sh_ids[i] = idx[i];
    __syncthreads();
    attend<DT, G, true>(p, sh_ids, 0, n, b, h, split, sh);
  } else {
    attend<DT, G, INDEXED>(p, INDEXED ? p.kv_idx + seg * p.idx_len : nullptr, begin, end, b, h, split, sh);
  }
}

template <int DT, bool INDEXED, bool STAGED>
int launch_g(const AttnParams& p, dim3 grid, hipStream_t stream) {
  switch (p.group) {
    case 2: attn_mfma_kernel<DT, 2, INDEXED, STAGED><<<grid, kThreads, 0, stream>>>(p); break;
    case 4: attn_mfma_kernel<DT, 4, INDEXED, STAGED><<<grid, kThreads, 0, stream>>>(p); break;
    case 8: attn_mfma_kernel<DT, 8, INDEXED, STAGED><<<grid, kThreads, 0, stream>>>(p); break;
    default: return TKA_EUNSUPPORTED;
  }
  return hip_status(hipGetLastError());
}

}  // namespace

// Grouped-query attention partials on the matrix cores (group 2, 4, 8; dense or indexed).
int launch_attn_partial_mfma(const AttnParams& p0, int dtype, hipStream_t stream) {
  AttnParams p = p0;
  // The dense scan of a long cache with sixteen or more KV heads (a head's rows 4 KB or more apart, half a gigabyte or more
  // of keys per batch entry): the splits that run together then take the same tokens of all heads instead of a long run of
  // tokens of a few heads - 2 x 16 heads x 131072 tokens 443 -> 364 us, 32 heads 397 -> 373.  Everywhere else that order is
  // 4-8 % slower (4 x 8 heads x 131072 tokens: 354 against 333 us; 16 heads x 65536 tokens: 86.8 against 83.3).
  const int64_t row_bytes = p.kv_stride_n * 2;
  p.head_fastest = !p.kv_idx && row_bytes >= 4096 && p.seq_len * row_bytes >= (512ll << 20) && p.num_splits <= 65535 ? 1 : 0;
  dim3 grid((unsigned)p.num_splits, (unsigned)p.num_kv_heads, (unsigned)p.batch);
  if (p.head_fastest) grid = dim3((unsigned)p.num_kv_heads, (unsigned)p.num_splits, (unsigned)p.batch);
  LaunchTimer timer(p.kv_idx ? "attn_mfma_indexed" : "attn_mfma_dense", stream);
  // (a split of one step has nothing to gain: each wave asks for its only tile's ids once either way)
  const bool staged = p.kv_idx && p.tokens_per_split <= kStagedIds && p.tokens_per_split > kStep;
  if (dtype == TKA_F16)
    return !p.kv_idx ? launch_g<TKA_F16, false, false>(p, grid, stream)
                     : (staged ? launch_g<TKA_F16, true, true>(p, grid, stream) : launch_g<TKA_F16, true, false>(p, grid, stream));
  return !p.kv_idx ? launch_g<TKA_BF16, false, false>(p, grid, stream)
                   : (staged ? launch_g<TKA_BF16, true, true>(p, grid, stream) : launch_g<TKA_BF16, true, false>(p, grid, stream));
}

}  // namespace tka
