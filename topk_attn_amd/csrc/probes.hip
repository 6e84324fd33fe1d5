// Read probes: what the memory system gives to the access patterns of the two kernels that carry the bytes of the
// decode step, with nothing else in the kernel (no arithmetic beyond an xor of the loaded words, no stores).
//   stream   rows of 256 B of one KV head per workgroup (16 lanes per row, eight 16-byte loads in flight per lane, a
//            chosen number of rounds per wave): the candidate GEMV's shape is 512 threads x 2 rounds;
//   gather   the rows of a token list, K and V, a 16-lane group per token, eight tokens in flight per group: the
//            pattern of the gathered attention.
// The figures are the reference for the achieved bandwidth of those kernels (bench.py --workload probe-stream /
// probe-gather).  No counterpart in the reference.
#include "kernels.hpp"

namespace tka {

namespace {

template <int THREADS, bool NT>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(8, 8))) void probe_stream_kernel(ProbeParams p, int rounds, int slices_per_seg) {
  constexpr int kRowsPerRound = THREADS / 16 * 8;
  const uint32_t seg = blockIdx.x / (uint32_t)slices_per_seg, sl = blockIdx.x % (uint32_t)slices_per_seg;   // all workgroups of a head before the next
  const int h = (int)(seg % (uint32_t)p.num_heads), b = (int)(seg / (uint32_t)p.num_heads);
  const int j = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const int64_t first = (int64_t)sl * kRowsPerRound * rounds;
  const unsigned char* base = (const unsigned char*)p.base + 2 * ((int64_t)b * p.stride_b + (int64_t)h * p.stride_h) + 16 * j;
  uint32_t acc = 0;
  for (int it = 0; it < rounds; ++it) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      int64_t t = first + (int64_t)it * kRowsPerRound + rg * 8 + u;
      t = t < p.seq_len ? t : p.seq_len - 1;
      const u32x4* a = (const u32x4*)(base + 2 * t * p.stride_n);
      v[u] = NT ? __builtin_nontemporal_load(a) : *a;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  if (acc == 0x12345678u) p.sink[0] = acc;   // (keeps the loads alive; the caches hold other values)
}

// One workgroup of 256 threads per `tokens_per_wg` ids of a (batch entry, head) list.
__global__ __launch_bounds__(256) void probe_gather_kernel(ProbeParams p, int tokens_per_wg, int wgs_per_list) {
  const uint32_t list = blockIdx.x / (uint32_t)wgs_per_list, part = blockIdx.x % (uint32_t)wgs_per_list;
  const int h = (int)(list % (uint32_t)p.num_heads), b = (int)(list / (uint32_t)p.num_heads);
  const int j = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const int32_t* idx = p.idx + (int64_t)list * p.idx_len;
  const int begin = (int)part * tokens_per_wg, end = min(begin + tokens_per_wg, p.idx_len);
  const int64_t head_off = 2 * ((int64_t)b * p.stride_b + (int64_t)h * p.stride_h) + 16 * j;
  const unsigned char* kb = (const unsigned char*)p.base + head_off;
  const unsigned char* vb = (const unsigned char*)p.base2 + head_off;
  uint32_t acc = 0;
  for (int base = begin; base < end; base += 16 * 8) {
    u32x4 kv[8], vv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int pos = base + rg * 8 + u;
      int64_t t = idx[pos < end ? pos : end - 1];
      t = t >= 0 && t < p.seq_len ? t : 0;
      kv[u] = *(const u32x4*)(kb + 2 * t * p.stride_n);
      vv[u] = *(const u32x4*)(vb + 2 * t * p.stride_n);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += kv[u][0] ^ kv[u][3] ^ vv[u][1] ^ vv[u][2];
  }
  if (acc == 0x12345678u) p.sink[0] = acc;
}

}  // namespace

int launch_probe_stream(const ProbeParams& p, int threads, int rounds, bool nontemporal, hipStream_t stream) {
  if ((threads != 256 && threads != 512) || rounds < 1 || rounds > 64) return TKA_EINVAL;
  const int64_t rows_per_wg = (int64_t)threads / 16 * 8 * rounds;
  const int64_t slices = (p.seq_len + rows_per_wg - 1) / rows_per_wg, wgs = slices * p.num_heads * p.batch;
  if (wgs > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  LaunchTimer timer("probe_stream", stream);
  if (threads == 512) {
    if (nontemporal) probe_stream_kernel<512, true><<<(unsigned)wgs, 512, 0, stream>>>(p, rounds, (int)slices);
    else probe_stream_kernel<512, false><<<(unsigned)wgs, 512, 0, stream>>>(p, rounds, (int)slices);
  } else {
    if (nontemporal) probe_stream_kernel<256, true><<<(unsigned)wgs, 256, 0, stream>>>(p, rounds, (int)slices);
    else probe_stream_kernel<256, false><<<(unsigned)wgs, 256, 0, stream>>>(p, rounds, (int)slices);
  }
  return hip_status(hipGetLastError());
}

int launch_probe_gather(const ProbeParams& p, int tokens_per_wg, hipStream_t stream) {
  if (tokens_per_wg < 1 || !p.idx || !p.base2 || p.idx_len < 1) return TKA_EINVAL;
  const int64_t per_list = ((int64_t)p.idx_len + tokens_per_wg - 1) / tokens_per_wg, wgs = per_list * p.num_heads * p.batch;
  if (wgs > 0x7fffffffLL) return TKA_EUNSUPPORTED;
  LaunchTimer timer("probe_gather", stream);
  probe_gather_kernel<<<(unsigned)wgs, 256, 0, stream>>>(p, tokens_per_wg, (int)per_list);
  return hip_status(hipGetLastError());
}

}  // namespace tka
