// Streaming-read probe in the shape of the candidate GEMV: rows of 256 B at a 2 KB stride (one of 8 KV heads of a
// [B][N][8][128] fp16 cache), one head per workgroup, 16 lanes per row, eight 16-byte loads in flight per lane.
// No arithmetic beyond an xor of the loaded words, no stores: what the memory system gives to a given shape of
// workgroups (threads, rounds of loads per wave, order of the workgroups, load hint, loads into registers or straight
// into LDS).  The figures are the reference for the GEMV kernels' achieved bandwidth.
//   tka_stream_probe [batch=8] [tokens=131072]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                        \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);     \
      std::exit(1);                                                                  \
    }                                                                                \
  } while (0)

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kHeads = 8;
constexpr int kRowBytes = 256;

// THREADS / 16 row groups of 16 lanes, ROUNDS rounds of eight loads per lane: THREADS / 2 * ROUNDS rows per workgroup.
// HEAD_MINOR: the workgroups of the heads of one token range are neighbours in the grid (else all workgroups of a
// head come before those of the next).  NT: non-temporal loads.
template <int THREADS, int ROUNDS, bool HEAD_MINOR, bool NT>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(8, 8))) void read_registers(const unsigned char* p, int slices_per_head,
                                                                                                        unsigned* out) {
  constexpr int kRowsPerRound = THREADS / 16 * 8;
  constexpr int kRows = kRowsPerRound * ROUNDS;
  const int h = HEAD_MINOR ? (int)(blockIdx.x % kHeads) : (int)(blockIdx.x / (unsigned)slices_per_head);
  const int sl = HEAD_MINOR ? (int)(blockIdx.x / kHeads) : (int)(blockIdx.x % (unsigned)slices_per_head);
  const int j = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const size_t stride = (size_t)kHeads * kRowBytes;
  const unsigned char* base = p + (size_t)h * kRowBytes + (size_t)sl * kRows * stride + 16 * j;
  unsigned acc = 0;
  for (int it = 0; it < ROUNDS; ++it) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const u32x4* a = (const u32x4*)(base + (size_t)(it * kRowsPerRound + rg * 8 + u) * stride);
      v[u] = NT ? __builtin_nontemporal_load(a) : *a;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x12345678u) out[0] = acc;   // (keeps the loads alive; the buffer holds other values)
}

// The candidate GEMV's shape (512 threads, two rounds of eight loads per lane: a slice of 512 rows) with the last
// `tail_slices` slices of the grid handled by two workgroups of one round each: does the end of a launch, where
// workgroups that are out of step finish one by one, cost what shorter workgroups there would save?
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(8, 8))) void read_registers_split_tail(const unsigned char* p, int slices_per_head,
                                                                                                              int full_slices, unsigned* out) {
  constexpr int kRowsPerRound = 512 / 16 * 8;
  const bool half = (int)blockIdx.x >= full_slices;
  const int slice = half ? full_slices + ((int)blockIdx.x - full_slices) / 2 : (int)blockIdx.x;
  const int first_round = half ? ((int)blockIdx.x - full_slices) % 2 : 0, rounds = half ? 1 : 2;
  const int h = slice / slices_per_head, sl = slice % slices_per_head;
  const int j = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const size_t stride = (size_t)kHeads * kRowBytes;
  const unsigned char* base = p + (size_t)h * kRowBytes + (size_t)sl * (2 * kRowsPerRound) * stride + 16 * j;
  unsigned acc = 0;
  for (int it = first_round; it < first_round + rounds; ++it) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load((const u32x4*)(base + (size_t)(it * kRowsPerRound + rg * 8 + u) * stride));
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x12345678u) out[0] = acc;
}

// Direct-to-LDS loads (global_load_lds_dwordx4): 256 threads, ROWS rows per workgroup (ROWS * 256 B of LDS), all loads
// of a lane in flight at once, then one pass over the LDS copy.
template <int ROWS>
__global__ __launch_bounds__(256) void read_lds(const unsigned char* p, int slices_per_head, unsigned* out) {
  __shared__ __attribute__((aligned(16))) unsigned char sh[ROWS * kRowBytes];
  const int h = (int)(blockIdx.x / (unsigned)slices_per_head), sl = (int)(blockIdx.x % (unsigned)slices_per_head);
  const int j = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const int wave = threadIdx.x >> 6;
  const size_t stride = (size_t)kHeads * kRowBytes;
  const unsigned char* base = p + (size_t)h * kRowBytes + (size_t)sl * ROWS * stride + 16 * j;
  constexpr int kLoads = ROWS / 16;
  // load u of wave w brings rows 16 u + 4 w .. + 3 to their place in LDS: 1 KB per wave and load, lane l at byte 16 l
#pragma unroll
  for (int u = 0; u < kLoads; ++u) {
    const unsigned char* src = base + (size_t)(u * 16 + rg) * stride;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(sh + (u * 16 + 4 * wave) * kRowBytes), 16, 0, 0);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  unsigned acc = 0;
#pragma unroll
  for (int u = 0; u < kLoads; ++u) {
    const u32x4 v = *(const u32x4*)(sh + (u * 16 + rg) * kRowBytes + 16 * j);
    acc += v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x12345678u) out[0] = acc;
}

unsigned char* g_buf;
unsigned* g_out;
size_t g_rows_per_head, g_bytes;

template <typename F>
float time_us(F launch) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int i = 0; i < 3; ++i) launch();
  CK(hipDeviceSynchronize());
  const int reps = 20;
  CK(hipEventRecord(e0));
  for (int i = 0; i < reps; ++i) launch();
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms = 0.0f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipGetLastError());
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
  return ms * 1000.0f / reps;
}

template <int THREADS, int ROUNDS, bool HEAD_MINOR, bool NT>
void run_registers(const char* what) {
  const int rows = THREADS / 16 * 8 * ROUNDS;
  if (g_rows_per_head % rows) return;
  const int sph = (int)(g_rows_per_head / rows);
  const float us = time_us([&] { read_registers<THREADS, ROUNDS, HEAD_MINOR, NT><<<kHeads * sph, THREADS>>>(g_buf, sph, g_out); });
  std::printf("%-78s %8.1f us  %6.0f GB/s\n", what, us, g_bytes / us / 1e3);
}

void run_split_tail(int tail_slices, const char* what) {
  const int sph = (int)(g_rows_per_head / 512), slices = kHeads * sph;
  if (g_rows_per_head % 512 || tail_slices > slices) return;
  const int full = slices - tail_slices;
  const float us = time_us([&] { read_registers_split_tail<<<full + 2 * tail_slices, 512>>>(g_buf, sph, full, g_out); });
  std::printf("%-78s %8.1f us  %6.0f GB/s\n", what, us, g_bytes / us / 1e3);
}

template <int ROWS>
void run_lds(const char* what) {
  if (g_rows_per_head % ROWS) return;
  const int sph = (int)(g_rows_per_head / ROWS);
  const float us = time_us([&] { read_lds<ROWS><<<kHeads * sph, 256>>>(g_buf, sph, g_out); });
  std::printf("%-78s %8.1f us  %6.0f GB/s\n", what, us, g_bytes / us / 1e3);
}

}  // namespace

int main(int argc, char** argv) {
  const size_t batch = argc > 1 ? (size_t)std::atoll(argv[1]) : 8, tokens = argc > 2 ? (size_t)std::atoll(argv[2]) : 131072;
  if (batch < 1 || tokens < 2048 || tokens % 2048 || batch * tokens > ((size_t)1 << 24)) {
    std::printf("usage: tka_stream_probe [batch] [tokens, a multiple of 2048; batch x tokens up to 16 M]\n");
    return 2;
  }
  g_rows_per_head = batch * tokens;
  g_bytes = g_rows_per_head * kHeads * kRowBytes;
  CK(hipMalloc(&g_buf, g_bytes));
  CK(hipMalloc(&g_out, sizeof(unsigned)));
  CK(hipMemset(g_buf, 1, g_bytes));
  std::printf("rows of 256 B at a 2 KB stride, %zu x %zu tokens x 8 heads = %.1f MB per pass; all workgroups of a head before the next head unless said\n",
              batch, tokens, g_bytes / 1e6);
  run_registers<512, 2, false, true>("512 threads, 2 rounds of 8 loads per lane (512 rows): the candidate GEMV's shape");
  run_registers<512, 2, true, true>("  the same, the heads of a token range next to each other in the grid");
  run_registers<512, 2, false, false>("  the same, loads without the non-temporal hint");
  run_registers<512, 1, false, true>("512 threads, 1 round (256 rows)");
  run_registers<512, 4, false, true>("512 threads, 4 rounds (1024 rows)");
  run_registers<512, 8, false, true>("512 threads, 8 rounds (2048 rows)");
  run_registers<256, 1, false, true>("256 threads, 1 round (128 rows): the dense GEMV's shape");
  run_registers<256, 2, false, true>("256 threads, 2 rounds (256 rows)");
  run_registers<256, 4, false, true>("256 threads, 4 rounds (512 rows)");
  run_registers<256, 8, false, true>("256 threads, 8 rounds (1024 rows)");
  run_registers<128, 8, false, true>("128 threads, 8 rounds (512 rows)");
  run_registers<64, 16, false, true>("64 threads, 16 rounds (512 rows): a wave per slice");
  run_registers<1024, 1, false, true>("1024 threads, 1 round (512 rows)");
  run_lds<64>("direct to LDS, 256 threads, 64 rows (16 KB of LDS) per workgroup");
  run_lds<128>("direct to LDS, 256 threads, 128 rows (32 KB)");
  run_lds<256>("direct to LDS, 256 threads, 256 rows (64 KB)");
  run_registers<512, 2, false, true>("512 threads, 2 rounds again");
  run_split_tail(0, "512 threads, 2 rounds, the rounds as a loop that is not unrolled");
  run_split_tail(1024, "  the same, the last 1024 slices (one resident set) as two workgroups of one round each");
  run_split_tail(4096, "  the same, the last 4096 slices so");
  CK(hipFree(g_buf));
  CK(hipFree(g_out));
  return 0;
}
