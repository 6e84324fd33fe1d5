// A caller written the way the reference's extension is (retrieval_attn/bind.cpp:5-43): it declares the
// launchers itself, with C++ linkage and `half` pointers, includes no header of this library, and is compiled by
// the host compiler alone.  That it links against libtka.so is the check; run on a GPU it also calls one
// launcher through that declaration and compares the output with the C symbol's, bit for bit.
//
//   tka_bind_link_check            link check only: prints the addresses of the thirty symbols it resolved
//   tka_bind_link_check run        one call each way on device 0 (needs a GPU)
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#define DECLARE_AS_BIND_CPP(variant, topk)                                                                  \
  void launch_retrieval_attention##variant##_##topk(const half* query, const half* key_cache,               \
                                                    const half* value_cache, half* output, int batch_size);
#define DECLARE_ALL(variant) \
  DECLARE_AS_BIND_CPP(variant, 32) DECLARE_AS_BIND_CPP(variant, 128) DECLARE_AS_BIND_CPP(variant, 256) \
  DECLARE_AS_BIND_CPP(variant, 512) DECLARE_AS_BIND_CPP(variant, 1024)
DECLARE_ALL()
DECLARE_ALL(_global)
DECLARE_ALL(_pipelined)
DECLARE_ALL(_pipelined_global)
DECLARE_ALL(_two_kernels)
DECLARE_ALL(_gather_baseline)

// the C symbol of one of them (what a cgo / ctypes binding reaches), for the comparison
extern "C" void launch_retrieval_attention_two_kernels_128(const void*, const void*, const void*, void*, int);

typedef void (*launcher_t)(const half*, const half*, const half*, half*, int);
#define ENTRY(variant, topk) {"launch_retrieval_attention" #variant "_" #topk, &launch_retrieval_attention##variant##_##topk},
#define ENTRIES(variant) ENTRY(variant, 32) ENTRY(variant, 128) ENTRY(variant, 256) ENTRY(variant, 512) ENTRY(variant, 1024)
static const struct { const char* name; launcher_t fn; } kLaunchers[] = {
    ENTRIES() ENTRIES(_global) ENTRIES(_pipelined) ENTRIES(_pipelined_global) ENTRIES(_two_kernels) ENTRIES(_gather_baseline)};

static uint16_t f32_to_f16_bits(float f) {   // round to nearest even; normal range only (|f| < 1 here)
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const int32_t e = (int32_t)((u >> 23) & 0xff) - 127 + 15;
  uint32_t m = u & 0x7fffffu;
  if (e <= 0) return (uint16_t)sign;
  uint32_t h = ((uint32_t)e << 10) | (m >> 13);
  const uint32_t rest = m & 0x1fffu;
  if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) ++h;
  return (uint16_t)(sign | h);
}

int main(int argc, char** argv) {
  const int n = (int)(sizeof kLaunchers / sizeof kLaunchers[0]);
  if (argc < 2 || strcmp(argv[1], "run") != 0) {
    for (int i = 0; i < n; ++i) printf("%s %p\n", kLaunchers[i].name, (void*)kLaunchers[i].fn);
    printf("linked %d launchers declared as in bind.cpp\n", n);
    return n == 30 ? 0 : 1;
  }
  const int batch = 2, heads = 32, dim = 128, seq = 8192;   // retrieval_attention.cu:30-32
  const size_t nq = (size_t)batch * heads * dim, nkv = (size_t)seq * heads * dim;
  std::vector<uint16_t> q(nq), k(nkv), v(nkv);
  uint32_t s = 12345u;
  auto next = [&]() { s = s * 1664525u + 1013904223u; return ((float)(s >> 8) / 8388608.0f - 1.0f) * 0.3f; };
  for (auto& x : q) x = f32_to_f16_bits(next());
  for (auto& x : k) x = f32_to_f16_bits(next());
  for (auto& x : v) x = f32_to_f16_bits(next());
  half *dq, *dk, *dv, *out_cxx, *out_c;
  if (hipSetDevice(0) != hipSuccess || hipMalloc((void**)&dq, nq * 2) != hipSuccess || hipMalloc((void**)&dk, nkv * 2) != hipSuccess ||
      hipMalloc((void**)&dv, nkv * 2) != hipSuccess || hipMalloc((void**)&out_cxx, nq * 2) != hipSuccess ||
      hipMalloc((void**)&out_c, nq * 2) != hipSuccess) {
    fprintf(stderr, "no GPU memory\n");
    return 2;
  }
  bool ok = hipMemcpy(dq, q.data(), nq * 2, hipMemcpyHostToDevice) == hipSuccess;
  ok = ok && hipMemcpy(dk, k.data(), nkv * 2, hipMemcpyHostToDevice) == hipSuccess;
  ok = ok && hipMemcpy(dv, v.data(), nkv * 2, hipMemcpyHostToDevice) == hipSuccess;
  ok = ok && hipMemset(out_cxx, 0, nq * 2) == hipSuccess && hipMemset(out_c, 0xff, nq * 2) == hipSuccess;
  if (!ok) {
    fprintf(stderr, "copy to the device failed\n");
    return 2;
  }
  printf("[case] launch_retrieval_attention_two_kernels_128 through its bind.cpp declaration, batch %d\n", batch);
  fflush(stdout);
  launch_retrieval_attention_two_kernels_128(dq, dk, dv, out_cxx, batch);                                    // C++ linkage
  launch_retrieval_attention_two_kernels_128((const void*)dq, (const void*)dk, (const void*)dv, (void*)out_c, batch);   // C symbol
  if (hipDeviceSynchronize() != hipSuccess) {
    fprintf(stderr, "device error\n");
    return 2;
  }
  std::vector<uint16_t> a(nq), b(nq);
  if (hipMemcpy(a.data(), out_cxx, nq * 2, hipMemcpyDeviceToHost) != hipSuccess ||
      hipMemcpy(b.data(), out_c, nq * 2, hipMemcpyDeviceToHost) != hipSuccess) {
    fprintf(stderr, "copy from the device failed\n");
    return 2;
  }
  size_t nonzero = 0;
  for (size_t i = 0; i < nq; ++i) nonzero += (a[i] & 0x7fffu) != 0;
  const bool same = memcmp(a.data(), b.data(), nq * 2) == 0;
  printf("outputs %s, %zu of %zu elements non-zero\n", same ? "identical" : "DIFFER", nonzero, nq);
  return same && nonzero > nq / 2 ? 0 : 1;
}
