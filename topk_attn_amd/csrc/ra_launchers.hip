// The thirty reference-named launchers of the retrieval_attention op (bind.cpp:5-243; defined in the
// reference at retrieval_attention.cu:1984-2282).  The six hand-off variants of the reference (DSM,
// global, pipelined x2, two kernels, gather + dense) compute one function, so all of them run the
// same path here: chunked GEMV + per-chunk top-k, then softmax over the survivors with gathered P.V.
#include <stdlib.h>

#include <mutex>

#include "../../include/topk_attn_ra_launchers.h"
#include "common.hpp"

namespace {

constexpr int kRaHeads = 32;       // retrieval_attention.cu:30
constexpr int kRaSeqLen = 8192;    // retrieval_attention.cu:32
constexpr int kRaChunks = 4;       // retrieval_attention.cu:34

// One workspace per device, created on first use and grown on demand; never freed before exit.
struct DeviceWorkspace {
  void* ptr = nullptr;
  size_t bytes = 0;
};
DeviceWorkspace g_ws[64];
std::mutex g_ws_mutex;

void run(const void* q, const void* k, const void* v, void* out, int batch, int topk) {
  tka_ra_args a = {};
  a.q = q;
  a.keys = k;
  a.values = v;
  a.out = out;
  a.dtype = TKA_F16;
  a.batch = batch;
  a.num_heads = kRaHeads;
  a.head_dim = TKA_HEAD_DIM;
  a.topk_per_chunk = topk;
  a.num_chunks = kRaChunks;
  a.softmax_mode = TKA_SOFTMAX_RAW_EXP;
  const char* env = getenv("TKA_BENCH_PRINT");
  a.bench_print = env && env[0] == '1';
  static const bool matrix_scores = [] {   // TKA_RA_SCORE_MODE=1, read once: scoring on the matrix cores
    const char* e = getenv("TKA_RA_SCORE_MODE");
    return e && e[0] == '1' && e[1] == 0;
  }();
  a.score_mode = matrix_scores ? TKA_SCORE_MATRIX : TKA_SCORE_CANONICAL;
  a.seq_len = kRaSeqLen;
  a.scale = 1.0f;
  a.stream = nullptr;  // the reference launches on the default stream
  const size_t need = tka_retrieval_attention_workspace_bytes(&a);
  int dev = 0;
  int rc = TKA_EHIP;
  if (need != 0 && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    DeviceWorkspace& w = g_ws[dev];
    if (w.bytes < need) {
      if (w.ptr) (void)hipFree(w.ptr);
      w.ptr = nullptr;
      w.bytes = 0;
      if (hipMalloc(&w.ptr, need) == hipSuccess) w.bytes = need;
    }
    if (w.bytes >= need) {
      a.workspace = w.ptr;
      a.workspace_bytes = w.bytes;
      rc = tka_retrieval_attention(&a);
    }
  } else if (need == 0) {
    rc = TKA_EINVAL;
  }
  if (rc != TKA_OK) fprintf(stderr, "launch_retrieval_attention(topk=%d, batch=%d): %s\n", topk, batch, tka_status_string(rc));
}

}  // namespace

#define TKA_RA_DEFINE(variant, topk)                                                                          \
  void launch_retrieval_attention##variant##_##topk(const void* query, const void* key_cache,                \
                                                    const void* value_cache, void* output, int batch_size) { \
    run(query, key_cache, value_cache, output, batch_size, topk);                                             \
  }
#define TKA_RA_DEFINE_ALL(variant) \
  TKA_RA_DEFINE(variant, 32)       \
  TKA_RA_DEFINE(variant, 128)      \
  TKA_RA_DEFINE(variant, 256)      \
  TKA_RA_DEFINE(variant, 512)      \
  TKA_RA_DEFINE(variant, 1024)

extern "C" {
TKA_RA_DEFINE_ALL()
TKA_RA_DEFINE_ALL(_global)
TKA_RA_DEFINE_ALL(_pipelined)
TKA_RA_DEFINE_ALL(_pipelined_global)
TKA_RA_DEFINE_ALL(_two_kernels)
TKA_RA_DEFINE_ALL(_gather_baseline)
}
