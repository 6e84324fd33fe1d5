// tka_standalone: command-line counterparts of the reference's stand-alone programs, on top of the C ABI of
// libtka.so.  Each subcommand builds the same synthetic problem as the program it stands in for (clustered keys:
// centre + normal noise, seeded mt19937), times 50 launches after 10 warm-ups with events, prints the latency and a
// sample of the result, and with --verify [heads] checks the result against a CPU computation made here:
//
//   gemv_topk       two-level selection, gemv_topk.cu:388-520 (32 heads, 32 clusters of 1280 tokens, top 5 clusters,
//                   top 512 tokens of each)
//   center_only     centre-only selection with expansion, center_only_topk/gemv_topk.cu:465-615 (1024 centroids of
//                   128 tokens, top 64); --centroids / --cluster-len / --topc change the shape
//   baseline_1      selection, then flash-decoding over the selected tokens, then both back to back,
//                   baseline_1.cu:613-723
//   flash_decoding  flash-decoding over a random index list of 2560 tokens per head, flash_decoding.cu:390-480;
//                   --dense attends to all 40 960 tokens instead
//   retrieval_attention   the operator's own program, retrieval_attention.cu:2351-2445: dense attention over the 8192
//                   shared keys as the baseline, then the op for K = 32 ... 1024 per chunk through the
//                   reference-named launchers (default and _global variant), 100 timed launches each; --batch N
//
// The CPU check scores in the library's documented order (16 partial fma chains over 8 dims each, pairwise tree with
// partner distances 8, 4, 2, 1), so selections are compared for equal order, not only as sets as the reference's
// --verify does (gemv_topk.cu:138-170); the set comparison and the recall figure are printed as well.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <numeric>
#include <random>
#include <string>
#include <vector>

#include "topk_attn.h"
#include "topk_attn_ra_launchers.h"

namespace {

constexpr int kHeads = 32, kDim = 128;

#define HIP_OK(call)                                                                               \
  do {                                                                                             \
    hipError_t e_ = (call);                                                                        \
    if (e_ != hipSuccess) {                                                                        \
      std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                                                \
    }                                                                                              \
  } while (0)

#define TKA_CALL(call)                                                                   \
  do {                                                                                   \
    int rc_ = (call);                                                                    \
    if (rc_ != TKA_OK) {                                                                 \
      std::fprintf(stderr, "%s returned %d (%s:%d)\n", #call, rc_, __FILE__, __LINE__); \
      std::exit(2);                                                                      \
    }                                                                                    \
  } while (0)

struct Options {
  bool verify = false;
  int verify_heads = kHeads;
  bool dense = false;
  int centroids = 1024, cluster_len = 128, topc = 64;
  int batch = 1;
  int warmup = 10, iters = 50;
};

uint16_t half_bits(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  std::memcpy(&b, &h, 2);
  return b;
}
float half_value(uint16_t b) {
  _Float16 h;
  std::memcpy(&h, &b, 2);
  return (float)h;
}

template <typename T>
T* to_device(const std::vector<T>& v) {
  T* d = nullptr;
  HIP_OK(hipMalloc(&d, v.size() * sizeof(T)));
  HIP_OK(hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}
void release(void* d) {
  if (d) (void)hipFree(d);
}
template <typename T>
T* device_buffer(size_t n) {
  T* d = nullptr;
  HIP_OK(hipMalloc(&d, (n ? n : 1) * sizeof(T)));
  return d;
}

// mean latency of `launch` in microseconds
double time_launches(const Options& o, const std::function<void()>& launch) {
  for (int i = 0; i < o.warmup; ++i) launch();
  HIP_OK(hipDeviceSynchronize());
  hipEvent_t t0, t1;
  HIP_OK(hipEventCreate(&t0));
  HIP_OK(hipEventCreate(&t1));
  HIP_OK(hipEventRecord(t0, nullptr));
  for (int i = 0; i < o.iters; ++i) launch();
  HIP_OK(hipEventRecord(t1, nullptr));
  HIP_OK(hipEventSynchronize(t1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, t0, t1));
  HIP_OK(hipEventDestroy(t0));
  HIP_OK(hipEventDestroy(t1));
  return (double)ms * 1000.0 / o.iters;
}

// ---- the synthetic problem -------------------------------------------------------------------------------------

struct Problem {
  int centroids, cluster_len;
  std::vector<uint16_t> q;        // [heads][128]
  std::vector<uint16_t> centers;  // [heads][centroids][128]
  std::vector<uint16_t> kv;       // [centroids*cluster_len][heads][128]; empty when with_tokens is false
  int64_t tokens() const { return (int64_t)centroids * cluster_len; }
};

// Centres uniform in (-half_width, half_width), tokens = centre of their cluster + N(0, sigma), queries uniform:
// the recipe of gemv_topk.cu:411-447.
Problem make_problem(int centroids, int cluster_len, bool with_tokens, float half_width = 0.5f, float sigma = 0.05f) {
  Problem p;
  p.centroids = centroids;
  p.cluster_len = cluster_len;
  std::mt19937 rng(12345);
  std::normal_distribution<float> noise(0.0f, sigma);
  std::uniform_real_distribution<float> uni(-half_width, half_width);
  p.centers.resize((size_t)kHeads * centroids * kDim);
  for (auto& c : p.centers) c = half_bits(uni(rng));
  if (with_tokens) {
    p.kv.resize((size_t)p.tokens() * kHeads * kDim);
    for (int c = 0; c < centroids; ++c)
      for (int t = 0; t < cluster_len; ++t)
        for (int h = 0; h < kHeads; ++h) {
          const uint16_t* centre = &p.centers[((size_t)h * centroids + c) * kDim];
          uint16_t* row = &p.kv[(((size_t)c * cluster_len + t) * kHeads + h) * kDim];
          for (int d = 0; d < kDim; ++d) row[d] = half_bits(half_value(centre[d]) + noise(rng));
        }
  }
  p.q.resize((size_t)kHeads * kDim);
  for (auto& x : p.q) x = half_bits(uni(rng));
  return p;
}

// ---- CPU side of --verify --------------------------------------------------------------------------------------

// fp32 score in the library's order: lane j of 16 runs an fma chain over dims 8j..8j+7, the 16 partial sums are
// added pairwise with partner distances 8, 4, 2, 1, one multiply by the scale.
float score_in_order(const uint16_t* q, const uint16_t* row, float scale) {
  float p[16];
  for (int j = 0; j < 16; ++j) {
    float acc = 0.0f;
    for (int i = 0; i < 8; ++i) acc = std::fmaf(half_value(q[8 * j + i]), half_value(row[8 * j + i]), acc);
    p[j] = acc;
  }
  for (int dist = 8; dist >= 1; dist >>= 1)
    for (int j = 0; j < dist; ++j) p[j] = p[j] + p[j + dist];
  return p[0] * scale;
}

// first k positions of the order (score descending, index ascending)
std::vector<int> stable_topk(const std::vector<float>& s, int k) {
  std::vector<int> order(s.size());
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return s[a] > s[b]; });
  order.resize(k);
  return order;
}

// Compares slices of `len` ids: equal order, equal sets, recall.  Prints one line per slice like the reference's
// checker and returns true when every slice holds the same set.
bool compare_slices(const std::vector<int>& cpu, const std::vector<int32_t>& gpu, int heads, int slices, int len,
                    int gpu_row_len) {
  bool sets_equal = true, order_equal = true;
  double recall_sum = 0.0;
  for (int h = 0; h < heads; ++h)
    for (int r = 0; r < slices; ++r) {
      const int* a = &cpu[((size_t)h * slices + r) * len];
      const int32_t* b = &gpu[(size_t)h * gpu_row_len + (size_t)r * len];
      order_equal = order_equal && std::equal(a, a + len, b);
      std::vector<int> sa(a, a + len), sb(b, b + len), common;
      std::sort(sa.begin(), sa.end());
      std::sort(sb.begin(), sb.end());
      std::set_intersection(sa.begin(), sa.end(), sb.begin(), sb.end(), std::back_inserter(common));
      const double recall = (double)common.size() / len;
      recall_sum += recall;
      sets_equal = sets_equal && sa == sb;
      if ((h == 0 && r < 8) || sa != sb)   // a sample of the slices, and every slice that differs
        std::printf("[VERIFY] head=%d cluster-rank=%d recall@%d = %.2f%%\n", h, r, len, recall * 100.0);
    }
  std::printf("Average recall(head-avg over %d heads) = %.2f%%\n", heads, recall_sum / ((double)heads * slices) * 100.0);
  if (sets_equal) std::printf("✓ GPU indices match CPU reference (set equality per cluster).\n");
  else std::printf("✗ GPU indices differ from CPU reference.\n");
  std::printf("%s rank order inside every slice: %s\n", order_equal ? "✓" : "✗", order_equal ? "identical" : "differs");
  return sets_equal && order_equal;
}

// ---- gemv_topk: two-level selection ----------------------------------------------------------------------------

struct TwoLevel {
  static constexpr int kClusters = 32, kClusterLen = 1280, kTopC = 5, kPerCluster = 512;
  static constexpr int kOutPerHead = kTopC * kPerCluster;
  Problem p;
  uint16_t *d_q = nullptr, *d_centers = nullptr, *d_kv = nullptr;
  int32_t* d_out = nullptr;
  void* d_ws = nullptr;
  tka_cluster_topk_args args{};

  TwoLevel() : p(make_problem(kClusters, kClusterLen, true)) {
    d_q = to_device(p.q);
    d_centers = to_device(p.centers);
    d_kv = to_device(p.kv);
    d_out = device_buffer<int32_t>((size_t)kHeads * kOutPerHead);
    args.q = d_q;
    args.centers = d_centers;
    args.keys = d_kv;
    args.dtype = TKA_F16;
    args.num_heads = kHeads;
    args.num_centers = kClusters;
    args.top_c = kTopC;
    args.cluster_len = kClusterLen;
    args.k = kPerCluster;
    args.head_dim = kDim;
    args.scale = 1.0f;   // the reference selects on unscaled scores
    args.key_stride_n = (int64_t)kHeads * kDim;
    args.key_stride_h = kDim;
    args.out_idx = d_out;
    args.workspace_bytes = tka_cluster_gemv_topk_workspace_bytes(&args);
    d_ws = device_buffer<unsigned char>(args.workspace_bytes);
    args.workspace = d_ws;
  }
  void launch() { TKA_CALL(tka_cluster_gemv_topk(&args)); }
  std::vector<int32_t> result() {
    std::vector<int32_t> out((size_t)kHeads * kOutPerHead);
    HIP_OK(hipMemcpy(out.data(), d_out, out.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
    return out;
  }
  // CPU selection of the first `heads` heads: [heads][top_c][k] global token ids
  std::vector<int> cpu_select(int heads) const {
    std::vector<int> out((size_t)heads * kOutPerHead);
    std::vector<float> cs(kClusters), ts(kClusterLen);
    for (int h = 0; h < heads; ++h) {
      const uint16_t* q = &p.q[(size_t)h * kDim];
      for (int c = 0; c < kClusters; ++c) cs[c] = score_in_order(q, &p.centers[((size_t)h * kClusters + c) * kDim], 1.0f);
      const std::vector<int> top = stable_topk(cs, kTopC);
      for (int r = 0; r < kTopC; ++r) {
        const int64_t base = (int64_t)top[r] * kClusterLen;
        for (int t = 0; t < kClusterLen; ++t) ts[t] = score_in_order(q, &p.kv[((size_t)(base + t) * kHeads + h) * kDim], 1.0f);
        const std::vector<int> loc = stable_topk(ts, kPerCluster);
        for (int i = 0; i < kPerCluster; ++i) out[((size_t)h * kTopC + r) * kPerCluster + i] = (int)(base + loc[i]);
      }
    }
    return out;
  }
  ~TwoLevel() {
    release(d_ws); release(d_out); release(d_kv); release(d_centers); release(d_q);
  }
};

int run_gemv_topk(const Options& o) {
  std::printf("Two-level selection: heads=%d dim=%d tokens=%d clusters=%d cluster_len=%d top_clusters=%d top_per_cluster=%d\n",
              kHeads, kDim, TwoLevel::kClusters * TwoLevel::kClusterLen, TwoLevel::kClusters, TwoLevel::kClusterLen,
              TwoLevel::kTopC, TwoLevel::kPerCluster);
  TwoLevel job;
  std::printf("Workspace: %zu bytes\n", job.args.workspace_bytes);
  const double us = time_launches(o, [&] { job.launch(); });
  std::printf("Fused kernel latency: %.3f us\n", us);
  const std::vector<int32_t> out = job.result();
  std::printf("head0 kv_indices[0..31]: ");
  for (int i = 0; i < 32; ++i) std::printf("%d ", out[i]);
  std::printf("\n");
  bool ok = true;
  if (o.verify) {
    std::printf("Running CPU reference for %d head(s)...\n", o.verify_heads);
    ok = compare_slices(job.cpu_select(o.verify_heads), out, o.verify_heads, TwoLevel::kTopC, TwoLevel::kPerCluster,
                        TwoLevel::kOutPerHead);
  }
  std::printf("Done: computed %d x %d indices on device.\n", kHeads, TwoLevel::kOutPerHead);
  return ok ? 0 : 1;
}

// ---- center_only: centroid selection with expansion ------------------------------------------------------------

int run_center_only(const Options& o) {
  const int C = o.centroids, L = o.cluster_len, T = o.topc, per_head = T * L;
  std::printf("Centre-only selection: heads=%d dim=%d tokens=%lld centroids=%d cluster_len=%d top_centroids=%d\n", kHeads, kDim,
              (long long)C * L, C, L, T);
  Problem p = make_problem(C, L, false);
  uint16_t* d_q = to_device(p.q);
  uint16_t* d_centers = to_device(p.centers);
  int32_t* d_out = device_buffer<int32_t>((size_t)kHeads * per_head);
  tka_center_topk_args a{};
  a.q = d_q;
  a.centers = d_centers;
  a.dtype = TKA_F16;
  a.num_heads = kHeads;
  a.num_centers = C;
  a.top_c = T;
  a.cluster_len = L;
  a.head_dim = kDim;
  a.scale = 1.0f;
  a.out_idx = d_out;
  a.workspace_bytes = tka_center_topk_expand_workspace_bytes(&a);
  a.workspace = device_buffer<unsigned char>(a.workspace_bytes);
  std::printf("Workspace: %zu bytes\n", a.workspace_bytes);
  const double us = time_launches(o, [&] { TKA_CALL(tka_center_topk_expand(&a)); });
  std::printf("Fused kernel latency: %.3f us\n", us);
  std::vector<int32_t> out((size_t)kHeads * per_head);
  HIP_OK(hipMemcpy(out.data(), d_out, out.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
  std::printf("head0 kv_indices[0..31]: ");
  for (int i = 0; i < 32 && i < per_head; ++i) std::printf("%d ", out[i]);
  std::printf("\n");
  bool ok = true;
  if (o.verify) {
    std::printf("Running CPU reference for %d head(s)...\n", o.verify_heads);
    std::vector<int> cpu((size_t)o.verify_heads * per_head);
    std::vector<float> cs(C);
    for (int h = 0; h < o.verify_heads; ++h) {
      for (int c = 0; c < C; ++c) cs[c] = score_in_order(&p.q[(size_t)h * kDim], &p.centers[((size_t)h * C + c) * kDim], 1.0f);
      const std::vector<int> top = stable_topk(cs, T);
      for (int j = 0; j < T; ++j)
        for (int i = 0; i < L; ++i) cpu[(size_t)h * per_head + (size_t)j * L + i] = top[j] * L + i;
    }
    ok = compare_slices(cpu, out, o.verify_heads, T, L, per_head);
  }
  std::printf("Done: computed %d x %d indices on device.\n", kHeads, per_head);
  release(a.workspace); release(d_out); release(d_centers); release(d_q);
  return ok ? 0 : 1;
}

// ---- flash-decoding over an index list -------------------------------------------------------------------------

struct Decode {
  tka_flash_decode_args args{};
  uint16_t* d_out = nullptr;
  void* d_ws = nullptr;
  // q [heads][128]; K, V [tokens][heads][128] on the device; idx [heads][idx_len] or null for dense
  Decode(const uint16_t* d_q, const uint16_t* d_k, const uint16_t* d_v, int64_t tokens, const int32_t* d_idx, int idx_len) {
    d_out = device_buffer<uint16_t>((size_t)kHeads * kDim);
    args.q = d_q;
    args.keys = d_k;
    args.values = d_v;
    args.out = d_out;
    args.dtype = args.out_dtype = TKA_F16;
    args.batch = 1;
    args.num_kv_heads = kHeads;
    args.group = 1;
    args.head_dim = kDim;
    args.softmax_mode = TKA_SOFTMAX_SCALED;
    args.seq_len = tokens;
    args.q_stride_b = args.out_stride_b = (int64_t)kHeads * kDim;
    args.kv_stride_n = (int64_t)kHeads * kDim;
    args.kv_stride_h = kDim;
    args.scale = 1.0f / std::sqrt((float)kDim);
    args.kv_idx = d_idx;
    args.idx_len = d_idx ? idx_len : 0;
    args.workspace_bytes = tka_flash_decode_workspace_bytes(&args);
    d_ws = device_buffer<unsigned char>(args.workspace_bytes);
    args.workspace = d_ws;
  }
  void launch() { TKA_CALL(tka_flash_decode(&args)); }
  ~Decode() { release(d_ws); release(d_out); }
};

// softmax(q.K/sqrt(d)).V in double over the listed tokens (all tokens when idx is null); returns the largest
// absolute difference to the device output over the first `heads` heads
double attention_error(const Problem& p, const std::vector<uint16_t>& values, const int32_t* idx, int idx_len,
                       const std::vector<uint16_t>& gpu_out, int heads) {
  const int64_t n = idx ? idx_len : p.tokens();
  double worst = 0.0;
  std::vector<double> w((size_t)n);
  for (int h = 0; h < heads; ++h) {
    double m = -1e300;
    for (int64_t i = 0; i < n; ++i) {
      const int64_t t = idx ? idx[(size_t)h * idx_len + i] : i;
      double dot = 0.0;
      for (int d = 0; d < kDim; ++d)
        dot += (double)half_value(p.q[(size_t)h * kDim + d]) * (double)half_value(p.kv[((size_t)t * kHeads + h) * kDim + d]);
      w[(size_t)i] = dot / std::sqrt((double)kDim);
      m = std::max(m, w[(size_t)i]);
    }
    double l = 0.0;
    for (int64_t i = 0; i < n; ++i) l += (w[(size_t)i] = std::exp(w[(size_t)i] - m));
    for (int d = 0; d < kDim; ++d) {
      double acc = 0.0;
      for (int64_t i = 0; i < n; ++i) {
        const int64_t t = idx ? idx[(size_t)h * idx_len + i] : i;
        acc += w[(size_t)i] * (double)half_value(values[((size_t)t * kHeads + h) * kDim + d]);
      }
      worst = std::max(worst, std::fabs(acc / l - (double)half_value(gpu_out[(size_t)h * kDim + d])));
    }
  }
  return worst;
}

bool report_attention(const Problem& p, const int32_t* idx, int idx_len, const Decode& dec, int heads) {
  std::vector<uint16_t> out((size_t)kHeads * kDim);
  HIP_OK(hipMemcpy(out.data(), dec.d_out, out.size() * 2, hipMemcpyDeviceToHost));
  const double err = attention_error(p, p.kv, idx, idx_len, out, heads);   // V = K, as in baseline_1.cu:639-640
  const bool ok = err < 2e-3;
  std::printf("%s attention output vs CPU (double) over %d head(s): max abs diff %.3e (bound 2e-3)\n", ok ? "✓" : "✗", heads, err);
  return ok;
}

int run_baseline_1(const Options& o) {
  std::printf("Selection then flash-decoding (two stages): heads=%d dim=%d clusters=%d cluster_len=%d ids_per_head=%d tokens=%d\n",
              kHeads, kDim, TwoLevel::kClusters, TwoLevel::kClusterLen, TwoLevel::kOutPerHead,
              TwoLevel::kClusters * TwoLevel::kClusterLen);
  TwoLevel sel;
  Decode dec(sel.d_q, sel.d_kv, sel.d_kv, sel.p.tokens(), sel.d_out, TwoLevel::kOutPerHead);
  std::printf("---- Stage 1: gemv_topk to build kv_indices ----\n");
  std::printf("gemv_topk (indices build) latency: %.3f us\n", time_launches(o, [&] { sel.launch(); }));
  const std::vector<int32_t> idx = sel.result();
  std::printf("head0 kv_indices[0..15]: ");
  for (int i = 0; i < 16; ++i) std::printf("%d ", idx[i]);
  std::printf("\n---- Stage 2: flash decoding ----\n");
  std::printf("flash decode latency: %.3f us\n", time_launches(o, [&] { dec.launch(); }));
  std::printf("---- Combined latency: run gemv_topk -> flash decode sequentially ----\n");
  std::printf("gemv_topk + flash decode latency: %.3f us\n", time_launches(o, [&] { sel.launch(); dec.launch(); }));
  bool ok = true;
  if (o.verify) {
    ok = compare_slices(sel.cpu_select(o.verify_heads), idx, o.verify_heads, TwoLevel::kTopC, TwoLevel::kPerCluster,
                        TwoLevel::kOutPerHead);
    ok = report_attention(sel.p, idx.data(), TwoLevel::kOutPerHead, dec, o.verify_heads) && ok;
  }
  std::printf("Done.\n");
  return ok ? 0 : 1;
}

int run_flash_decoding(const Options& o) {
  constexpr int kIds = 2560;
  Problem p = make_problem(TwoLevel::kClusters, TwoLevel::kClusterLen, true);
  std::printf("Flash-decoding: heads=%d dim=%d ids_per_head=%d tokens=%lld%s\n", kHeads, kDim, kIds, (long long)p.tokens(),
              o.dense ? " (dense: all tokens)" : "");
  std::vector<int32_t> idx((size_t)kHeads * kIds);
  std::mt19937 rng(2560);
  std::uniform_int_distribution<int> pick(0, (int)p.tokens() - 1);
  for (auto& t : idx) t = pick(rng);
  uint16_t* d_q = to_device(p.q);
  uint16_t* d_kv = to_device(p.kv);
  int32_t* d_idx = to_device(idx);
  {
    Decode dec(d_q, d_kv, d_kv, p.tokens(), o.dense ? nullptr : d_idx, kIds);
    std::printf("kv_indices[0..7]: ");
    for (int i = 0; i < 8; ++i) std::printf("%d ", idx[i]);
    std::printf("\nWorkspace: %zu bytes\n", dec.args.workspace_bytes);
    std::printf("flash decode latency: %.3f us\n", time_launches(o, [&] { dec.launch(); }));
    bool ok = true;
    if (o.verify) ok = report_attention(p, o.dense ? nullptr : idx.data(), kIds, dec, o.verify_heads);
    std::printf("Done.\n");
    if (!ok) return 1;
  }
  release(d_idx); release(d_kv); release(d_q);
  return 0;
}

// ---- retrieval_attention: the operator ------------------------------------------------------------------------

typedef void (*RaLauncher)(const void*, const void*, const void*, void*, int);

// softmax(exp of the 4K surviving scores) . V for one (batch entry, head), in double; survivors = per chunk of 2048
// keys the K largest scores (library order, no scale, ties to the lower index)
void operator_on_cpu(const uint16_t* q, const std::vector<uint16_t>& keys, const std::vector<uint16_t>& values, int h, int topk,
                     double* out) {
  constexpr int kSeq = 8192, kChunks = 4, kChunk = kSeq / kChunks;
  std::vector<float> sc(kChunk);
  std::vector<double> w;
  std::vector<int> ids;
  for (int c = 0; c < kChunks; ++c) {
    for (int t = 0; t < kChunk; ++t) sc[t] = score_in_order(q, &keys[((size_t)(c * kChunk + t) * kHeads + h) * kDim], 1.0f);
    for (int i : stable_topk(sc, topk)) {
      ids.push_back(c * kChunk + i);
      w.push_back(std::exp((double)sc[i]));
    }
  }
  double l = 0.0;
  for (double x : w) l += x;
  for (int d = 0; d < kDim; ++d) {
    double acc = 0.0;
    for (size_t i = 0; i < ids.size(); ++i) acc += w[i] * (double)half_value(values[((size_t)ids[i] * kHeads + h) * kDim + d]);
    out[d] = acc / l;
  }
}

int run_retrieval_attention(const Options& o) {
  constexpr int kSeq = 8192;
  const int B = o.batch;
  std::printf("Retrieval attention: batch=%d heads=%d dim=%d keys=%d (shared by the batch), 4 chunks of 2048\n", B, kHeads, kDim, kSeq);
  std::mt19937 rng(2025);
  std::uniform_real_distribution<float> small(0.0f, 0.1f);   // the value range of retrieval_attention.cu:2286-2296
  std::vector<uint16_t> q((size_t)B * kHeads * kDim), k((size_t)kSeq * kHeads * kDim), v(k.size());
  for (auto& x : q) x = half_bits(small(rng));
  for (size_t i = 0; i < k.size(); ++i) {
    k[i] = half_bits(small(rng));
    v[i] = half_bits(small(rng));
  }
  uint16_t* d_q = to_device(q);
  uint16_t* d_k = to_device(k);
  uint16_t* d_v = to_device(v);
  uint16_t* d_out = device_buffer<uint16_t>(q.size());
  Options t = o;
  t.iters = o.iters == 50 ? 100 : o.iters;   // this program times 100 launches (retrieval_attention.cu:2303)
  bool ok = true;

  std::printf("\n=== Running Baseline Attention ===\n");
  {
    tka_flash_decode_args a{};
    a.q = d_q; a.keys = d_k; a.values = d_v; a.out = d_out;
    a.dtype = a.out_dtype = TKA_F16;
    a.batch = B; a.num_kv_heads = kHeads; a.group = 1; a.head_dim = kDim;
    a.softmax_mode = TKA_SOFTMAX_SCALED;
    a.seq_len = kSeq;
    a.q_stride_b = a.out_stride_b = (int64_t)kHeads * kDim;
    a.kv_stride_b = 0;
    a.kv_stride_n = (int64_t)kHeads * kDim;
    a.kv_stride_h = kDim;
    a.scale = 1.0f;   // the reference's dense kernel applies no 1/sqrt(d)
    a.workspace_bytes = tka_flash_decode_workspace_bytes(&a);
    a.workspace = device_buffer<unsigned char>(a.workspace_bytes);
    const double us = time_launches(t, [&] { TKA_CALL(tka_flash_decode(&a)); });
    std::printf("Baseline Attention - Avg time: %.3f ms, Throughput: %.2f iter/s\n", us / 1000.0, 1e6 / us);
    release(a.workspace);
  }

  static const struct { int topk; RaLauncher plain, global; } kOps[] = {
      {32, launch_retrieval_attention_32, launch_retrieval_attention_global_32},
      {128, launch_retrieval_attention_128, launch_retrieval_attention_global_128},
      {256, launch_retrieval_attention_256, launch_retrieval_attention_global_256},
      {512, launch_retrieval_attention_512, launch_retrieval_attention_global_512},
      {1024, launch_retrieval_attention_1024, launch_retrieval_attention_global_1024}};
  std::vector<uint16_t> out(q.size());
  std::vector<double> want(kDim);
  for (const auto& op : kOps) {
    for (int variant = 0; variant < 2; ++variant) {
      std::printf("\n=== Running Retrieval Attention (%sTOPK=%d per block) ===\n", variant ? "Global Memory, " : "", op.topk);
      const RaLauncher launch = variant ? op.global : op.plain;
      const double us = time_launches(t, [&] { launch(d_q, d_k, d_v, d_out, B); });
      std::printf("Retrieval Attention - Avg time: %.3f ms, Throughput: %.2f iter/s\n", us / 1000.0, 1e6 / us);
      if (o.verify) {
        HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost));
        double worst = 0.0;
        for (int b = 0; b < B; b += (B > 1 ? B - 1 : 1))          // first and last batch entry
          for (int h = 0; h < o.verify_heads; ++h) {
            operator_on_cpu(&q[((size_t)b * kHeads + h) * kDim], k, v, h, op.topk, want.data());
            for (int d = 0; d < kDim; ++d)
              worst = std::max(worst, std::fabs(want[d] - (double)half_value(out[((size_t)b * kHeads + h) * kDim + d])));
          }
        const bool good = worst < 2e-3;
        std::printf("%s output vs CPU (double) over %d head(s): max abs diff %.3e (bound 2e-3)\n", good ? "✓" : "✗", o.verify_heads, worst);
        ok = ok && good;
      }
    }
  }
  HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost));
  std::printf("\nSample output values (head 0, first 8 dims): ");
  for (int i = 0; i < 8; ++i) std::printf("%.4f ", half_value(out[i]));
  std::printf("\n\nDone!\n");
  release(d_out); release(d_v); release(d_k); release(d_q);
  return ok ? 0 : 1;
}

void usage() {
  std::fprintf(stderr,
               "usage: tka_standalone <gemv_topk|center_only|baseline_1|flash_decoding|retrieval_attention> [--verify [heads]] [--iters N] [--warmup N]\n"
               "       center_only: [--centroids N] [--cluster-len N] [--topc N]    flash_decoding: [--dense]    retrieval_attention: [--batch N]\n");
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 2) {
    usage();
    return 64;
  }
  const std::string cmd = argv[1];
  Options o;
  auto int_after = [&](int& i, int lo, int hi, int* dst) {
    if (i + 1 >= argc) return false;
    const int v = std::atoi(argv[i + 1]);
    if (v < lo || v > hi) return false;
    *dst = v;
    ++i;
    return true;
  };
  for (int i = 2; i < argc; ++i) {
    const std::string a = argv[i];
    bool ok = true;
    if (a == "--verify") {
      o.verify = true;
      int_after(i, 1, kHeads, &o.verify_heads);   // the head count is optional
    } else if (a == "--dense") {
      o.dense = true;
    } else if (a == "--iters") {
      ok = int_after(i, 1, 100000, &o.iters);
    } else if (a == "--warmup") {
      ok = int_after(i, 0, 100000, &o.warmup);
    } else if (a == "--batch") {
      ok = int_after(i, 1, 4096, &o.batch);
    } else if (a == "--centroids") {
      ok = int_after(i, 1, 1 << 20, &o.centroids);
    } else if (a == "--cluster-len") {
      ok = int_after(i, 1, 1 << 20, &o.cluster_len);
    } else if (a == "--topc") {
      ok = int_after(i, 1, 8192, &o.topc);
    } else {
      ok = false;
    }
    if (!ok) {
      std::fprintf(stderr, "bad argument: %s\n", a.c_str());
      usage();
      return 64;
    }
  }
  if (cmd == "gemv_topk") return run_gemv_topk(o);
  if (cmd == "center_only") return run_center_only(o);
  if (cmd == "baseline_1") return run_baseline_1(o);
  if (cmd == "flash_decoding") return run_flash_decoding(o);
  if (cmd == "retrieval_attention") return run_retrieval_attention(o);
  usage();
  return 64;
}
