/*
 * tka_oracle.c — CPU restatement of the reference's sparse-decode path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP kernels are compared against.  Nothing in the shipped
 * library links, loads or calls it; only tests, the smoke check and the CPU leg of the benchmark do.
 *
 * Each function cites the reference code it restates (paths relative to the reference tree).
 * The reference's own CPU checkers live inside CUDA translation units that need cuda_fp16.h and
 * cannot be compiled with gcc, so they are restated here rather than built.
 *
 * Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):
 *   orc_half_to_float / orc_bf16_to_float  exhaustive 65536-value comparison against numpy
 *   orc_scores_canonical                   fp64 dot within 1e-5; unit-vector queries reproduce a K column
 *                                          exactly; permuting dims inside a lane block of equal terms
 *   orc_topk_stable                        numpy lexsort / torch stable sort; brute force on tiny inputs;
 *                                          all-equal, +-0, NaN, ramps
 *   orc_attention_f64                      scipy softmax + numpy matmul; uniform logits -> mean of V;
 *                                          one dominant logit -> that row; permutation invariance
 *   orc_lse_combine                        split-vs-unsplit identity; empty split; equal maxima
 *   orc_center_expand, orc_index_union     closed form / numpy union1d
 *   orc_retrieval_attention, orc_sparse_decode_step, orc_cluster_topk
 *                                          compositions of the above, re-derived in numpy in the tests
 * Tie ORDER of the reference itself (CUB BlockRadixSort, version unpinned, outside the reference tree)
 * is not pinned by any reference test: "parity unpinned" there; the rule used is lower index first.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_D 128

/* ---- element conversions ------------------------------------------------------------------- */

float orc_half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

float orc_bf16_to_float(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline float elem_to_float(const uint16_t* p, int dtype) {
  return dtype == 0 ? orc_half_to_float(*p) : orc_bf16_to_float(*p);
}

/* ---- stage 1: scores ------------------------------------------------------------------------ */

/* Group query: qf[d] = ((q0[d] + q1[d]) + ...) in fp32, ascending head.  The reference has one
 * query head per KV head (gemv_topk.cu:21); with a group the selection score is the sum of the
 * group's scores, i.e. the score of the summed query. */
void orc_group_query(const uint16_t* q, int dtype, int group, float* qf) {
  for (int d = 0; d < ORC_D; ++d) {
    float s = elem_to_float(q + d, dtype);
    for (int g = 1; g < group; ++g) s = s + elem_to_float(q + (size_t)g * ORC_D + d, dtype);
    qf[d] = s;
  }
}

/* Canonical fp32 score of one row: the 16-lane order of gemv_topk.cu:320-328 — lane j runs an fma
 * chain over dims 8j..8j+7 from 0.0f, then a butterfly with partner distances 8, 4, 2, 1 — and a
 * single multiply by `scale` (the folded scale of flash_decoding.cu:208). */
static float score_row(const float* qf, const uint16_t* krow, int dtype, float scale) {
  float p[16], s[16];
  for (int j = 0; j < 16; ++j) {
    float acc = 0.0f;
    for (int i = 0; i < 8; ++i) acc = fmaf(qf[8 * j + i], elem_to_float(krow + 8 * j + i, dtype), acc);
    p[j] = acc;
  }
  for (int dist = 8; dist >= 1; dist >>= 1) {
    for (int j = 0; j < 16; ++j) s[j] = p[j] + p[j ^ dist];
    memcpy(p, s, sizeof p);
  }
  return p[0] * scale;
}

void orc_scores_canonical(const uint16_t* keys, int dtype, int64_t n, int64_t stride_n,
                          const float* qf, float scale, float* out) {
  for (int64_t t = 0; t < n; ++t) out[t] = score_row(qf, keys + t * stride_n, dtype, scale);
}

/* fp64 truth for the tolerance check: sum over the group of q_g . k, times scale. */
void orc_scores_f64(const uint16_t* keys, int dtype, int64_t n, int64_t stride_n, const uint16_t* q,
                    int group, double scale, double* out) {
  for (int64_t t = 0; t < n; ++t) {
    double acc = 0.0;
    for (int g = 0; g < group; ++g)
      for (int d = 0; d < ORC_D; ++d)
        acc += (double)elem_to_float(q + (size_t)g * ORC_D + d, dtype) *
               (double)elem_to_float(keys + t * stride_n + d, dtype);
    out[t] = acc * scale;
  }
}

/* ---- stage 1: selection --------------------------------------------------------------------- */

/* Order-preserving map fp32 -> uint32: larger score <=> larger key; -0.0 == +0.0; NaN lowest.
 * (The same "twiddle" CUB applies inside BlockRadixSort, gemv_topk.cu:361, plus the two policies.) */
uint32_t orc_score_key(float x) {
  uint32_t u;
  if (x != x) return 0u;
  x = x + 0.0f; /* -0.0 -> +0.0 */
  memcpy(&u, &x, 4);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

float orc_key_score(uint32_t key) {
  uint32_t u = (key & 0x80000000u) ? (key & 0x7fffffffu) : ~key;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

typedef struct { uint32_t key; int32_t idx; } orc_pair;

static int pair_cmp(const void* a, const void* b) {
  const orc_pair* x = (const orc_pair*)a;
  const orc_pair* y = (const orc_pair*)b;
  if (x->key != y->key) return x->key > y->key ? -1 : 1; /* score descending */
  if (x->idx != y->idx) return x->idx < y->idx ? -1 : 1; /* index ascending  */
  return 0;
}

/* First k of the order (score desc, index asc): what a stable descending sort of the blocked-order
 * items gives (gemv_topk.cu:353-378, retrieval_attention.cu:335-354).  Returns 0, or -1 on bad k. */
int orc_topk_stable(const float* scores, int64_t n, int k, int32_t* out_idx, float* out_val) {
  if (k < 0 || k > n) return -1;
  orc_pair* a = (orc_pair*)malloc((size_t)n * sizeof(orc_pair));
  if (!a) return -1;
  for (int64_t i = 0; i < n; ++i) { a[i].key = orc_score_key(scores[i]); a[i].idx = (int32_t)i; }
  qsort(a, (size_t)n, sizeof(orc_pair), pair_cmp); /* total order on distinct (key, idx): stability moot */
  for (int i = 0; i < k; ++i) {
    out_idx[i] = a[i].idx;
    if (out_val) out_val[i] = orc_key_score(a[i].key);
  }
  free(a);
  return 0;
}

/* Centroid expansion, center_only_topk/gemv_topk.cu:272-279. */
void orc_center_expand(const int32_t* centers, int top_c, int cluster_len, int32_t* out) {
  for (int j = 0; j < top_c; ++j)
    for (int i = 0; i < cluster_len; ++i) out[(size_t)j * cluster_len + i] = centers[j] * cluster_len + i;
}

/* Centre-only selection for one head, center_only_topk/gemv_topk.cu:82-119 (scores in the canonical
 * fp32 order instead of that checker's double accumulate). */
int orc_center_topk_expand(const uint16_t* q, const uint16_t* centers, int dtype, int num_centers,
                           int top_c, int cluster_len, float scale, int32_t* out_idx,
                           int32_t* out_centers, float* out_center_val) {
  float qf[ORC_D];
  orc_group_query(q, dtype, 1, qf);
  float* sc = (float*)malloc((size_t)num_centers * sizeof(float));
  int32_t* top = (int32_t*)malloc((size_t)top_c * sizeof(int32_t));
  float* val = (float*)malloc((size_t)top_c * sizeof(float));
  orc_scores_canonical(centers, dtype, num_centers, ORC_D, qf, scale, sc);
  int rc = orc_topk_stable(sc, num_centers, top_c, top, val);
  if (rc == 0) {
    orc_center_expand(top, top_c, cluster_len, out_idx);
    if (out_centers) memcpy(out_centers, top, (size_t)top_c * sizeof(int32_t));
    if (out_center_val) memcpy(out_center_val, val, (size_t)top_c * sizeof(float));
  }
  free(sc); free(top); free(val);
  return rc;
}

/* Two-level selection for one head, gemv_topk.cu:75-135: top_c centroids, then top k tokens inside
 * each chosen cluster of cluster_len consecutive tokens; out[r*k+i] = c_r*cluster_len + local_i. */
int orc_cluster_topk(const uint16_t* q, const uint16_t* centers, const uint16_t* keys, int dtype,
                     int num_centers, int top_c, int cluster_len, int k, int64_t key_stride_n,
                     float scale, int32_t* out_idx) {
  float qf[ORC_D];
  orc_group_query(q, dtype, 1, qf);
  float* cs = (float*)malloc((size_t)num_centers * sizeof(float));
  int32_t* top = (int32_t*)malloc((size_t)top_c * sizeof(int32_t));
  float* ts = (float*)malloc((size_t)cluster_len * sizeof(float));
  int32_t* loc = (int32_t*)malloc((size_t)k * sizeof(int32_t));
  orc_scores_canonical(centers, dtype, num_centers, ORC_D, qf, scale, cs);
  int rc = orc_topk_stable(cs, num_centers, top_c, top, NULL);
  for (int r = 0; rc == 0 && r < top_c; ++r) {
    int64_t base = (int64_t)top[r] * cluster_len;
    orc_scores_canonical(keys + base * key_stride_n, dtype, cluster_len, key_stride_n, qf, scale, ts);
    rc = orc_topk_stable(ts, cluster_len, k, loc, NULL);
    for (int i = 0; rc == 0 && i < k; ++i) out_idx[(size_t)r * k + i] = (int32_t)(base + loc[i]);
  }
  free(cs); free(top); free(ts); free(loc);
  return rc;
}

/* Ascending duplicate-free union of ids with [0,sink) and [n-local,n).  Returns the count. */
static int int_cmp(const void* a, const void* b) {
  int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
  return x < y ? -1 : (x > y ? 1 : 0);
}
int orc_index_union(const int32_t* ids, int k, int sink, int local, int64_t n, int32_t* out) {
  int64_t lo = sink < n ? sink : n;
  int64_t hi = n - local > lo ? n - local : lo;
  int cnt = 0;
  for (int64_t t = 0; t < lo; ++t) out[cnt++] = (int32_t)t;
  int mid0 = cnt;
  for (int i = 0; i < k; ++i)
    if (ids[i] >= lo && ids[i] < hi) out[cnt++] = ids[i];
  qsort(out + mid0, (size_t)(cnt - mid0), sizeof(int32_t), int_cmp);
  int w = mid0;
  for (int i = mid0; i < cnt; ++i)
    if (i == mid0 || out[i] != out[i - 1]) out[w++] = out[i];
  cnt = w;
  for (int64_t t = hi; t < n; ++t) out[cnt++] = (int32_t)t;
  return cnt;
}

/* ---- stages 2 and 3: attention -------------------------------------------------------------- */

/* One query head over a token list (idx == NULL: dense 0..count-1), fp64 throughout:
 *   logits x_i = scale * q.k_i  (or logit[i] when supplied), out = softmax(x) . V
 * baseline_1.py:97-110 (scaled softmax) and test_ra.py:134-160 (raw exp; identical to the
 * max-subtracted form evaluated here).  Also returns the natural-log LSE. */
void orc_attention_f64(const uint16_t* q, const uint16_t* keys, const uint16_t* values, int dtype,
                       int64_t stride_n, const int32_t* idx, int64_t count, const float* logit,
                       double scale, double* out, double* out_lse) {
  double* x = (double*)malloc((size_t)(count > 0 ? count : 1) * sizeof(double));
  double mx = -INFINITY;
  for (int64_t i = 0; i < count; ++i) {
    int64_t t = idx ? idx[i] : i;
    double acc;
    if (logit) {
      acc = (double)logit[i];
    } else {
      acc = 0.0;
      for (int d = 0; d < ORC_D; ++d)
        acc += (double)elem_to_float(q + d, dtype) * (double)elem_to_float(keys + t * stride_n + d, dtype);
      acc *= scale;
    }
    x[i] = acc;
    if (acc > mx) mx = acc;
  }
  double sum = 0.0;
  for (int d = 0; d < ORC_D; ++d) out[d] = 0.0;
  for (int64_t i = 0; i < count; ++i) {
    int64_t t = idx ? idx[i] : i;
    double p = exp(x[i] - mx);
    sum += p;
    for (int d = 0; d < ORC_D; ++d) out[d] += p * (double)elem_to_float(values + t * stride_n + d, dtype);
  }
  for (int d = 0; d < ORC_D; ++d) out[d] = count > 0 ? out[d] / sum : 0.0;
  if (out_lse) *out_lse = count > 0 ? mx + log(sum) : -INFINITY;
  free(x);
}

/* Split combine, the algebra of baseline_1.cu:549-609 in the base-2 domain:
 *   M = max m_s; L = sum l_s 2^(m_s-M); out = sum acc_s 2^(m_s-M) / L.  Splits with l == 0 are empty. */
void orc_lse_combine(const float* m, const float* l, const float* acc, int num_splits, double* out,
                     double* out_lse) {
  double M = -INFINITY;
  for (int s = 0; s < num_splits; ++s)
    if (l[s] > 0.0f && (double)m[s] > M) M = (double)m[s];
  double L = 0.0;
  for (int d = 0; d < ORC_D; ++d) out[d] = 0.0;
  for (int s = 0; s < num_splits; ++s) {
    if (!(l[s] > 0.0f)) continue;
    double w = exp2((double)m[s] - M);
    L += (double)l[s] * w;
    for (int d = 0; d < ORC_D; ++d) out[d] += (double)acc[(size_t)s * ORC_D + d] * w;
  }
  for (int d = 0; d < ORC_D; ++d) out[d] = L > 0.0 ? out[d] / L : 0.0;
  if (out_lse) *out_lse = L > 0.0 ? (M + log2(L)) * 0.69314718055994530942 : -INFINITY;
}

/* The retrieval_attention op for one (batch entry, head): retrieval_attention.cu:1162-1339 /
 * test_ra.py:88-160.  Per chunk: canonical fp32 scores (no scale unless given), stable top-k,
 * hand-off slot [c*k + r]; then softmax over the num_chunks*k fp32 scores and gathered P.V in fp64.
 * (The reference rounds the handed-off scores to fp16 and does the softmax in fp16; that arithmetic
 * is not reproduced — outputs are compared at the stated tolerance.) */
int orc_retrieval_attention(const uint16_t* q, const uint16_t* keys, const uint16_t* values, int dtype,
                            int64_t seq_len, int64_t stride_n, int num_chunks, int k, float scale,
                            double* out, int32_t* out_idx, float* out_val) {
  int64_t chunk = seq_len / num_chunks;
  int total = num_chunks * k;
  float qf[ORC_D];
  orc_group_query(q, dtype, 1, qf);
  float* sc = (float*)malloc((size_t)chunk * sizeof(float));
  int32_t* ids = (int32_t*)malloc((size_t)total * sizeof(int32_t));
  float* val = (float*)malloc((size_t)total * sizeof(float));
  int rc = 0;
  for (int c = 0; rc == 0 && c < num_chunks; ++c) {
    int64_t base = (int64_t)c * chunk;
    orc_scores_canonical(keys + base * stride_n, dtype, chunk, stride_n, qf, scale, sc);
    rc = orc_topk_stable(sc, chunk, k, ids + (size_t)c * k, val + (size_t)c * k);
    for (int r = 0; r < k; ++r) ids[(size_t)c * k + r] += (int32_t)base;
  }
  if (rc == 0) {
    orc_attention_f64(q, keys, values, dtype, stride_n, ids, total, val, 1.0, out, NULL);
    if (out_idx) memcpy(out_idx, ids, (size_t)total * sizeof(int32_t));
    if (out_val) memcpy(out_val, val, (size_t)total * sizeof(float));
  }
  free(sc); free(ids); free(val);
  return rc;
}

/* End-to-end sparse decode for one (batch entry, KV head): group-summed canonical scores, stable
 * top-k, union with sink/local, fp64 attention for each of the group's query heads over the union.
 * Composition of baseline_1.py:71-110 with the GQA and union rules stated in the library header.
 * out is [group][128]; union_idx must hold k+sink+local entries.  Returns the union count or -1. */
int orc_sparse_decode_step(const uint16_t* q, const uint16_t* keys, const uint16_t* values, int dtype,
                           int group, int64_t seq_len, int64_t stride_n, int k, int sink, int local,
                           float scale, double* out, int32_t* topk_idx, float* topk_val,
                           int32_t* union_idx) {
  float qf[ORC_D];
  orc_group_query(q, dtype, group, qf);
  float* sc = (float*)malloc((size_t)seq_len * sizeof(float));
  orc_scores_canonical(keys, dtype, seq_len, stride_n, qf, scale, sc);
  int rc = orc_topk_stable(sc, seq_len, k, topk_idx, topk_val);
  free(sc);
  if (rc != 0) return -1;
  int cnt = orc_index_union(topk_idx, k, sink, local, seq_len, union_idx);
  for (int g = 0; g < group; ++g)
    orc_attention_f64(q + (size_t)g * ORC_D, keys, values, dtype, stride_n, union_idx, cnt, NULL,
                      (double)scale, out + (size_t)g * ORC_D, NULL);
  return cnt;
}
