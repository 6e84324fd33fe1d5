// PyTorch extension module `retrieval_attention_cpp`: the Python surface of the reference's bind.cpp
// (retrieval_attn/bind.cpp:246-757) on top of the C ABI of libtka.so.  Thirty ops
//     retrieval_attention[_global|_pipelined|_pipelined_global|_two_kernels|_gather_baseline]_{32,128,256,512,1024}
//         (Tensor query, Tensor key_cache, Tensor value_cache, Tensor output) -> None
// write `output` in place, batch = query.size(0) (bind.cpp:252), plus one generic op with the top-k as an argument.
// Differences from the reference wrappers: the work goes to PyTorch's current stream (the reference uses the default
// stream and synchronises the device), scratch memory comes from PyTorch's caching allocator (the reference calls
// cudaMalloc / cudaFree in every call, retrieval_attention.cu:1658-1659), shapes, device and contiguity are checked,
// and failures raise instead of ending the process.  All variants share one implementation: they differ in the
// reference only in how the CUDA kernels hand data to each other.
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <cstdlib>
#include <cstring>

#include "topk_attn.h"

namespace {

constexpr int64_t kHeads = 32, kDim = 128, kSeqLen = 8192, kChunks = 4;   // retrieval_attention.cu:30-34

void run(const torch::Tensor& query, const torch::Tensor& key_cache, const torch::Tensor& value_cache, torch::Tensor& output,
         int64_t topk, int64_t num_chunks, double scale, bool fixed_shape, int64_t score_mode) {
  for (const torch::Tensor* t : {&query, &key_cache, &value_cache, (const torch::Tensor*)&output}) {
    TORCH_CHECK(t->is_cuda(), "retrieval_attention: tensors must live on the GPU");
    TORCH_CHECK(t->scalar_type() == at::kHalf || (!fixed_shape && t->scalar_type() == at::kBFloat16),
                "expected scalar type Half but found ", t->scalar_type());
    TORCH_CHECK(t->is_contiguous(), "retrieval_attention: tensors must be contiguous");
    TORCH_CHECK(t->scalar_type() == query.scalar_type() && t->device() == query.device(),
                "retrieval_attention: tensors must share type and device");
  }
  TORCH_CHECK(query.dim() == 3 && key_cache.dim() == 3 && query.size(2) == kDim && key_cache.size(2) == kDim &&
                  key_cache.size(1) == query.size(1),
              "expected query [B,H,128] and key/value cache [N,H,128]");
  TORCH_CHECK(value_cache.sizes() == key_cache.sizes() && output.sizes() == query.sizes(),
              "value cache must match the key cache and output must match the query");
  if (fixed_shape)
    TORCH_CHECK(query.size(1) == kHeads && key_cache.size(0) == kSeqLen, "expected query/output [B,32,128] and key/value cache [8192,32,128]");

  tka_ra_args a;
  std::memset(&a, 0, sizeof a);
  a.q = query.data_ptr();
  a.keys = key_cache.data_ptr();
  a.values = value_cache.data_ptr();
  a.out = output.data_ptr();
  a.dtype = query.scalar_type() == at::kHalf ? TKA_F16 : TKA_BF16;
  a.batch = (int32_t)query.size(0);
  a.num_heads = (int32_t)query.size(1);
  a.head_dim = (int32_t)kDim;
  a.topk_per_chunk = (int32_t)topk;
  a.num_chunks = (int32_t)num_chunks;
  a.softmax_mode = TKA_SOFTMAX_RAW_EXP;
  const char* print = std::getenv("TKA_BENCH_PRINT");
  a.bench_print = print && print[0] == '1' && print[1] == 0;   // the timing line that test_ra.py:63-75 parses
  a.seq_len = key_cache.size(0);
  a.scale = (float)scale;
  a.score_mode = (int32_t)score_mode;
  const size_t need = tka_retrieval_attention_workspace_bytes(&a);
  TORCH_CHECK(need != 0, "retrieval_attention: unsupported arguments (top-k ", topk, ", chunks ", num_chunks, ")");
  torch::Tensor workspace = torch::empty({(int64_t)need}, query.options().dtype(torch::kUInt8));
  a.workspace = workspace.data_ptr();
  a.workspace_bytes = need;
  a.stream = c10::hip::getCurrentHIPStream(query.device().index()).stream();
  const int rc = tka_retrieval_attention(&a);
  TORCH_CHECK(rc == TKA_OK, "tka_retrieval_attention: ", tka_status_string(rc), " (status ", rc, ")");
}

// TKA_RA_SCORE_MODE=1 (read once): the fixed-shape ops score on the matrix cores (tka_score_mode in topk_attn.h)
int64_t env_score_mode() {
  static const int64_t mode = [] {
    const char* e = std::getenv("TKA_RA_SCORE_MODE");
    return (int64_t)(e && e[0] == '1' && e[1] == 0 ? TKA_SCORE_MATRIX : TKA_SCORE_CANONICAL);
  }();
  return mode;
}

}  // namespace

#define RA_OP(variant, K, title)                                                                             \
  m.def("retrieval_attention" variant "_" #K,                                                                \
        [](torch::Tensor query, torch::Tensor key_cache, torch::Tensor value_cache, torch::Tensor output) {  \
          run(query, key_cache, value_cache, output, K, kChunks, 1.0, true, env_score_mode());               \
        },                                                                                                   \
        title " (TopK=" #K ")");
#define RA_OPS(variant, title) \
  RA_OP(variant, 32, title) RA_OP(variant, 128, title) RA_OP(variant, 256, title) RA_OP(variant, 512, title) RA_OP(variant, 1024, title)

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  RA_OPS("", "Retrieval Attention")                                       // bind.cpp:727-731
  RA_OPS("_global", "Retrieval Attention Global")                        // bind.cpp:732-736
  RA_OPS("_pipelined", "Retrieval Attention Pipelined")                  // bind.cpp:737-741
  RA_OPS("_pipelined_global", "Retrieval Attention Pipelined Global")    // bind.cpp:742-746
  RA_OPS("_two_kernels", "Retrieval Attention Two Kernels")              // bind.cpp:747-751
  RA_OPS("_gather_baseline", "Retrieval Attention Gather Baseline")      // bind.cpp:752-756
  m.def("retrieval_attention",
        [](torch::Tensor query, torch::Tensor key_cache, torch::Tensor value_cache, torch::Tensor output, int64_t topk,
           int64_t num_chunks, double scale, int64_t score_mode) {
          run(query, key_cache, value_cache, output, topk, num_chunks, scale, false, score_mode);
        },
        "Retrieval attention with the top-k per chunk, the chunk count and the score scale as arguments (fp16 or bf16); "
        "score_mode 1 computes the scores on the matrix cores",
        py::arg("query"), py::arg("key_cache"), py::arg("value_cache"), py::arg("output"), py::arg("topk"),
        py::arg("num_chunks") = 4, py::arg("scale") = 1.0, py::arg("score_mode") = 0);
}
