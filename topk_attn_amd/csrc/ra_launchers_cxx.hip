// The thirty launchers of the retrieval_attention op once more, with C++ linkage and the reference's own
// parameter types (bind.cpp:5-243 declares them `const half*, const half*, const half*, half*, int` without
// extern "C"), so that bind.cpp-style callers link against the library unchanged.  Each forwards to the C
// symbol of the same name in ra_launchers.hip.
#include "../../include/topk_attn_ra_launchers.hpp"
#include "../../include/topk_attn_ra_launchers.h"

#define TKA_RA_DEFINE_CXX(variant, topk)                                                                    \
  void launch_retrieval_attention##variant##_##topk(const half* query, const half* key_cache,               \
                                                    const half* value_cache, half* output, int batch_size) { \
    ::launch_retrieval_attention##variant##_##topk((const void*)query, (const void*)key_cache,              \
                                                   (const void*)value_cache, (void*)output, batch_size);    \
  }
#define TKA_RA_DEFINE_CXX_ALL(variant) \
  TKA_RA_DEFINE_CXX(variant, 32)       \
  TKA_RA_DEFINE_CXX(variant, 128)      \
  TKA_RA_DEFINE_CXX(variant, 256)      \
  TKA_RA_DEFINE_CXX(variant, 512)      \
  TKA_RA_DEFINE_CXX(variant, 1024)

TKA_RA_DEFINE_CXX_ALL()
TKA_RA_DEFINE_CXX_ALL(_global)
TKA_RA_DEFINE_CXX_ALL(_pipelined)
TKA_RA_DEFINE_CXX_ALL(_pipelined_global)
TKA_RA_DEFINE_CXX_ALL(_two_kernels)
TKA_RA_DEFINE_CXX_ALL(_gather_baseline)
