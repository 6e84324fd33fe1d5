/*
 * topk_attn_ra_launchers.hpp — the thirty launchers of the reference's retrieval_attention op with C++ linkage
 * and the reference's exact signatures, so that a translation unit that declares them the way
 * retrieval_attn/bind.cpp:5-243 does,
 *
 *     void launch_retrieval_attention_128(const half* query, const half* key_cache, const half* value_cache,
 *                                         half* output, int batch_size);
 *
 * links against libtka.so as it is (the reference defines them in retrieval_attention.cu:1984-2282).  `half` is
 * the type of <hip/hip_fp16.h> (what <cuda_fp16.h> becomes on ROCm); the exported symbols are the Itanium
 * manglings of these declarations, e.g. _Z30launch_retrieval_attention_128PK6__halfS1_S1_PS_i, identical under
 * g++ and hipcc.  Each forwards to the C symbol of the same name (topk_attn_ra_launchers.h), whose behaviour
 * it shares: fixed shapes of the reference op, default stream, no synchronisation, library-owned scratch.
 */
#ifndef TOPK_ATTN_RA_LAUNCHERS_HPP_
#define TOPK_ATTN_RA_LAUNCHERS_HPP_

#ifndef __cplusplus
#error "C++ only: C callers use topk_attn_ra_launchers.h"
#endif

#include <hip/hip_fp16.h>

#define TKA_RA_DECLARE_CXX(variant, topk)                                                        \
  void launch_retrieval_attention##variant##_##topk(const half* query, const half* key_cache,    \
                                                    const half* value_cache, half* output, int batch_size);
#define TKA_RA_DECLARE_CXX_ALL(variant) \
  TKA_RA_DECLARE_CXX(variant, 32)       \
  TKA_RA_DECLARE_CXX(variant, 128)      \
  TKA_RA_DECLARE_CXX(variant, 256)      \
  TKA_RA_DECLARE_CXX(variant, 512)      \
  TKA_RA_DECLARE_CXX(variant, 1024)

TKA_RA_DECLARE_CXX_ALL()                  /* bind.cpp:5-43    */
TKA_RA_DECLARE_CXX_ALL(_global)           /* bind.cpp:45-83   */
TKA_RA_DECLARE_CXX_ALL(_pipelined)        /* bind.cpp:85-123  */
TKA_RA_DECLARE_CXX_ALL(_pipelined_global) /* bind.cpp:125-163 */
TKA_RA_DECLARE_CXX_ALL(_two_kernels)      /* bind.cpp:165-203 */
TKA_RA_DECLARE_CXX_ALL(_gather_baseline)  /* bind.cpp:205-243 */

#undef TKA_RA_DECLARE_CXX_ALL
#undef TKA_RA_DECLARE_CXX

#endif /* TOPK_ATTN_RA_LAUNCHERS_HPP_ */
