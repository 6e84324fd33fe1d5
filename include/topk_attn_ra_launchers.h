/*
 * topk_attn_ra_launchers.h — the thirty launchers of the reference's retrieval_attention op, with the
 * reference's names and argument order (declared in retrieval_attn/bind.cpp:5-243, defined in
 * retrieval_attn/retrieval_attention.cu:1984-2282):
 *
 *     void launch_retrieval_attention[_global|_pipelined|_pipelined_global|_two_kernels|_gather_baseline]_
 *          {32,128,256,512,1024}(const half* query, const half* key_cache, const half* value_cache,
 *                                half* output, int batch_size);
 *
 * Fixed shapes of the reference op (retrieval_attention.cu:30-46): query [batch][32][128], key and
 * value cache [8192][32][128] shared by the batch, output [batch][32][128], all fp16 device memory;
 * 4 chunks of 2048 keys, top-K per chunk, raw-exp softmax, no 1/sqrt(d) scale.
 * `half*` is spelled `void*` so the header needs no HIP types, and linkage is C so that a binding in any
 * language can reach the symbols.  Like the reference the calls use the default stream; unlike it they
 * return without synchronising, run one launch (no warm-up loop) and print nothing unless the
 * environment variable TKA_BENCH_PRINT=1 asks for the reference's "Avg time ... Throughput" line.
 * Scratch memory is owned by the library: one buffer per device, allocated on the first call.
 * Errors are reported on stderr (the reference's CUDA_CHECK exits the process instead).
 */
#ifndef TOPK_ATTN_RA_LAUNCHERS_H_
#define TOPK_ATTN_RA_LAUNCHERS_H_

#include "topk_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

#define TKA_RA_DECLARE(variant, topk)                                                          \
  void launch_retrieval_attention##variant##_##topk(const void* query, const void* key_cache, \
                                                    const void* value_cache, void* output, int batch_size);
#define TKA_RA_DECLARE_ALL(variant) \
  TKA_RA_DECLARE(variant, 32)       \
  TKA_RA_DECLARE(variant, 128)      \
  TKA_RA_DECLARE(variant, 256)      \
  TKA_RA_DECLARE(variant, 512)      \
  TKA_RA_DECLARE(variant, 1024)

TKA_RA_DECLARE_ALL()                  /* bind.cpp:5-43    DSM hand-off           */
TKA_RA_DECLARE_ALL(_global)           /* bind.cpp:45-83   global-memory hand-off */
TKA_RA_DECLARE_ALL(_pipelined)        /* bind.cpp:85-123  batch loop in-kernel   */
TKA_RA_DECLARE_ALL(_pipelined_global) /* bind.cpp:125-163                         */
TKA_RA_DECLARE_ALL(_two_kernels)      /* bind.cpp:165-203 topk kernel + reduce   */
TKA_RA_DECLARE_ALL(_gather_baseline)  /* bind.cpp:205-243 gather + dense         */

#undef TKA_RA_DECLARE_ALL
#undef TKA_RA_DECLARE

#ifdef __cplusplus
}
#endif

#endif /* TOPK_ATTN_RA_LAUNCHERS_H_ */
