"""Python surface of the reference's extension module `retrieval_attention_cpp` (bind.cpp:726-757):
thirty ops ``retrieval_attention[_variant]_<K>(query, key_cache, value_cache, output) -> None`` that write
``output`` in place, plus one generic ``retrieval_attention``.  batch = query.size(0) as in bind.cpp:252.

The ops run on the current PyTorch stream.  Like ``data_ptr<at::Half>()`` in the reference wrappers they
insist on float16 tensors; unlike them they also check device, shape and contiguity.
"""
import torch

from . import _lib as L
from . import ops

NUM_HEADS, HEAD_DIM, SEQ_LEN, NUM_CHUNKS = 32, 128, 8192, 4  # retrieval_attention.cu:30-34


def _env_score_mode():
    """TKA_RA_SCORE_MODE=1: the fixed-shape ops score on the matrix cores (see tka_score_mode in include/topk_attn.h)."""
    import os
    return L.TKA_SCORE_MATRIX if os.environ.get("TKA_RA_SCORE_MODE") == "1" else L.TKA_SCORE_CANONICAL


def retrieval_attention(query, key_cache, value_cache, output, topk, num_chunks=NUM_CHUNKS, scale=1.0,
                        bench_print=False, score_mode=L.TKA_SCORE_CANONICAL):
    return ops.retrieval_attention(query, key_cache, value_cache, output, topk, num_chunks, scale,
                                   L.TKA_SOFTMAX_RAW_EXP, bench_print, score_mode)


def _make(variant, topk):
    def op(query, key_cache, value_cache, output):
        for t in (query, key_cache, value_cache, output):
            if t.dtype != torch.float16:
                raise TypeError("expected scalar type Half but found %s" % t.dtype)
        if tuple(query.shape[1:]) != (NUM_HEADS, HEAD_DIM) or tuple(key_cache.shape) != (SEQ_LEN, NUM_HEADS, HEAD_DIM) \
                or key_cache.shape != value_cache.shape or output.shape != query.shape:
            raise ValueError("expected query/output [B,32,128] and key/value cache [8192,32,128]")
        import os
        ops.retrieval_attention(query, key_cache, value_cache, output, topk, NUM_CHUNKS, 1.0, L.TKA_SOFTMAX_RAW_EXP,
                                os.environ.get("TKA_BENCH_PRINT") == "1", _env_score_mode())

    op.__name__ = "retrieval_attention%s_%d" % (variant, topk)
    op.__doc__ = "Retrieval Attention%s (TopK=%d)" % (variant.replace("_", " ").title(), topk)
    return op


for _v in L.RA_VARIANTS:
    for _k in L.RA_TOPKS:
        globals()["retrieval_attention%s_%d" % (_v, _k)] = _make(_v, _k)
del _v, _k
