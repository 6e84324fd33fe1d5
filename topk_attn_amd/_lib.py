"""ctypes binding of libtka.so: the structs and prototypes of include/topk_attn.h, field for field."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtka.so")

TKA_OK, TKA_EINVAL, TKA_EUNSUPPORTED, TKA_EHIP, TKA_EWORKSPACE, TKA_ESCRATCH = 0, 1, 2, 3, 4, 5
TKA_NOALLOC_SCRATCH_BYTES = 128 << 20
TKA_F16, TKA_BF16 = 0, 1
TKA_SOFTMAX_SCALED, TKA_SOFTMAX_RAW_EXP = 0, 1
TKA_SCORE_CANONICAL, TKA_SCORE_MATRIX = 0, 1
TKA_MAX_TOPK = 8192
TKA_MAX_SPLITS = 1024

_p, _i32, _i64, _f, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t


class GemvTopkArgs(C.Structure):
    _fields_ = [("q", _p), ("keys", _p), ("dtype", _i32), ("batch", _i32), ("num_kv_heads", _i32), ("group", _i32),
                ("head_dim", _i32), ("k", _i32), ("num_chunks", _i32), ("score_mode", _i32), ("seq_len", _i64),
                ("q_stride_b", _i64), ("key_stride_b", _i64), ("key_stride_n", _i64), ("key_stride_h", _i64),
                ("scale", _f), ("reserved1", _i32), ("out_idx", _p), ("out_val", _p), ("out_scores", _p),
                ("workspace", _p), ("workspace_bytes", _sz), ("stream", _p)]


class TopkArgs(C.Structure):
    _fields_ = [("scores", _p), ("num_segments", _i32), ("k", _i32), ("seg_len", _i64), ("seg_stride", _i64),
                ("out_idx", _p), ("out_val", _p), ("workspace", _p), ("workspace_bytes", _sz), ("stream", _p)]


class CenterTopkArgs(C.Structure):
    _fields_ = [("q", _p), ("centers", _p), ("dtype", _i32), ("num_heads", _i32), ("num_centers", _i32),
                ("top_c", _i32), ("cluster_len", _i32), ("head_dim", _i32), ("scale", _f), ("reserved0", _i32),
                ("out_idx", _p), ("out_centers", _p), ("out_center_val", _p), ("workspace", _p),
                ("workspace_bytes", _sz), ("stream", _p)]


class ClusterTopkArgs(C.Structure):
    _fields_ = [("q", _p), ("centers", _p), ("keys", _p), ("dtype", _i32), ("num_heads", _i32),
                ("num_centers", _i32), ("top_c", _i32), ("cluster_len", _i32), ("k", _i32), ("head_dim", _i32),
                ("scale", _f), ("key_stride_n", _i64), ("key_stride_h", _i64), ("out_idx", _p), ("workspace", _p),
                ("workspace_bytes", _sz), ("stream", _p)]


class IndexUnionArgs(C.Structure):
    _fields_ = [("idx", _p), ("num_segments", _i32), ("k", _i32), ("sink", _i32), ("local", _i32),
                ("seq_len", _i64), ("out_idx", _p), ("out_count", _p), ("stream", _p)]


class FlashDecodeArgs(C.Structure):
    _fields_ = [("q", _p), ("keys", _p), ("values", _p), ("out", _p), ("dtype", _i32), ("out_dtype", _i32),
                ("batch", _i32), ("num_kv_heads", _i32), ("group", _i32), ("head_dim", _i32), ("num_splits", _i32),
                ("softmax_mode", _i32), ("seq_len", _i64), ("q_stride_b", _i64), ("out_stride_b", _i64),
                ("kv_stride_b", _i64), ("kv_stride_n", _i64), ("kv_stride_h", _i64), ("scale", _f),
                ("idx_len", _i32), ("kv_idx", _p), ("kv_count", _p), ("kv_logit", _p), ("out_lse", _p),
                ("workspace", _p), ("workspace_bytes", _sz), ("stream", _p)]


class LseCombineArgs(C.Structure):
    _fields_ = [("part_m", _p), ("part_l", _p), ("part_acc", _p), ("rows", _i32), ("num_splits", _i32),
                ("out_dtype", _i32), ("reserved0", _i32), ("out", _p), ("out_lse", _p), ("stream", _p)]


class RaArgs(C.Structure):
    _fields_ = [("q", _p), ("keys", _p), ("values", _p), ("out", _p), ("dtype", _i32), ("batch", _i32),
                ("num_heads", _i32), ("head_dim", _i32), ("topk_per_chunk", _i32), ("num_chunks", _i32),
                ("softmax_mode", _i32), ("bench_print", _i32), ("seq_len", _i64), ("scale", _f),
                ("score_mode", _i32), ("workspace", _p), ("workspace_bytes", _sz), ("stream", _p)]


class SparseDecodeArgs(C.Structure):
    _fields_ = [("q", _p), ("keys", _p), ("values", _p), ("out", _p), ("dtype", _i32), ("out_dtype", _i32),
                ("batch", _i32), ("num_kv_heads", _i32), ("group", _i32), ("head_dim", _i32), ("k", _i32),
                ("sink", _i32), ("local", _i32), ("num_splits", _i32), ("seq_len", _i64), ("q_stride_b", _i64),
                ("out_stride_b", _i64), ("kv_stride_b", _i64), ("kv_stride_n", _i64), ("kv_stride_h", _i64),
                ("scale", _f), ("reserved0", _i32), ("out_topk_idx", _p), ("out_topk_val", _p),
                ("out_union_idx", _p), ("out_union_count", _p), ("workspace", _p), ("workspace_bytes", _sz),
                ("stream", _p)]


class TestHooks(C.Structure):
    _fields_ = [("force_segment_redo", _i32), ("tau_spin_limit", _i32), ("tau_withhold_mod", _i32),
                ("tau_withhold_rem", _i32), ("tau_withhold_mode", _i32), ("union_handoff_order", _i32), ("fused_tail", _i32)]


RA_VARIANTS = ("", "_global", "_pipelined", "_pipelined_global", "_two_kernels", "_gather_baseline")
RA_TOPKS = (32, 128, 256, 512, 1024)

# name -> (restype, argtypes); every symbol include/*.h declares
class ProbeArgs(C.Structure):
    _fields_ = [("keys", _p), ("values", _p), ("idx", _p), ("sink", _p), ("kind", _i32), ("batch", _i32), ("num_kv_heads", _i32),
                ("idx_len", _i32), ("threads", _i32), ("rounds", _i32), ("nontemporal", _i32), ("tokens_per_wg", _i32),
                ("seq_len", _i64), ("kv_stride_b", _i64), ("kv_stride_n", _i64), ("kv_stride_h", _i64), ("stream", _p)]


TKA_PROBE_STREAM, TKA_PROBE_GATHER = 0, 1

PROTOTYPES = {
    "tka_status_string": (C.c_char_p, [C.c_int]),
    "tka_version": (C.c_int, []),
    "tka_gemv_topk_workspace_bytes": (_sz, [C.POINTER(GemvTopkArgs)]),
    "tka_gemv_topk": (C.c_int, [C.POINTER(GemvTopkArgs)]),
    "tka_gemv_scores": (C.c_int, [C.POINTER(GemvTopkArgs)]),
    "tka_gemv_topk_redone_segments": (C.c_int, [C.POINTER(GemvTopkArgs), C.POINTER(C.c_int32)]),
    "tka_gemv_topk_gave_up_slices": (C.c_int, [C.POINTER(GemvTopkArgs), C.POINTER(C.c_int32)]),
    "tka_set_test_hooks": (C.c_int, [C.POINTER(TestHooks)]),
    "tka_probe_read": (C.c_int, [C.POINTER(ProbeArgs)]),
    "tka_topk_workspace_bytes": (_sz, [C.POINTER(TopkArgs)]),
    "tka_topk_f32": (C.c_int, [C.POINTER(TopkArgs)]),
    "tka_center_topk_expand_workspace_bytes": (_sz, [C.POINTER(CenterTopkArgs)]),
    "tka_center_topk_expand": (C.c_int, [C.POINTER(CenterTopkArgs)]),
    "tka_cluster_gemv_topk_workspace_bytes": (_sz, [C.POINTER(ClusterTopkArgs)]),
    "tka_cluster_gemv_topk": (C.c_int, [C.POINTER(ClusterTopkArgs)]),
    "tka_index_union": (C.c_int, [C.POINTER(IndexUnionArgs)]),
    "tka_flash_decode_workspace_bytes": (_sz, [C.POINTER(FlashDecodeArgs)]),
    "tka_flash_decode": (C.c_int, [C.POINTER(FlashDecodeArgs)]),
    "tka_lse_combine": (C.c_int, [C.POINTER(LseCombineArgs)]),
    "tka_retrieval_attention_workspace_bytes": (_sz, [C.POINTER(RaArgs)]),
    "tka_retrieval_attention": (C.c_int, [C.POINTER(RaArgs)]),
    "tka_sparse_decode_workspace_bytes": (_sz, [C.POINTER(SparseDecodeArgs)]),
    "tka_sparse_decode_step": (C.c_int, [C.POINTER(SparseDecodeArgs)]),
    "tka_sparse_decode_step_noalloc": (C.c_int, [C.POINTER(SparseDecodeArgs)]),
    "tka_sparse_decode_redone_segments": (C.c_int, [C.POINTER(SparseDecodeArgs), C.POINTER(C.c_int32)]),
    "tka_profile_enable": (C.c_int, [C.c_int]),
    "tka_profile_reset": (C.c_int, []),
    "tka_profile_read": (C.c_int, [C.POINTER(C.c_char_p), C.POINTER(C.c_double), C.POINTER(_i64), C.c_int]),
}
for _v in RA_VARIANTS:
    for _k in RA_TOPKS:
        PROTOTYPES["launch_retrieval_attention%s_%d" % (_v, _k)] = (None, [_p, _p, _p, _p, C.c_int])

_lib = None


class LibraryMissing(RuntimeError):
    pass


def lib():
    """Load libtka.so (built by topk_attn_amd.build).  There is no fallback: without the HIP library
    every op of this package raises."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                                 "or `make -C topk_attn_amd/csrc`" % LIB_PATH)
        try:
            import torch  # noqa: F401  (loads the HIP runtime this process will use before libtka binds to it)
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def status_string(rc):
    return lib().tka_status_string(rc).decode()


class TkaError(RuntimeError):
    def __init__(self, rc, where):
        super().__init__("%s: %s (status %d)" % (where, status_string(rc), rc))
        self.status = rc


def check(rc, where):
    if rc != TKA_OK:
        raise TkaError(rc, where)
