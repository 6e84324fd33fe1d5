"""The C-ABI boundary without a GPU: libtka.so loads, exports every symbol include/*.h declares, the ctypes
structs match the C layout, and argument validation answers before any HIP call."""
import ctypes as C
import os
import re
import subprocess
import sys
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")

from topk_attn_amd import _lib as L  # noqa: E402


def _declared_symbols():
    names = set()
    with open(os.path.join(INCLUDE, "topk_attn.h")) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    for m in re.finditer(r"^\s*(?:const\s+char\s*\*|int|size_t)\s+(tka_\w+)\s*\(", text, flags=re.M):
        names.add(m.group(1))
    with open(os.path.join(INCLUDE, "topk_attn_ra_launchers.h")) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    variants = re.findall(r"^TKA_RA_DECLARE_ALL\((\w*)\)", text, flags=re.M)
    topks = re.findall(r"TKA_RA_DECLARE\(variant, (\d+)\)", text)
    assert len(variants) == 6 and len(topks) == 5
    for v in variants:
        for k in topks:
            names.add("launch_retrieval_attention%s_%s" % (v, k))
    return names


def test_library_exports_every_declared_symbol():
    lib = L.lib()
    declared = _declared_symbols()
    assert len(declared) == 28 + 30
    for name in sorted(declared):
        assert hasattr(lib, name), "libtka.so does not export %s" % name
    assert declared == set(L.PROTOTYPES), "ctypes prototypes and headers disagree"


def test_reference_launcher_names_match_bind_cpp():
    """The thirty names are those of the reference's extension (bind.cpp:726-757): 6 variants x 5 K values."""
    want = {"launch_retrieval_attention%s_%d" % (v, k)
            for v in ("", "_global", "_pipelined", "_pipelined_global", "_two_kernels", "_gather_baseline")
            for k in (32, 128, 256, 512, 1024)}
    assert want <= set(L.PROTOTYPES)
    from topk_attn_amd import retrieval_attention_cpp as ra
    for name in want:
        assert callable(getattr(ra, name.replace("launch_", "")))


def test_bind_cpp_style_caller_links_unchanged():
    """The reference's extension declares the thirty launchers with C++ linkage and `half` pointers
    (bind.cpp:5-243).  libtka.so exports exactly those manglings, and a caller written that way (csrc/bind_link_check.cpp,
    compiled by g++ with no header of this library) links against it and resolves all thirty."""
    lib_dir = os.path.join(ROOT, "topk_attn_amd", "lib")
    syms = subprocess.run(["nm", "-D", "--defined-only", os.path.join(lib_dir, "libtka.so")], capture_output=True, text=True, check=True).stdout
    for v in L.RA_VARIANTS:
        for k in L.RA_TOPKS:
            name = "launch_retrieval_attention%s_%d" % (v, k)
            mangled = "_Z%d%sPK6__halfS1_S1_PS_i" % (len(name), name)
            assert re.search(r" T %s$" % re.escape(mangled), syms, flags=re.M), "missing C++ symbol for " + name
            assert re.search(r" T %s$" % re.escape(name), syms, flags=re.M), "missing C symbol " + name
    r = subprocess.run([os.path.join(lib_dir, "tka_bind_link_check")], capture_output=True, text=True)
    assert r.returncode == 0 and "linked 30 launchers declared as in bind.cpp" in r.stdout


STRUCTS = {"tka_gemv_topk_args": L.GemvTopkArgs, "tka_topk_args": L.TopkArgs, "tka_center_topk_args": L.CenterTopkArgs,
           "tka_cluster_topk_args": L.ClusterTopkArgs, "tka_index_union_args": L.IndexUnionArgs,
           "tka_flash_decode_args": L.FlashDecodeArgs, "tka_lse_combine_args": L.LseCombineArgs, "tka_ra_args": L.RaArgs,
           "tka_sparse_decode_args": L.SparseDecodeArgs, "tka_test_hooks": L.TestHooks, "tka_probe_args": L.ProbeArgs}


def test_ctypes_structs_match_the_c_layout():
    """Compile a C program against the header that prints sizeof / offsetof of every field."""
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "topk_attn.h"', '#include "topk_attn_ra_launchers.h"',
             'int main(void) {']
    for cname, cls in STRUCTS.items():
        lines.append('printf("%s %%zu\\n", sizeof(%s));' % (cname, cname))
        for fname, _ in cls._fields_:
            lines.append('printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (cname, fname, cname, fname))
    lines += ['return 0; }']
    with tempfile.TemporaryDirectory() as d:
        src, exe = os.path.join(d, "layout.c"), os.path.join(d, "layout")
        with open(src, "w") as f:
            f.write("\n".join(lines))
        subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-I", INCLUDE, "-o", exe, src])
        out = subprocess.check_output([exe], text=True)
    got = dict(line.split() for line in out.strip().splitlines())
    for cname, cls in STRUCTS.items():
        assert int(got[cname]) == C.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert int(got["%s.%s" % (cname, fname)]) == getattr(cls, fname).offset, "%s.%s" % (cname, fname)


def test_status_strings_and_version():
    lib = L.lib()
    assert lib.tka_version() >= 200            # 2.0.0: score_mode took the place of a reserved field
    assert L.status_string(L.TKA_OK) == "ok"
    assert "workspace" in L.status_string(L.TKA_EWORKSPACE)
    assert L.status_string(99) == "unknown status"


def _valid_gemv():
    a = L.GemvTopkArgs()
    a.q, a.keys, a.out_idx = 0x1000, 0x2000, 0x3000   # never dereferenced: validation precedes every HIP call
    a.dtype, a.batch, a.num_kv_heads, a.group, a.head_dim = L.TKA_F16, 2, 8, 4, 128
    a.k, a.num_chunks, a.seq_len = 64, 1, 4096
    a.q_stride_b, a.key_stride_b, a.key_stride_n, a.key_stride_h = 32 * 128, 4096 * 8 * 128, 8 * 128, 128
    a.scale = 1.0
    return a


def test_redone_segments_validation():
    """The diagnostic validates like the call it reports on, and a call that cannot take the long-segment path
    reports zero without touching the device."""
    lib = L.lib()
    n = C.c_int32(-1)
    a = _valid_gemv()
    assert lib.tka_gemv_topk_redone_segments(C.byref(a), None) == L.TKA_EINVAL
    assert lib.tka_gemv_topk_redone_segments(None, C.byref(n)) == L.TKA_EINVAL
    assert lib.tka_gemv_topk_redone_segments(C.byref(a), C.byref(n)) == L.TKA_EWORKSPACE
    a.workspace, a.workspace_bytes = 0x10000, lib.tka_gemv_topk_workspace_bytes(C.byref(a))
    assert lib.tka_gemv_topk_redone_segments(C.byref(a), C.byref(n)) == L.TKA_OK and n.value == 0   # 4096-token segments
    a.k = 0
    assert lib.tka_gemv_topk_redone_segments(C.byref(a), C.byref(n)) == L.TKA_EINVAL


def test_gemv_topk_validation():
    lib = L.lib()
    a = _valid_gemv()
    need = lib.tka_gemv_topk_workspace_bytes(C.byref(a))
    assert need > 2 * 8 * 4096 * 4                                   # at least the scores
    assert lib.tka_gemv_topk(C.byref(a)) == L.TKA_EWORKSPACE          # valid arguments, no workspace
    a.workspace, a.workspace_bytes = 0x10000, need - 1
    assert lib.tka_gemv_topk(C.byref(a)) == L.TKA_EWORKSPACE
    assert lib.tka_gemv_topk(None) == L.TKA_EINVAL
    for field, value, want in [("head_dim", 64, L.TKA_EUNSUPPORTED), ("dtype", 7, L.TKA_EUNSUPPORTED),
                               ("group", 3, L.TKA_EUNSUPPORTED), ("k", 0, L.TKA_EINVAL), ("k", 5000, L.TKA_EINVAL),
                               ("k", 9000, L.TKA_EINVAL), ("q", None, L.TKA_EINVAL), ("keys", None, L.TKA_EINVAL),
                               ("out_idx", None, L.TKA_EINVAL), ("num_chunks", 3, L.TKA_EINVAL),
                               ("key_stride_n", 100, L.TKA_EINVAL), ("key_stride_n", 1028, L.TKA_EINVAL),
                               ("q", 0x1004, L.TKA_EINVAL), ("seq_len", 0, L.TKA_EINVAL), ("batch", 0, L.TKA_EINVAL)]:
        b = _valid_gemv()
        setattr(b, field, value)
        assert lib.tka_gemv_topk(C.byref(b)) == want, (field, value)
        assert lib.tka_gemv_topk_workspace_bytes(C.byref(b)) == 0
    b = _valid_gemv()
    b.seq_len, b.k = 1 << 20, 8193
    assert lib.tka_gemv_topk(C.byref(b)) == L.TKA_EUNSUPPORTED        # k above TKA_MAX_TOPK
    b = _valid_gemv()
    b.out_scores = None
    assert lib.tka_gemv_scores(C.byref(b)) == L.TKA_EINVAL            # the GEMV phase alone needs out_scores
    b = _valid_gemv()
    b.reserved1 = 1
    assert lib.tka_gemv_topk(C.byref(b)) == L.TKA_EINVAL              # reserved fields must be zero
    # scores on the matrix cores: only where they apply (keys shared by a batch of two or more, one query head per KV
    # head, chunks of up to 16384 keys); anywhere else the call is refused, never silently scored in the other order
    b = _valid_gemv()
    b.score_mode = L.TKA_SCORE_MATRIX
    assert lib.tka_gemv_topk(C.byref(b)) == L.TKA_EUNSUPPORTED        # grouped queries, keys per batch entry
    b.group, b.key_stride_b, b.q_stride_b = 1, 0, 8 * 128
    assert lib.tka_gemv_topk(C.byref(b)) == L.TKA_EWORKSPACE          # applies: valid, no workspace
    b.batch = 1
    assert lib.tka_gemv_topk(C.byref(b)) == L.TKA_EUNSUPPORTED        # a batch of one
    b.batch, b.seq_len = 2, 32768
    assert lib.tka_gemv_topk(C.byref(b)) == L.TKA_EUNSUPPORTED        # chunks of more than 16384 keys


def test_topk_validation():
    lib = L.lib()
    a = L.TopkArgs()
    a.scores, a.out_idx, a.num_segments, a.k, a.seg_len, a.seg_stride = 0x1000, 0x2000, 4, 10, 100, 100
    assert lib.tka_topk_workspace_bytes(C.byref(a)) > 0
    assert lib.tka_topk_f32(C.byref(a)) == L.TKA_EWORKSPACE
    a.k = 101
    assert lib.tka_topk_f32(C.byref(a)) == L.TKA_EINVAL
    a.k, a.seg_stride = 10, 99
    assert lib.tka_topk_f32(C.byref(a)) == L.TKA_EINVAL


def test_flash_decode_validation():
    lib = L.lib()

    def valid():
        a = L.FlashDecodeArgs()
        a.q, a.keys, a.values, a.out = 0x1000, 0x2000, 0x3000, 0x4000
        a.dtype, a.out_dtype, a.batch, a.num_kv_heads, a.group, a.head_dim = L.TKA_F16, L.TKA_BF16, 1, 8, 4, 128
        a.seq_len, a.kv_stride_n, a.kv_stride_h, a.scale = 131072, 1024, 128, 0.088
        return a

    a = valid()
    need = lib.tka_flash_decode_workspace_bytes(C.byref(a))
    assert need > 0 and lib.tka_flash_decode(C.byref(a)) == L.TKA_EWORKSPACE
    for field, value, want in [("group", 5, L.TKA_EUNSUPPORTED), ("num_splits", 5000, L.TKA_EINVAL),
                               ("softmax_mode", 9, L.TKA_EUNSUPPORTED), ("values", None, L.TKA_EINVAL),
                               ("kv_count", 0x5000, L.TKA_EINVAL), ("kv_logit", 0x5000, L.TKA_EINVAL)]:
        b = valid()
        setattr(b, field, value)
        assert lib.tka_flash_decode(C.byref(b)) == want, (field, value)
    b = valid()
    b.kv_idx, b.idx_len, b.kv_logit = 0x6000, 128, 0x7000              # supplied logits need one query head per KV head
    assert lib.tka_flash_decode(C.byref(b)) == L.TKA_EUNSUPPORTED


def test_other_entry_points_reject_nulls():
    lib = L.lib()
    assert lib.tka_center_topk_expand(C.byref(L.CenterTopkArgs())) == L.TKA_EINVAL
    assert lib.tka_cluster_gemv_topk(C.byref(L.ClusterTopkArgs())) == L.TKA_EINVAL
    assert lib.tka_index_union(C.byref(L.IndexUnionArgs())) == L.TKA_EINVAL
    assert lib.tka_lse_combine(C.byref(L.LseCombineArgs())) == L.TKA_EINVAL
    assert lib.tka_retrieval_attention(C.byref(L.RaArgs())) == L.TKA_EINVAL
    assert lib.tka_sparse_decode_step(C.byref(L.SparseDecodeArgs())) == L.TKA_EINVAL
    assert lib.tka_retrieval_attention_workspace_bytes(C.byref(L.RaArgs())) == 0
    a = L.RaArgs()                                                      # the reference op's own shape
    a.q, a.keys, a.values, a.out = 0x1000, 0x2000, 0x3000, 0x4000
    a.dtype, a.batch, a.num_heads, a.head_dim, a.topk_per_chunk, a.num_chunks = L.TKA_F16, 4, 32, 128, 128, 4
    a.softmax_mode, a.seq_len, a.scale = L.TKA_SOFTMAX_RAW_EXP, 8192, 1.0
    assert lib.tka_retrieval_attention_workspace_bytes(C.byref(a)) > 0
    assert lib.tka_retrieval_attention(C.byref(a)) == L.TKA_EWORKSPACE
    a.topk_per_chunk = 4096                                             # more than a chunk holds
    assert lib.tka_retrieval_attention(C.byref(a)) == L.TKA_EINVAL


def test_lse_combine_bounds():
    """The combine kernel keeps one weight per split in LDS: more splits than TKA_MAX_SPLITS are refused before launch."""
    lib = L.lib()
    a = L.LseCombineArgs()
    a.part_m, a.part_l, a.part_acc, a.out = 0x1000, 0x2000, 0x3000, 0x4000
    a.rows, a.num_splits, a.out_dtype = 4, L.TKA_MAX_SPLITS + 1, L.TKA_F16
    assert lib.tka_lse_combine(C.byref(a)) == L.TKA_EUNSUPPORTED
    a.num_splits = 0
    assert lib.tka_lse_combine(C.byref(a)) == L.TKA_EINVAL
    a.rows, a.num_splits = 1 << 30, 4
    assert lib.tka_lse_combine(C.byref(a)) == L.TKA_EUNSUPPORTED


def test_sparse_decode_rejects_values_without_indices():
    lib = L.lib()
    a = L.SparseDecodeArgs()
    a.q, a.keys, a.values, a.out = 0x1000, 0x2000, 0x3000, 0x4000
    a.dtype, a.out_dtype, a.batch, a.num_kv_heads, a.group, a.head_dim = L.TKA_F16, L.TKA_BF16, 1, 8, 4, 128
    a.k, a.sink, a.local, a.seq_len = 64, 4, 16, 4096
    a.q_stride_b = a.out_stride_b = 32 * 128
    a.kv_stride_b, a.kv_stride_n, a.kv_stride_h, a.scale = 4096 * 1024, 1024, 128, 0.088
    assert lib.tka_sparse_decode_workspace_bytes(C.byref(a)) > 0
    assert lib.tka_sparse_decode_step(C.byref(a)) == L.TKA_EWORKSPACE     # valid arguments, no workspace
    a.out_topk_val = 0x5000                                              # values without the rank-ordered ids
    assert lib.tka_sparse_decode_step(C.byref(a)) == L.TKA_EINVAL
    a.out_topk_val = None
    a.out_union_count = 0x6000                                           # the count of a list that is not asked for
    assert lib.tka_sparse_decode_step(C.byref(a)) == L.TKA_EINVAL
    a.out_union_count = None
    n = C.c_int32(-1)
    assert lib.tka_sparse_decode_redone_segments(C.byref(a), C.byref(n)) == L.TKA_EWORKSPACE
    assert lib.tka_sparse_decode_redone_segments(C.byref(a), None) == L.TKA_EINVAL


def test_probe_read_validation():
    lib = L.lib()
    a = L.ProbeArgs()
    assert lib.tka_probe_read(None) == L.TKA_EINVAL
    assert lib.tka_probe_read(C.byref(a)) == L.TKA_EINVAL            # no cache, no sink
    a.keys, a.sink, a.batch, a.num_kv_heads, a.seq_len = 4096, 8192, 1, 1, 1000
    a.kv_stride_n, a.kv_stride_h, a.kind, a.threads, a.rounds = 128, 128, L.TKA_PROBE_STREAM, 300, 2
    assert lib.tka_probe_read(C.byref(a)) == L.TKA_EINVAL            # threads must be 256 or 512
    a.kind = L.TKA_PROBE_GATHER
    assert lib.tka_probe_read(C.byref(a)) == L.TKA_EINVAL            # gather without values and ids
    a.kind = 7
    assert lib.tka_probe_read(C.byref(a)) == L.TKA_EUNSUPPORTED


def test_test_hooks_validation():
    lib = L.lib()
    assert lib.tka_set_test_hooks(None) == L.TKA_OK
    assert lib.tka_set_test_hooks(C.byref(L.TestHooks(1, 64, 2, 1, 1, 0, 1))) == L.TKA_OK
    assert lib.tka_set_test_hooks(C.byref(L.TestHooks(0, -1, 0, 0, 0, 0))) == L.TKA_EINVAL
    assert lib.tka_set_test_hooks(C.byref(L.TestHooks(0, 0, 0, 0, 2, 0, 0))) == L.TKA_EINVAL
    assert lib.tka_set_test_hooks(C.byref(L.TestHooks(0, 0, 0, 0, 0, 0, 3))) == L.TKA_EINVAL
    assert lib.tka_set_test_hooks(None) == L.TKA_OK


def test_profile_interface_without_gpu():
    lib = L.lib()
    assert lib.tka_profile_enable(0) == L.TKA_OK and lib.tka_profile_reset() == L.TKA_OK
    assert lib.tka_profile_read(None, None, None, 0) == 0


def test_ops_refuse_cpu_tensors():
    """No CPU fallback: the Python layer rejects host tensors instead of computing anything itself."""
    import torch
    from topk_attn_amd import ops
    q, K = torch.zeros(1, 8, 128, dtype=torch.float16), torch.zeros(1, 64, 8, 128, dtype=torch.float16)
    with pytest.raises(ValueError):
        ops.gemv_topk(q, K, 4)
    with pytest.raises(ValueError):
        ops.flash_decode(q, K, K, 1.0)


def test_missing_library_is_loud(monkeypatch):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libtka.so")
    with pytest.raises(L.LibraryMissing):
        L.lib()
