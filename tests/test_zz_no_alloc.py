"""tka_sparse_decode_step_noalloc, the step for callers that cannot allocate: called through the C ABI, it must
give exactly what tka_sparse_decode_step gives on the same inputs (same kernels, the library's built-in scratch
instead of a caller workspace) - on calls in a row that leave differently laid-out contents in that scratch."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from tests.util import announce, randn_bits, to_dev
from topk_attn_amd import _lib as L

SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


def _args(q, K, V, out, k, sink, local, G, tidx, tval, uidx, ucnt):
    B, N, H = K.shape[:3]
    a = L.SparseDecodeArgs()
    a.q, a.keys, a.values, a.out = q.data_ptr(), K.data_ptr(), V.data_ptr(), out.data_ptr()
    a.dtype = L.TKA_F16 if K.dtype == torch.float16 else L.TKA_BF16
    a.out_dtype = L.TKA_F16 if out.dtype == torch.float16 else L.TKA_BF16
    a.batch, a.num_kv_heads, a.group, a.head_dim = B, H, G, 128
    a.k, a.sink, a.local, a.num_splits, a.seq_len = k, sink, local, 0, N
    a.q_stride_b, a.out_stride_b = q.stride(0), out.stride(0)
    a.kv_stride_b, a.kv_stride_n, a.kv_stride_h = K.stride(0), K.stride(1), K.stride(2)
    a.scale = SCALE
    a.out_topk_idx, a.out_topk_val = tidx.data_ptr(), tval.data_ptr()
    a.out_union_idx, a.out_union_count = uidx.data_ptr(), ucnt.data_ptr()
    a.stream = torch.cuda.current_stream().cuda_stream
    return a


def _one_case(rng, dtype, B, H, G, N, k, sink, local, kind):
    """Both entry points on the same inputs; every output must agree bit for bit.  Returns what the oracle needs."""
    lib = L.lib()
    if kind == "levels":
        Kf = np.linspace(-2, 2, 16)[rng.integers(0, 16, (B, N, H, 128))]
    else:
        Kf = rng.standard_normal((B, N, H, 128))
        Kf[:, rng.permutation(N)[:max(1, N // 100)]] *= 4.0
    qb, Kb, Vb = randn_bits(rng, (B, H * G, 128), dtype), oracle.to_bits(Kf, dtype), randn_bits(rng, (B, N, H, 128), dtype)
    q, K, V = to_dev(qb, dtype), to_dev(Kb, dtype), to_dev(Vb, dtype)
    outs = []
    for noalloc in (False, True):
        out = torch.full((B, H * G, 128), 7.0, dtype=torch.bfloat16, device="cuda")
        tidx = torch.full((B, H, k), -7, dtype=torch.int32, device="cuda")
        tval = torch.full((B, H, k), -7.0, dtype=torch.float32, device="cuda")
        uidx = torch.full((B, H, k + sink + local), -7, dtype=torch.int32, device="cuda")
        ucnt = torch.full((B, H), -7, dtype=torch.int32, device="cuda")
        a = _args(q, K, V, out, k, sink, local, G, tidx, tval, uidx, ucnt)
        if noalloc:
            a.workspace, a.workspace_bytes = None, 0          # ignored by this entry point
            L.check(lib.tka_sparse_decode_step_noalloc(C.byref(a)), "tka_sparse_decode_step_noalloc")
        else:
            need = lib.tka_sparse_decode_workspace_bytes(C.byref(a))
            assert 0 < need <= L.TKA_NOALLOC_SCRATCH_BYTES
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            a.workspace, a.workspace_bytes = ws.data_ptr(), need
            L.check(lib.tka_sparse_decode_step(C.byref(a)), "tka_sparse_decode_step")
        torch.cuda.synchronize()
        outs.append((out, tidx, tval, uidx, ucnt))
    ref, got = outs
    names = ("out", "topk_idx", "topk_val", "union_idx", "union_count")
    for name, r, g in zip(names, ref, got):
        r8, g8 = r.contiguous().view(torch.uint8), g.contiguous().view(torch.uint8)
        assert torch.equal(r8, g8), "%s differs between tka_sparse_decode_step and its no-alloc form" % name
    # and both are right: the selection against the oracle (bit-exact), the output within the tolerance of the step
    tidx, ucnt = got[1].cpu().numpy(), got[4].cpu().numpy()
    outf = got[0].float().cpu().numpy()
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(qb[b, h * G:(h + 1) * G], Kb[b, :, h], Vb[b, :, h], dtype, G, k, sink, local, SCALE)
            assert np.array_equal(tidx[b, h], ri) and ucnt[b, h] == len(ru)
            assert (np.abs(outf[b, h * G:(h + 1) * G] - ro) < 2e-3 + np.abs(ro) * 2.0 ** -8).all()   # bf16 output: its half ulp on top


@pytest.mark.gpu
def test_noalloc_step_matches_the_workspace_form_on_calls_in_a_row():
    """Three calls in a row on the GPU's one built-in buffer: a long-segment shape (sampled thresholds, candidate
    slices), then a smaller input with another layout of the same memory, then the long shape again with new data."""
    rng = np.random.default_rng(2024)
    for dtype, B, H, G, N, k, sink, local, kind in [(oracle.F16, 1, 2, 4, 70000, 1024, 16, 128, "heavy"),
                                                    (oracle.BF16, 2, 2, 2, 5000, 300, 8, 8, "levels"),
                                                    (oracle.F16, 1, 2, 4, 70000, 1024, 16, 128, "levels")]:
        announce("sparse_decode_step_noalloc vs sparse_decode_step: dtype=%d B=%d H=%d G=%d N=%d k=%d %s" % (dtype, B, H, G, N, k, kind))
        _one_case(rng, dtype, B, H, G, N, k, sink, local, kind)


@pytest.mark.gpu
def test_noalloc_step_without_list_outputs():
    """The production form (attention output only, no token list asked for) on the routes it opens: a few segments of
    middling length where the ranking workgroups hand the list to the attention themselves - one segment, then four
    (whose GEMV launch announces the cuts to its own workgroups through words of the scratch buffer), then a smaller
    input.  Output and rank-ordered top-k of the two entry points bit for bit, the top-k as the oracle's."""
    lib = L.lib()
    rng = np.random.default_rng(2025)
    for dtype, B, H, G, N, k, sink, local in [(oracle.F16, 1, 1, 8, 32768, 2048, 64, 512), (oracle.BF16, 1, 4, 4, 32768, 2048, 64, 512),
                                              (oracle.F16, 2, 1, 2, 20000, 1200, 0, 100)]:
        announce("sparse_decode_step_noalloc vs sparse_decode_step, no list outputs: dtype=%d B=%d H=%d G=%d N=%d k=%d" % (dtype, B, H, G, N, k))
        qb, Kb, Vb = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)
        q, K, V = to_dev(qb, dtype), to_dev(Kb, dtype), to_dev(Vb, dtype)
        outs = []
        for noalloc in (False, True):
            out = torch.full((B, H * G, 128), 7.0, dtype=torch.float16, device="cuda")
            tidx = torch.full((B, H, k), -7, dtype=torch.int32, device="cuda")
            tval = torch.full((B, H, k), -7.0, dtype=torch.float32, device="cuda")
            a = _args(q, K, V, out, k, sink, local, G, tidx, tval, tidx, tidx)
            a.out_union_idx, a.out_union_count = None, None
            if noalloc:
                a.workspace, a.workspace_bytes = None, 0
                L.check(lib.tka_sparse_decode_step_noalloc(C.byref(a)), "tka_sparse_decode_step_noalloc")
            else:
                need = lib.tka_sparse_decode_workspace_bytes(C.byref(a))
                assert 0 < need <= L.TKA_NOALLOC_SCRATCH_BYTES
                ws = torch.empty(need, dtype=torch.uint8, device="cuda")
                a.workspace, a.workspace_bytes = ws.data_ptr(), need
                L.check(lib.tka_sparse_decode_step(C.byref(a)), "tka_sparse_decode_step")
            torch.cuda.synchronize()
            outs.append((out, tidx, tval))
        for name, r, g in zip(("out", "topk_idx", "topk_val"), outs[0], outs[1]):
            assert torch.equal(r.contiguous().view(torch.uint8), g.contiguous().view(torch.uint8)), "%s differs between the two entry points" % name
        tidx, outf = outs[1][1].cpu().numpy(), outs[1][0].float().cpu().numpy()
        for b in range(B):
            for h in range(H):
                ro, ri, rv, ru = oracle.sparse_decode_step(qb[b, h * G:(h + 1) * G], Kb[b, :, h], Vb[b, :, h], dtype, G, k, sink, local, SCALE)
                assert np.array_equal(tidx[b, h], ri)
                assert (np.abs(outf[b, h * G:(h + 1) * G] - ro) < 2e-3).all()


@pytest.mark.gpu
def test_noalloc_step_captured_in_a_graph():
    """The use the entry point is for: captured into a HIP graph (after one eager call, which looks up the address of the
    built-in buffer) and replayed - twice, with new queries each time and, between the replays, an eager call of another
    shape that leaves the buffer in another layout.  Every replay must give what the eager call with the workspace gives."""
    lib = L.lib()
    announce("sparse_decode_step_noalloc captured in a graph, two replays with another layout of the scratch in between")
    rng = np.random.default_rng(2026)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 1, 2, 4, 70000, 1024, 16, 128

    def tensors(B, H, G, N, k, sink, local):
        q = to_dev(randn_bits(rng, (B, H * G, 128), dtype), dtype)
        K, V = to_dev(randn_bits(rng, (B, N, H, 128), dtype), dtype), to_dev(randn_bits(rng, (B, N, H, 128), dtype), dtype)
        out = torch.zeros((B, H * G, 128), dtype=torch.float16, device="cuda")
        tidx = torch.zeros((B, H, k), dtype=torch.int32, device="cuda")
        tval = torch.zeros((B, H, k), dtype=torch.float32, device="cuda")
        uidx = torch.zeros((B, H, k + sink + local), dtype=torch.int32, device="cuda")
        ucnt = torch.zeros((B, H), dtype=torch.int32, device="cuda")
        return q, K, V, out, tidx, tval, uidx, ucnt

    q, K, V, out, tidx, tval, uidx, ucnt = tensors(B, H, G, N, k, sink, local)
    q2, K2, V2, out2, tidx2, tval2, uidx2, ucnt2 = tensors(2, 2, 2, 5000, 300, 8, 8)       # the other layout
    a = _args(q, K, V, out, k, sink, local, G, tidx, tval, uidx, ucnt)
    other = _args(q2, K2, V2, out2, 300, 8, 8, 2, tidx2, tval2, uidx2, ucnt2)
    L.check(lib.tka_sparse_decode_step_noalloc(C.byref(a)), "first call, eager")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        a.stream = side.cuda_stream
        L.check(lib.tka_sparse_decode_step_noalloc(C.byref(a)), "warm-up on the side stream")
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            a.stream = torch.cuda.current_stream().cuda_stream
            L.check(lib.tka_sparse_decode_step_noalloc(C.byref(a)), "captured call")
    torch.cuda.synchronize()
    # the reference for every replay: the workspace form, eager
    ref_out, ref_tidx, ref_uidx, ref_ucnt = (torch.zeros_like(t) for t in (out, tidx, uidx, ucnt))
    ref_tval = torch.zeros_like(tval)
    r = _args(q, K, V, ref_out, k, sink, local, G, ref_tidx, ref_tval, ref_uidx, ref_ucnt)
    need = lib.tka_sparse_decode_workspace_bytes(C.byref(r))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    r.workspace, r.workspace_bytes = ws.data_ptr(), need
    for it in range(2):
        q.copy_(to_dev(randn_bits(rng, (B, H * G, 128), dtype), dtype))
        r.stream = other.stream = torch.cuda.current_stream().cuda_stream
        L.check(lib.tka_sparse_decode_step(C.byref(r)), "reference step")
        L.check(lib.tka_sparse_decode_step_noalloc(C.byref(other)), "eager call of another shape")   # another layout in the scratch
        for t in (out, tidx, tval, uidx, ucnt):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, g_, r_ in (("out", out, ref_out), ("topk_idx", tidx, ref_tidx), ("topk_val", tval, ref_tval), ("union_idx", uidx, ref_uidx),
                             ("union_count", ucnt, ref_ucnt)):
            assert torch.equal(g_.view(torch.uint8), r_.view(torch.uint8)), "replay %d: %s differs from the eager step" % (it, name)


def test_noalloc_step_rejects_what_does_not_fit():
    """Batch 16 of the 128k configuration needs 203 MiB of scratch: refused with TKA_ESCRATCH before any HIP call
    (so this runs without a GPU)."""
    lib = L.lib()
    a = L.SparseDecodeArgs()
    a.q, a.keys, a.values, a.out = 0x1000, 0x2000, 0x3000, 0x4000     # never dereferenced
    a.dtype, a.out_dtype, a.batch, a.num_kv_heads, a.group, a.head_dim = L.TKA_F16, L.TKA_BF16, 16, 8, 4, 128
    a.k, a.sink, a.local, a.seq_len = 2048, 64, 512, 131072
    a.q_stride_b = a.out_stride_b = 32 * 128
    a.kv_stride_b, a.kv_stride_n, a.kv_stride_h, a.scale = 131072 * 1024, 1024, 128, SCALE
    assert lib.tka_sparse_decode_workspace_bytes(C.byref(a)) > L.TKA_NOALLOC_SCRATCH_BYTES
    assert lib.tka_sparse_decode_step_noalloc(C.byref(a)) == L.TKA_ESCRATCH
    assert "scratch" in L.status_string(L.TKA_ESCRATCH)
    a.k = 0
    assert lib.tka_sparse_decode_step_noalloc(C.byref(a)) == L.TKA_EINVAL
