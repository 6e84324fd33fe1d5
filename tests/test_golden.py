"""Committed fixtures (tests/golden/, written by make_golden.py: an end-to-end step, a call of the operator, a
two-level / centre-only selection): the oracle must still reproduce them, and on a GPU the library must match them
through the C ABI."""
import os

import numpy as np
import pytest

import oracle

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sparse_decode_small.npz"))
N, H, G, K_TOP, SINK, LOCAL = (int(x) for x in FIX["params"])
SCALE = float(np.float32(1.0 / np.sqrt(128.0)))
CASES = [("f16", oracle.F16), ("bf16", oracle.BF16)]


@pytest.mark.parametrize("tag,dtype", CASES)
def test_oracle_reproduces_fixture(tag, dtype):
    q, K, V = FIX[tag + "_q"], FIX[tag + "_K"], FIX[tag + "_V"]
    for h in range(H):
        o, ti, tv, u = oracle.sparse_decode_step(q[h * G:(h + 1) * G], K[:, h], V[:, h], dtype, G, K_TOP, SINK, LOCAL, SCALE)
        assert np.array_equal(ti, FIX[tag + "_topk_idx"][h])
        assert np.array_equal(tv.view(np.uint32), FIX[tag + "_topk_val"][h].view(np.uint32))
        assert len(u) == FIX[tag + "_union_count"][h] and np.array_equal(u, FIX[tag + "_union"][h][:len(u)])
        assert np.abs(o - FIX[tag + "_out"][h]).max() < 1e-12


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", CASES)
def test_gpu_matches_fixture(tag, dtype):
    import torch
    from tests.util import announce, f32_of, to_dev
    from topk_attn_amd import ops
    announce("golden fixture %s" % tag)
    q, K, V = FIX[tag + "_q"], FIX[tag + "_K"], FIX[tag + "_V"]
    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(to_dev(q[None], dtype), to_dev(K[None], dtype), to_dev(V[None], dtype),
                                                         K_TOP, SINK, LOCAL, SCALE, G, out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert np.array_equal(tidx[0].cpu().numpy(), FIX[tag + "_topk_idx"])
    assert np.array_equal(tval[0].cpu().numpy().view(np.uint32), FIX[tag + "_topk_val"].view(np.uint32))
    cnt = ucnt[0].cpu().numpy()
    assert np.array_equal(cnt, FIX[tag + "_union_count"])
    for h in range(H):
        assert np.array_equal(uidx[0, h, :cnt[h]].cpu().numpy(), FIX[tag + "_union"][h][:cnt[h]])
    assert np.abs(f32_of(out)[0] - FIX[tag + "_out"].reshape(H * G, 128)).max() < 2e-3


OP = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "retrieval_op_small.npz"))
OP_B, OP_N, OP_H, OP_CHUNKS, OP_TOPK = (int(x) for x in OP["params"])


@pytest.mark.parametrize("tag,dtype", CASES)
def test_oracle_reproduces_operator_fixture(tag, dtype):
    q, K, V = OP[tag + "_q"], OP[tag + "_K"], OP[tag + "_V"]
    for b in range(OP_B):
        for h in range(OP_H):
            o, i, v = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, OP_CHUNKS, OP_TOPK, 1.0)
            assert np.array_equal(i, OP[tag + "_idx"][b, h])
            assert np.array_equal(v.view(np.uint32), OP[tag + "_val"][b, h].view(np.uint32))
            assert np.abs(o - OP[tag + "_out"][b, h]).max() < 1e-12


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", CASES)
def test_gpu_matches_operator_fixture(tag, dtype):
    """The operator and its selection stage on the fixture: 128 short segments over caches shared by 16 batch entries."""
    import torch
    from tests.util import TORCH_DT, announce, f32_of, to_dev
    from topk_attn_amd import ops
    announce("golden operator fixture %s" % tag)
    q, K, V = to_dev(OP[tag + "_q"], dtype), to_dev(OP[tag + "_K"], dtype), to_dev(OP[tag + "_V"], dtype)
    out = torch.zeros((OP_B, OP_H, 128), dtype=TORCH_DT[dtype], device="cuda")
    ops.retrieval_attention(q, K, V, out, OP_TOPK, OP_CHUNKS, 1.0)
    idx, val = ops.gemv_topk(q, K, OP_TOPK, group=1, scale=1.0, num_chunks=OP_CHUNKS)
    torch.cuda.synchronize()
    assert np.array_equal(idx.cpu().numpy(), OP[tag + "_idx"])
    assert np.array_equal(val.cpu().numpy().view(np.uint32), OP[tag + "_val"].view(np.uint32))
    tol = 2e-3 if dtype == oracle.F16 else 2e-3 + np.abs(OP[tag + "_out"]).max() * 2.0 ** -8   # (bf16 output: its own rounding)
    assert np.abs(f32_of(out) - OP[tag + "_out"]).max() < tol


CL = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cluster_small.npz"))
CL_CSZ, CL_CLEN, CL_TOPC, CL_K = (int(x) for x in CL["params"])


@pytest.mark.parametrize("tag,dtype", CASES)
def test_oracle_reproduces_cluster_fixture(tag, dtype):
    q, cen, keys = CL[tag + "_q"], CL[tag + "_centers"], CL[tag + "_keys"]
    for h in range(q.shape[0]):
        two = oracle.cluster_topk(q[h], cen[h], keys[:, h, :], dtype, CL_TOPC, CL_CLEN, CL_K, 1.0)
        assert np.array_equal(two, CL[tag + "_two_level"][h])
        out, ids, val = oracle.center_topk_expand(q[h], cen[h], dtype, CL_TOPC, CL_CLEN, 1.0)
        assert np.array_equal(out, CL[tag + "_expand"][h]) and np.array_equal(ids, CL[tag + "_center_ids"][h])
        assert np.array_equal(val.view(np.uint32), CL[tag + "_center_val"][h].view(np.uint32))
        assert list(ids[:3]) == [3, 7, 9]          # the three tied centroids, lower id first


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", CASES)
def test_gpu_matches_cluster_fixture(tag, dtype):
    """Two-level and centre-only selection on the fixture (fp16: 128 segments, centre stage inside the token launch;
    bf16: 16 segments, centre stage as its own launch)."""
    import torch
    from tests.util import announce, to_dev
    from topk_attn_amd import ops
    announce("golden cluster fixture %s" % tag)
    q, cen, keys = to_dev(CL[tag + "_q"], dtype), to_dev(CL[tag + "_centers"], dtype), to_dev(CL[tag + "_keys"], dtype)
    two = ops.cluster_gemv_topk(q, cen, keys, CL_TOPC, CL_CLEN, CL_K, 1.0)
    exp = ops.center_topk_expand(q, cen, CL_TOPC, CL_CLEN, 1.0)
    torch.cuda.synchronize()
    assert np.array_equal(two.cpu().numpy(), CL[tag + "_two_level"])
    exp = exp[0] if isinstance(exp, (tuple, list)) else exp
    assert np.array_equal(exp.cpu().numpy(), CL[tag + "_expand"])
