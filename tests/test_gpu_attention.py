"""Split-K flash-decoding, LSE combine, index union, the retrieval_attention op and the end-to-end step,
each against the fp64 oracle at 2e-3 max-abs (fp16/bf16 I/O)."""
import numpy as np
import pytest
import torch

import oracle
from tests.util import announce, bits_of, f32_of, randn_bits, to_dev

pytestmark = pytest.mark.gpu

TOL = 2e-3
SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


def out_tol(ref, out_is_bf16):
    """2e-3 max-abs on the computed value; a bfloat16 OUTPUT adds its own rounding of up to half an ulp
    (2^-9 relative, 3.9e-3 at |x| in [1,2)), which no kernel can avoid, so it is allowed on top."""
    return TOL + (np.abs(ref) * 2.0 ** -8 if out_is_bf16 else 0.0)


def _dense_ref(q, K, V, dtype, G, scale):
    B, Hq = q.shape[:2]
    out = np.empty((B, Hq, 128))
    lse = np.empty((B, Hq))
    for b in range(B):
        for hq in range(Hq):
            h = hq // G
            Kh = K[:, h] if K.ndim == 3 else K[b, :, h]
            Vh = V[:, h] if V.ndim == 3 else V[b, :, h]
            out[b, hq], lse[b, hq] = oracle.attention_f64(q[b, hq], Kh, Vh, dtype, scale=scale)
    return out, lse


@pytest.mark.parametrize("dtype,B,H,G,N,splits", [
    (oracle.F16, 1, 8, 4, 4096, 0), (oracle.F16, 2, 2, 1, 1000, 3), (oracle.BF16, 1, 2, 8, 3333, 7),
    (oracle.F16, 1, 1, 2, 77, 1), (oracle.BF16, 2, 4, 4, 2048, 64), (oracle.BF16, 3, 2, 1, 700, 1),
    # sixteen and thirty-two KV heads with one query head each (rows of a head 4 and 8 KB apart: the heads in the grid's x)
    (oracle.F16, 2, 16, 1, 1500, 0), (oracle.BF16, 1, 32, 1, 999, 5), (oracle.F16, 1, 16, 1, 300, 1)])
def test_flash_decode_dense(dtype, B, H, G, N, splits):
    from topk_attn_amd import ops
    announce("flash_decode dense dtype=%d B=%d H=%d G=%d N=%d splits=%d" % (dtype, B, H, G, N, splits))
    rng = np.random.default_rng(N + G)
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)
    out, lse = ops.flash_decode(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), SCALE, group=G,
                                num_splits=splits, return_lse=True)
    torch.cuda.synchronize()
    ref, ref_lse = _dense_ref(q, K, V, dtype, G, SCALE)
    assert (np.abs(f32_of(out) - ref) < out_tol(ref, dtype == oracle.BF16)).all()
    assert np.abs(lse.cpu().numpy() - ref_lse).max() < 1e-3


def test_flash_decode_split_invariance():
    """Split-K must not change the result beyond rounding: S = 1, 5, 64 agree."""
    from topk_attn_amd import ops
    announce("flash_decode split invariance")
    rng = np.random.default_rng(5)
    dtype = oracle.F16
    q, K, V = randn_bits(rng, (1, 8, 128), dtype), randn_bits(rng, (6000, 2, 128), dtype), randn_bits(rng, (6000, 2, 128), dtype)
    outs = [f32_of(ops.flash_decode(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), SCALE, group=4, num_splits=s))
            for s in (1, 5, 64)]
    assert np.abs(outs[0] - outs[1]).max() < 1e-3 and np.abs(outs[0] - outs[2]).max() < 1e-3


def test_flash_decode_dominant_and_uniform():
    """One dominant logit returns that V row; equal keys return the mean of V (no oracle involved)."""
    from topk_attn_amd import ops
    announce("flash_decode closed forms")
    rng = np.random.default_rng(9)
    dtype = oracle.F16
    N = 2000
    V = rng.standard_normal((N, 1, 128))
    qv = rng.standard_normal((1, 1, 128))
    Kv = np.zeros((N, 1, 128))
    out = ops.flash_decode(to_dev(oracle.to_bits(qv, dtype), dtype), to_dev(oracle.to_bits(Kv, dtype), dtype),
                           to_dev(oracle.to_bits(V, dtype), dtype), 1.0)
    Vr = oracle.from_bits(oracle.to_bits(V, dtype), dtype)
    assert np.abs(f32_of(out)[0, 0] - Vr[:, 0].mean(0)).max() < TOL
    Kv[1234, 0] = qv[0, 0] * 4.0
    out = ops.flash_decode(to_dev(oracle.to_bits(qv, dtype), dtype), to_dev(oracle.to_bits(Kv, dtype), dtype),
                           to_dev(oracle.to_bits(V, dtype), dtype), 1.0)
    assert np.abs(f32_of(out)[0, 0] - Vr[1234, 0]).max() < TOL


@pytest.mark.parametrize("dtype,G", [(oracle.F16, 1), (oracle.F16, 4), (oracle.BF16, 8)])
def test_flash_decode_indexed(dtype, G):
    """Gathered attention over ragged index lists (counts differ per head, one list empty-ish, ids out of range skipped)."""
    from topk_attn_amd import ops
    announce("flash_decode indexed dtype=%d G=%d" % (dtype, G))
    rng = np.random.default_rng(17 + G)
    B, H, N, Lmax = 2, 3, 5000, 700
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)
    idx = np.full((B, H, Lmax), -1, np.int32)
    cnt = np.zeros((B, H), np.int32)
    for b in range(B):
        for h in range(H):
            c = [Lmax, 1, 333][(b * H + h) % 3]
            idx[b, h, :c] = np.sort(rng.choice(N, c, replace=False))
            cnt[b, h] = c
    out = ops.flash_decode(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), SCALE, group=G,
                           kv_idx=torch.from_numpy(idx).cuda(), kv_count=torch.from_numpy(cnt).cuda())
    torch.cuda.synchronize()
    out = f32_of(out)
    for b in range(B):
        for hq in range(H * G):
            h = hq // G
            ref, _ = oracle.attention_f64(q[b, hq], K[b, :, h], V[b, :, h], dtype, idx=idx[b, h], count=int(cnt[b, h]), scale=SCALE)
            assert (np.abs(out[b, hq] - ref) < out_tol(ref, dtype == oracle.BF16)).all()


@pytest.mark.parametrize("dtype,G,logits", [(oracle.F16, 1, False), (oracle.F16, 4, False), (oracle.BF16, 8, False), (oracle.F16, 1, True)])
def test_flash_decode_indexed_skips_ids_outside_the_cache(dtype, G, logits):
    """Ids below 0 or at/after seq_len in the MIDDLE of a list are skipped (retrieval_attention.cu:1325); the
    kernels load row 0 in their place, so row 0 of K and V is filled with infinities here: nothing of it may
    reach the output (0 * inf).  Token 0 itself is not in the list."""
    from topk_attn_amd import _lib as L
    from topk_attn_amd import ops
    announce("flash_decode indexed with ids outside the cache, dtype=%d G=%d logits=%s" % (dtype, G, logits))
    rng = np.random.default_rng(170 + G)
    B, H, N, Lmax = 1, 2, 3000, 600
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)
    inf_bits = oracle.to_bits(np.array([np.inf]), dtype)[0]
    K[:, 0], V[:, 0] = inf_bits, inf_bits
    idx = np.empty((B, H, Lmax), np.int32)
    for h in range(H):
        idx[0, h] = np.sort(rng.choice(np.arange(1, N), Lmax, replace=False))
    bad = [3, 40, 41, 100, 257, 258, 511]
    idx[0, 0, bad] = [-1, N, N + 7, -5, 2 ** 31 - 1, -2 ** 31, N]
    idx[0, 1, 300] = -1
    lg = (rng.standard_normal((B, H, Lmax)) * 2).astype(np.float32) if logits else None
    out = ops.flash_decode(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), 1.0 if logits else SCALE, group=G,
                           kv_idx=torch.from_numpy(idx).cuda(), kv_logit=torch.from_numpy(lg).cuda() if logits else None,
                           softmax_mode=L.TKA_SOFTMAX_SCALED)
    torch.cuda.synchronize()
    out = f32_of(out)
    assert np.isfinite(out).all()
    for hq in range(H * G):
        h = hq // G
        keep = (idx[0, h] >= 0) & (idx[0, h] < N)
        ref, _ = oracle.attention_f64(q[0, hq], K[0, :, h], V[0, :, h], dtype, idx=idx[0, h][keep],
                                      logit=lg[0, h][keep] if logits else None, scale=SCALE)
        assert (np.abs(out[0, hq] - ref) < out_tol(ref, dtype == oracle.BF16)).all()


def test_lse_combine_matches_unsplit():
    from topk_attn_amd import ops
    announce("lse_combine")
    rng = np.random.default_rng(21)
    R, S = 6, 9
    m = rng.standard_normal((R, S)).astype(np.float32) * 5
    l = rng.uniform(0.5, 50, (R, S)).astype(np.float32)
    acc = rng.standard_normal((R, S, 128)).astype(np.float32) * 10
    l[0, 3] = 0.0
    m[0, 3] = -np.inf  # empty split
    m[1, :] = 2.0      # equal maxima
    out, lse = ops.lse_combine(torch.from_numpy(m).cuda(), torch.from_numpy(l).cuda(), torch.from_numpy(acc).cuda(),
                               torch.float16, return_lse=True)
    torch.cuda.synchronize()
    for r in range(R):
        ref, ref_lse = oracle.lse_combine(m[r], l[r], acc[r])
        assert np.abs(f32_of(out)[r] - ref).max() < TOL * max(1.0, np.abs(ref).max())
        assert abs(lse[r].item() - ref_lse) < 1e-3


@pytest.mark.parametrize("k,sink,local,n", [(2048, 64, 512, 131072), (100, 0, 0, 5000), (300, 16, 16, 400), (64, 64, 64, 100),
                                            (2048, 64, 512, 65536), (4096, 0, 1, 65535), (2048, 64, 512, 262144), (1024, 8, 8, 300000)])
def test_index_union(k, sink, local, n):
    from topk_attn_amd import ops
    announce("index_union k=%d sink=%d local=%d n=%d" % (k, sink, local, n))
    rng = np.random.default_rng(k)
    S = 5
    ids = np.stack([rng.choice(n, k, replace=False) for _ in range(S)]).astype(np.int32)
    ids[0, :min(k, sink + 5)] = np.arange(min(k, sink + 5))  # overlap with the sink range
    out, cnt = ops.index_union(torch.from_numpy(ids).cuda(), sink, local, n)
    torch.cuda.synchronize()
    out, cnt = out.cpu().numpy(), cnt.cpu().numpy()
    for s in range(S):
        want = np.union1d(np.union1d(ids[s], np.arange(min(sink, n))), np.arange(max(n - local, 0), n))
        eo, ec = oracle.index_union(ids[s], sink, local, n)
        assert ec == len(want) and np.array_equal(eo[:ec], want)      # pins the oracle against numpy
        assert cnt[s] == len(want) and np.array_equal(out[s, :cnt[s]], want)
        assert (out[s, cnt[s]:] == -1).all()


@pytest.mark.parametrize("topk", [32, 128, 256, 512, 1024])
def test_retrieval_attention_op(topk):
    """The reference's own test (test_ra.py:162-205): B=4, randn*0.1, seq 8192, 32 heads, all K; tolerance 2e-3
    against the fp64 oracle instead of the reference's 1e-2 against fp16 torch."""
    from topk_attn_amd import retrieval_attention_cpp as ra
    announce("retrieval_attention op topk=%d" % topk)
    rng = np.random.default_rng(0)
    dtype = oracle.F16
    B, H, N = 4, 32, 8192
    q, K, V = randn_bits(rng, (B, H, 128), dtype, 0.1), randn_bits(rng, (N, H, 128), dtype, 0.1), randn_bits(rng, (N, H, 128), dtype, 0.1)
    out = torch.zeros((B, H, 128), dtype=torch.float16, device="cuda")
    getattr(ra, "retrieval_attention_%d" % topk)(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), out)
    torch.cuda.synchronize()
    got = f32_of(out)
    for b in range(B):
        for h in range(0, H, 5):
            ref, _, _ = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, 4, topk, 1.0)
            assert np.abs(got[b, h] - ref).max() < TOL


@pytest.mark.parametrize("B,topk", [(4, 128), (32, 256)])
def test_retrieval_attention_op_matrix_core_scores(B, topk):
    """The operator with score_mode = TKA_SCORE_MATRIX (its scoring stage on the matrix cores): same tolerance against
    the fp64 oracle as the canonical form (a token at the very edge of a chunk's top K may change places with its
    neighbour in score; its weight is about 1/(4K))."""
    from topk_attn_amd import _lib as L
    from topk_attn_amd import retrieval_attention_cpp as ra
    announce("retrieval_attention op on the matrix cores B=%d topk=%d" % (B, topk))
    rng = np.random.default_rng(5)
    dtype = oracle.F16
    H, N = 32, 8192
    q, K, V = randn_bits(rng, (B, H, 128), dtype, 0.1), randn_bits(rng, (N, H, 128), dtype, 0.1), randn_bits(rng, (N, H, 128), dtype, 0.1)
    out = torch.zeros((B, H, 128), dtype=torch.float16, device="cuda")
    ra.retrieval_attention(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), out, topk, score_mode=L.TKA_SCORE_MATRIX)
    torch.cuda.synchronize()
    got = f32_of(out)
    for b in range(0, B, 7):
        for h in range(0, H, 5):
            ref, _, _ = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, 4, topk, 1.0)
            assert np.abs(got[b, h] - ref).max() < TOL


@pytest.mark.parametrize("B,topk", [(9, 128), (33, 1024), (2, 32)])
def test_retrieval_attention_op_batches(B, topk):
    """Batches whose keys are scored several entries per pass (with a ragged last tile), selected one segment per
    small workgroup, and, from 32 entries on, attended by one workgroup per row without a combine launch."""
    from topk_attn_amd import retrieval_attention_cpp as ra
    announce("retrieval_attention op B=%d topk=%d" % (B, topk))
    rng = np.random.default_rng(B)
    dtype = oracle.F16
    H, N = 32, 8192
    q, K, V = randn_bits(rng, (B, H, 128), dtype, 0.1), randn_bits(rng, (N, H, 128), dtype, 0.1), randn_bits(rng, (N, H, 128), dtype, 0.1)
    out = torch.zeros((B, H, 128), dtype=torch.float16, device="cuda")
    getattr(ra, "retrieval_attention_%d" % topk)(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), out)
    torch.cuda.synchronize()
    got = f32_of(out)
    for b in sorted({0, 1, B // 2, B - 2, B - 1}):
        for h in range(b % 7, H, 7):
            ref, _, _ = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, 4, topk, 1.0)
            assert np.abs(got[b, h] - ref).max() < TOL, "b=%d h=%d" % (b, h)


@pytest.mark.parametrize("binding", ["ctypes", "extension"])
def test_harness_ra(capfd, binding):
    """The harness in the shape of the reference's test_ra.py: PASSED lines per variant, a performance table built
    from the timing line the op prints on request, exit status 0; through the ctypes binding and through the compiled
    PyTorch extension module.  (Parity proper is checked against the oracle in the tests above; the harness's own
    torch model is held to 5e-3 here, test_ra.py:202 uses 1e-2.)"""
    from topk_attn_amd import harness_ra
    announce("harness_ra --batch 2 --topk 32 256 --binding %s" % binding)
    rc = harness_ra.main(["--batch", "2", "--topk", "32", "256", "--tol", "5e-3", "--binding", binding])
    text = capfd.readouterr().out
    assert rc == 0, text[-2000:]
    assert text.count("PASSED") == 12 and "FAILED" not in text
    rows = [ln for ln in text.splitlines() if ln.startswith("| 32 ") or ln.startswith("| 256 ")]
    assert len(rows) == 12 and all(float(r.split("|")[3]) > 0 for r in rows)


def test_retrieval_attention_variants_agree():
    """All six reference variants are one function here: identical bits."""
    from topk_attn_amd import retrieval_attention_cpp as ra
    from topk_attn_amd._lib import RA_VARIANTS
    announce("retrieval_attention variants")
    rng = np.random.default_rng(1)
    dtype = oracle.F16
    q, K, V = randn_bits(rng, (2, 32, 128), dtype, 0.1), randn_bits(rng, (8192, 32, 128), dtype, 0.1), randn_bits(rng, (8192, 32, 128), dtype, 0.1)
    outs = []
    for v in RA_VARIANTS:
        out = torch.zeros((2, 32, 128), dtype=torch.float16, device="cuda")
        getattr(ra, "retrieval_attention%s_128" % v)(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), out)
        outs.append(bits_of(out))
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])


def test_bind_cpp_style_caller_runs():
    """The caller that declares the launchers as the reference's bind.cpp does (C++ linkage, `half` pointers, built
    by g++ alone) calls one of them on the GPU; the output equals the C symbol's bit for bit."""
    import os
    import subprocess
    announce("tka_bind_link_check run")
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "topk_attn_amd", "lib", "tka_bind_link_check")
    r = subprocess.run([exe, "run"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "outputs identical" in r.stdout


def test_reference_named_launchers():
    """The C-linkage launchers with the reference's names (bind.cpp:5-243), called on the default stream."""
    import ctypes as C
    from topk_attn_amd import _lib as L
    announce("launch_retrieval_attention_* shims")
    rng = np.random.default_rng(2)
    dtype = oracle.F16
    q, K, V = randn_bits(rng, (3, 32, 128), dtype, 0.1), randn_bits(rng, (8192, 32, 128), dtype, 0.1), randn_bits(rng, (8192, 32, 128), dtype, 0.1)
    qd, Kd, Vd = to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype)
    torch.cuda.synchronize()
    for name, topk in (("launch_retrieval_attention_256", 256), ("launch_retrieval_attention_two_kernels_32", 32)):
        out = torch.zeros((3, 32, 128), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        getattr(L.lib(), name)(qd.data_ptr(), Kd.data_ptr(), Vd.data_ptr(), out.data_ptr(), 3)
        torch.cuda.synchronize()
        got = f32_of(out)
        for b, h in ((0, 0), (2, 31), (1, 13)):
            ref, _, _ = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, 4, topk, 1.0)
            assert np.abs(got[b, h] - ref).max() < TOL


_LAUNCHER_MATRIX_SCORES = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
import oracle
from topk_attn_amd import _lib as L, ops
from tests.util import f32_of, randn_bits, to_dev
rng = np.random.default_rng(12)
dtype = oracle.F16
q, K, V = randn_bits(rng, (4, 32, 128), dtype, 0.1), randn_bits(rng, (8192, 32, 128), dtype, 0.1), randn_bits(rng, (8192, 32, 128), dtype, 0.1)
qd, Kd, Vd = to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype)
out = torch.zeros((4, 32, 128), dtype=torch.float16, device="cuda")
torch.cuda.synchronize()
ops.profile_enable(True)
L.lib().launch_retrieval_attention_128(qd.data_ptr(), Kd.data_ptr(), Vd.data_ptr(), out.data_ptr(), 4)
torch.cuda.synchronize()
ran = ops.profile_read()
assert "gemv_scores_mfma" in ran, sorted(ran)
got = f32_of(out)
for b, h in ((0, 0), (3, 31), (2, 7)):
    ref, _, _ = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, 4, 128, 1.0)
    assert np.abs(got[b, h] - ref).max() < 2e-3
print("launcher with matrix-core scores ok")
"""


def test_ra_launchers_matrix_core_scores_by_environment():
    """TKA_RA_SCORE_MODE=1 makes the thirty fixed-shape launchers (which have no argument for it) score on the matrix
    cores.  The variable is read once per process, so the case runs in a child process started with it set, before
    any GPU call: the kernel that ran, and the output against the oracle at 2e-3."""
    import os
    import subprocess
    import sys
    announce("launch_retrieval_attention_128 in a child process with TKA_RA_SCORE_MODE=1")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, TKA_RA_SCORE_MODE="1")
    done = subprocess.run([sys.executable, "-c", _LAUNCHER_MATRIX_SCORES, root], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and "ok" in done.stdout, done.stdout[-2000:] + done.stderr[-4000:]


@pytest.mark.parametrize("dtype,out_dt,B,H,G,N,k,sink,local", [
    (oracle.F16, torch.bfloat16, 2, 2, 4, 16384, 2048, 64, 512),
    (oracle.BF16, torch.bfloat16, 1, 2, 8, 8192, 512, 16, 128),
    (oracle.F16, torch.float16, 1, 1, 1, 3000, 100, 0, 0)])
def test_sparse_decode_step(dtype, out_dt, B, H, G, N, k, sink, local):
    """End to end: heavy-hitter keys (1% scaled x4), top-k per KV head on the group-summed score, union with
    sink and local window, attention per query head."""
    from topk_attn_amd import ops
    announce("sparse_decode_step dtype=%d B=%d H=%d G=%d N=%d k=%d" % (dtype, B, H, G, N, k))
    rng = np.random.default_rng(4)
    Kf = rng.standard_normal((B, N, H, 128))
    for b in range(B):
        for h in range(H):
            hh = rng.permutation(N)[:N // 100]
            Kf[b, hh, h] *= 4.0
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), oracle.to_bits(Kf, dtype), randn_bits(rng, (B, N, H, 128), dtype)
    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink,
                                                         local, SCALE, G, out_dtype=out_dt)
    torch.cuda.synchronize()
    out, tidx, tval, uidx, ucnt = f32_of(out), tidx.cpu().numpy(), tval.cpu().numpy(), uidx.cpu().numpy(), ucnt.cpu().numpy()
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(q[b, h * G:(h + 1) * G], K[b, :, h], V[b, :, h], dtype, G, k, sink,
                                                       local, SCALE)
            assert np.array_equal(tidx[b, h], ri), "top-k indices differ"
            assert np.array_equal(tval[b, h].view(np.uint32), rv.view(np.uint32))
            assert ucnt[b, h] == len(ru) and np.array_equal(uidx[b, h, :len(ru)], ru)
            assert (np.abs(out[b, h * G:(h + 1) * G] - ro) < out_tol(ro, out_dt == torch.bfloat16)).all()


@pytest.mark.parametrize("dtype,B,H,G,N,k,sink,local,kind", [
    (oracle.F16, 2, 2, 4, 16384, 2048, 64, 512, "heavy"),
    (oracle.BF16, 1, 2, 8, 70000, 1024, 16, 128, "levels"),
    (oracle.F16, 1, 2, 2, 66000, 2000, 8, 8, "equal"),
    (oracle.F16, 1, 2, 1, 5000, 300, 8, 8, "equal"),
    (oracle.F16, 1, 1, 2, 4099, 129, 0, 0, "heavy"),
    (oracle.BF16, 1, 3, 4, 8000, 8000, 4, 4, "heavy"),
    (oracle.F16, 1, 2, 4, 1500, 300, 8, 8, "heavy"),
    (oracle.BF16, 1, 2, 2, 2048, 2048, 0, 16, "levels"),
    (oracle.F16, 1, 1, 8, 16384, 4000, 64, 512, "equal"),
    (oracle.F16, 1, 2, 2, 5000, 700, 3000, 3000, "heavy"),        # sink range and local window overlap
    (oracle.BF16, 3, 2, 4, 9000, 2048, 1, 8999, "levels"),        # the window covers nearly everything
    (oracle.F16, 2, 2, 1, 12289, 2048, 5, 7, "equal"),
    # 16385 .. 65536 tokens with the list asked for: the common-cut route with a list of its own for the attention, the
    # caller's ascending list from the rank-ordered ids by one more launch (a bitmap of the sequence)
    (oracle.F16, 1, 2, 4, 32768, 2048, 64, 512, "heavy"),
    (oracle.BF16, 2, 3, 2, 20001, 1000, 100, 300, "levels"),
    (oracle.F16, 1, 8, 4, 24000, 1400, 6000, 22000, "heavy"),     # more than 65536 rows; range and window overlap
    (oracle.F16, 1, 1, 2, 65536, 2048, 0, 0, "equal")])
def test_sparse_decode_step_union_only(dtype, B, H, G, N, k, sink, local, kind, out_dt=torch.float16):
    """Production form of the step: no rank-ordered output.  The union list must still equal the oracle's bit for
    bit — with heavy hitters, with 16-level keys (large tie buckets), with all keys equal (every token ties) and
    with k = N."""
    from topk_attn_amd import ops
    announce("sparse_decode_step union-only dtype=%d B=%d H=%d G=%d N=%d k=%d %s" % (dtype, B, H, G, N, k, kind))
    rng = np.random.default_rng(N + k)
    if kind == "levels":
        Kf = np.linspace(-2, 2, 16)[rng.integers(0, 16, (B, N, H, 128))]
    elif kind == "equal":
        Kf = np.broadcast_to(rng.standard_normal((1, 1, 1, 128)), (B, N, H, 128)).copy()
    else:
        Kf = rng.standard_normal((B, N, H, 128))
        Kf[:, rng.permutation(N)[:max(1, N // 100)]] *= 4.0
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), oracle.to_bits(Kf, dtype), randn_bits(rng, (B, N, H, 128), dtype)
    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink,
                                                         local, SCALE, G, out_dtype=out_dt, want_topk=False)
    torch.cuda.synchronize()
    assert tidx is None and tval is None
    out, uidx, ucnt = f32_of(out), uidx.cpu().numpy(), ucnt.cpu().numpy()
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(q[b, h * G:(h + 1) * G], K[b, :, h], V[b, :, h], dtype, G, k, sink,
                                                       local, SCALE)
            assert ucnt[b, h] == len(ru) and np.array_equal(uidx[b, h, :len(ru)], ru), "union differs (b=%d h=%d)" % (b, h)
            assert (np.abs(out[b, h * G:(h + 1) * G] - ro) < out_tol(ro, False)).all()


def test_sparse_decode_step_shared_cache_long():
    """The step over ONE cache that the batch shares (kv_stride_b = 0) at a length of the candidate route: the keys are
    scored for a tile of batch entries per pass; top-k, union list and output of every (entry, head) against the oracle."""
    from topk_attn_amd import ops
    announce("sparse_decode_step, cache shared by a batch of 5, N=70000 k=1024 G=4")
    rng = np.random.default_rng(4242)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 5, 2, 4, 70000, 1024, 16, 128
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (N, H, 128), dtype), randn_bits(rng, (N, H, 128), dtype)
    ops.profile_reset()
    ops.profile_enable(True)
    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink, local,
                                                         SCALE, G, out_dtype=torch.float16)
    torch.cuda.synchronize()
    ran = ops.profile_read()
    ops.profile_enable(False)
    assert "gemv_candidates_shared" in ran, sorted(ran)
    out, tidx, tval, uidx, ucnt = f32_of(out), tidx.cpu().numpy(), tval.cpu().numpy(), uidx.cpu().numpy(), ucnt.cpu().numpy()
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(q[b, h * G:(h + 1) * G], K[:, h], V[:, h], dtype, G, k, sink, local, SCALE)
            assert np.array_equal(tidx[b, h], ri) and np.array_equal(tval[b, h].view(np.uint32), rv.view(np.uint32))
            assert ucnt[b, h] == len(ru) and np.array_equal(uidx[b, h, :len(ru)], ru), "union differs (b=%d h=%d)" % (b, h)
            assert (np.abs(out[b, h * G:(h + 1) * G] - ro) < out_tol(ro, False)).all()


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_short_token_list_bf16_weights(seed):
    """A step that attends to 17 tokens only (top 1 + a window of 16), bf16 inputs, grouped queries on the matrix cores,
    fp16 output: with so few terms nothing averages out, so the softmax weights must reach the P.V product with more than
    the 8 bits of a bf16 operand (they go in as a high and a low part).  Half the 2e-3 tolerance."""
    from topk_attn_amd import ops
    announce("sparse_decode_step bf16 G=8, 17 tokens, seed %d" % seed)
    rng = np.random.default_rng(900 + seed)
    dtype, B, H, G, N, k, sink, local = oracle.BF16, 2, 2, 8, 6000, 1, 0, 16
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)
    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink,
                                                         local, SCALE, G, out_dtype=torch.float16, want_topk=False)
    torch.cuda.synchronize()
    out = f32_of(out)
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(q[b, h * G:(h + 1) * G], K[b, :, h], V[b, :, h], dtype, G, k, sink,
                                                       local, SCALE)
            assert np.abs(out[b, h * G:(h + 1) * G] - ro).max() < 1e-3


@pytest.mark.parametrize("layout", ["padded_heads", "head_major"])
@pytest.mark.parametrize("N,k", [(9000, 1024), (70000, 2048)])
def test_sparse_decode_step_cache_layouts(layout, N, k):
    """K and V caches that are views (unused heads on either side of the ones in use; head-major storage): the step
    must give what it gives on contiguous copies — selection bit for bit, attention within tolerance."""
    from topk_attn_amd import ops
    announce("sparse_decode_step cache layout %s N=%d k=%d" % (layout, N, k))
    rng = np.random.default_rng(N + k + 7)
    dtype, B, H, G, sink, local = oracle.F16, 1, 2, 4, 16, 128
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)

    def view(x):
        if layout == "padded_heads":
            full = randn_bits(rng, (B, N, H + 2, 128), dtype)
            full[:, :, 1:1 + H] = x
            return to_dev(full, dtype)[:, :, 1:1 + H]
        return to_dev(np.ascontiguousarray(x.transpose(0, 2, 1, 3)), dtype).permute(0, 2, 1, 3)

    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(to_dev(q, dtype), view(K), view(V), k, sink, local, SCALE, G,
                                                         out_dtype=torch.float16, want_topk=False)
    torch.cuda.synchronize()
    out, uidx, ucnt = f32_of(out), uidx.cpu().numpy(), ucnt.cpu().numpy()
    for h in range(H):
        ro, ri, rv, ru = oracle.sparse_decode_step(q[0, h * G:(h + 1) * G], K[0, :, h], V[0, :, h], dtype, G, k, sink, local, SCALE)
        assert ucnt[0, h] == len(ru) and np.array_equal(uidx[0, h, :len(ru)], ru), "union differs (h=%d)" % h
        assert (np.abs(out[0, h * G:(h + 1) * G] - ro) < out_tol(ro, False)).all()


@pytest.fixture
def hooks():
    """Testing hooks of the candidate route, restored to their defaults afterwards."""
    from topk_attn_amd import ops
    yield ops.set_test_hooks
    ops.set_test_hooks()


@pytest.mark.parametrize("dtype,B,H,G,N,k,sink,local,kind,want_topk,cut", [
    (oracle.F16, 1, 1, 8, 32768, 2048, 64, 512, "heavy", False, True),
    (oracle.F16, 1, 1, 8, 32768, 2048, 64, 512, "heavy", True, True),
    (oracle.BF16, 1, 2, 4, 30000, 1000, 16, 128, "levels", True, True),       # large tie buckets: slices beyond their head entries
    (oracle.F16, 1, 1, 2, 17000, 1024, 8, 8, "equal", False, True),            # every token ties
    (oracle.F16, 2, 2, 4, 20000, 1200, 64, 512, "heavy", False, True),
    (oracle.F16, 1, 1, 1, 65536, 2048, 0, 0, "heavy", False, True),            # no sink range, no window
    (oracle.F16, 1, 1, 4, 24000, 1400, 6000, 22000, "heavy", True, True),      # range and window overlap: nothing in between
    (oracle.BF16, 3, 1, 4, 20000, 1200, 1, 19990, "levels", False, True),      # the window covers nearly everything
    (oracle.F16, 1, 8, 4, 32768, 2048, 64, 512, "heavy", False, True),         # more than 65536 rows: the route in three launches
    (oracle.BF16, 2, 4, 2, 20001, 1000, 100, 300, "levels", True, True),
    (oracle.F16, 1, 2, 4, 24577, 3000, 300, 300, "heavy", False, False),       # k too large for that route: the dense path, ascending list
    (oracle.F16, 2, 2, 4, 16384, 1024, 64, 512, "heavy", False, True),         # would also fit the registers of a workgroup
    (oracle.F16, 1, 8, 4, 12000, 1024, 64, 512, "heavy", False, True),         # the same on a call of more than 65536 rows
    (oracle.BF16, 3, 8, 2, 28000, 1500, 64, 512, "heavy", False, True),        # more than 655360 rows
    (oracle.F16, 2, 2, 4, 8000, 512, 64, 512, "heavy", False, False),          # short enough for the registers of a workgroup
    (oracle.BF16, 1, 3, 2, 5000, 700, 3000, 3000, "levels", True, False),      # the same with range and window overlapping, ties
    (oracle.F16, 1, 2, 8, 3000, 100, 5, 9, "equal", False, False)])
def test_sparse_decode_step_handoff_order(hooks, dtype, B, H, G, N, k, sink, local, kind, want_topk, cut):
    """A step that is not asked for its union list hands the tokens to the attention in the order of its route: for a few
    segments of 8193 .. 65536 tokens the ranking workgroups of the common-cut route write the middle part themselves, part
    in rank order behind the sink range and the local window, with -1 in the place of a selected token that lies inside the
    ranges (the attention skips such ids).  The union_handoff_order hook makes that list visible: without the -1 it must be
    the oracle's as a set, and the oracle's top-k in rank order behind the ranges; -1 behind the count; rank-ordered top-k
    output (when asked for) bit for bit; attention within tolerance."""
    from topk_attn_amd import ops
    announce("sparse_decode_step hand-off order dtype=%d B=%d H=%d G=%d N=%d k=%d sink=%d local=%d %s" % (dtype, B, H, G, N, k, sink, local, kind))
    hooks(union_handoff_order=1)
    rng = np.random.default_rng(N + 3 * k + sink)
    if kind == "levels":
        Kf = np.linspace(-2, 2, 16)[rng.integers(0, 16, (B, N, H, 128))]
    elif kind == "equal":
        Kf = np.broadcast_to(rng.standard_normal((1, 1, 1, 128)), (B, N, H, 128)).copy()
    else:
        Kf = rng.standard_normal((B, N, H, 128))
        Kf[:, rng.permutation(N)[:max(1, N // 100)]] *= 4.0
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), oracle.to_bits(Kf, dtype), randn_bits(rng, (B, N, H, 128), dtype)
    plan = ops.SparseDecodePlan(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink, local, SCALE, G,
                                out_dtype=torch.float16, want_topk=want_topk)
    ops.profile_reset()
    ops.profile_enable(True)
    plan.step()
    torch.cuda.synchronize()
    kernels = ops.profile_read()
    ops.profile_enable(False)
    if cut:
        assert ("gemv_cut" in kernels or "gemv_cut_slices" in kernels) and "select_rank" in kernels, "not the common-cut route: %s" % sorted(kernels)
        assert plan.redone_segments() == 0
    out, uidx, ucnt = f32_of(plan.out), plan.union_idx.cpu().numpy(), plan.union_count.cpu().numpy()
    lo = min(sink, N)
    hi = max(N - local, lo)
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(q[b, h * G:(h + 1) * G], K[b, :, h], V[b, :, h], dtype, G, k, sink,
                                                       local, SCALE)
            got, cnt = uidx[b, h], int(ucnt[b, h])
            listed = got[:cnt]
            assert np.array_equal(np.sort(listed[listed >= 0]), ru), "union differs as a set (b=%d h=%d)" % (b, h)
            assert (got[cnt:] == -1).all()
            if cut or "select_wave" in kernels:
                # these routes: the two ranges, then a place per selected token (-1 where it lies inside the ranges)
                assert cnt == lo + (N - hi) + k
                assert np.array_equal(got[:lo], np.arange(lo)) and np.array_equal(got[lo:lo + N - hi], np.arange(hi, N))
                if cut:   # here the places are the ranks
                    mid = ri[(ri >= lo) & (ri < hi)]
                    assert np.array_equal(listed[lo + N - hi:][listed[lo + N - hi:] >= 0], mid), "rank order of the listed tokens"
            else:
                assert cnt == len(ru)
            if want_topk:
                assert np.array_equal(plan.topk_idx[b, h].cpu().numpy(), ri), "top-k indices differ"
                assert np.array_equal(plan.topk_val[b, h].cpu().numpy().view(np.uint32), rv.view(np.uint32))
            assert (np.abs(out[b, h * G:(h + 1) * G] - ro) < out_tol(ro, False)).all()


def test_sparse_decode_step_handoff_order_forced_redo(hooks):
    """The same hand-off when the ranking kernel redoes its segments from the keys (then the list comes ascending)."""
    from topk_attn_amd import ops
    announce("sparse_decode_step hand-off order, segments redone from the keys (N=20000 k=1200 G=4)")
    hooks(union_handoff_order=1, force_segment_redo=1)
    rng = np.random.default_rng(61)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 1, 2, 4, 20000, 1200, 32, 100
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype), randn_bits(rng, (B, N, H, 128), dtype)
    plan = ops.SparseDecodePlan(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink, local, SCALE, G,
                                out_dtype=torch.float16, want_topk=False)
    plan.step()
    torch.cuda.synchronize()
    assert plan.redone_segments() == 2
    out, uidx, ucnt = f32_of(plan.out), plan.union_idx.cpu().numpy(), plan.union_count.cpu().numpy()
    for h in range(H):
        ro, ri, rv, ru = oracle.sparse_decode_step(q[0, h * G:(h + 1) * G], K[0, :, h], V[0, :, h], dtype, G, k, sink, local, SCALE)
        assert ucnt[0, h] == len(ru) and np.array_equal(uidx[0, h, :len(ru)], ru), "union differs (h=%d)" % h
        assert (np.abs(out[0, h * G:(h + 1) * G] - ro) < out_tol(ro, False)).all()


def test_sparse_decode_step_forced_redo(hooks):
    """Union mode of the path that redoes a segment from the keys (force_segment_redo hook), 16-level keys."""
    hooks(force_segment_redo=1)
    test_sparse_decode_step_union_only(oracle.BF16, 1, 2, 4, 66001, 1500, 32, 100, "levels")


@pytest.mark.parametrize("kind,N,k,sink,local", [("equal", 70000, 1500, 32, 100), ("levels", 140000, 2048, 64, 512),
                                                 ("heavy", 80000, 2048, 30000, 60000), ("heavy", 70001, 1000, 0, 0)])
def test_sparse_decode_step_redo_launch_union(hooks, kind, N, k, sink, local):
    """Union mode of the launch that redoes flagged long segments: one score for all tokens (a bucket beyond the LDS, cut
    by rank in index order), 16-level keys (ties inside the bucket), a sink range and a local window that overlap (nothing
    between them), and neither of the two."""
    hooks(force_segment_redo=1)
    test_sparse_decode_step_union_only(oracle.F16, 1, 2, 4, N, k, sink, local, kind)


@pytest.mark.parametrize("N,k", [(70001, 1500), (140000, 4096)])
def test_sparse_decode_step_redo_launch_all_outputs(hooks, N, k):
    """The step that returns everything - rank-ordered top-k, ascending union list, attention output - on long segments
    with every segment redone by the launch behind the selection (its form that sorts the selection at the end); and
    without the hook, from the candidates."""
    for forced in (1, 0):
        hooks(force_segment_redo=forced)
        test_sparse_decode_step(oracle.F16, torch.float16, 1, 2, 4, N, k, 64, 512)


def test_sparse_decode_step_list_behind_forced_redo(hooks):
    """A caller that asks for the ascending list on segments that the common-cut route takes (the list for the attention stays
    in the workspace, the caller's list is made from the rank-ordered ids by one more launch), with every segment redone from
    the keys by its first ranking workgroup; and the same with the cuts of every other segment never announced."""
    hooks(force_segment_redo=1)
    test_sparse_decode_step_union_only(oracle.F16, 1, 2, 4, 30001, 1500, 32, 100, "levels")
    hooks(tau_spin_limit=64, tau_withhold_mod=2, tau_withhold_rem=1, tau_withhold_mode=0)
    test_sparse_decode_step_union_only(oracle.F16, 1, 8, 2, 20000, 1000, 64, 512, "heavy")


def test_sparse_decode_step_threshold_never_published(hooks):
    """Union mode when the streaming workgroups of one segment run out of their wait for the threshold: that segment
    is redone from the keys, the other keeps the candidate route, union lists and outputs as the oracle's."""
    from topk_attn_amd import ops
    announce("sparse_decode_step, threshold of segment 0 withheld for good (N=70000 k=1024 G=4)")
    hooks(tau_spin_limit=64, tau_withhold_mod=2, tau_withhold_rem=0, tau_withhold_mode=0)
    rng = np.random.default_rng(78)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 1, 2, 4, 70000, 1024, 16, 128
    Kf = rng.standard_normal((B, N, H, 128))
    Kf[:, rng.permutation(N)[:N // 100]] *= 4.0
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), oracle.to_bits(Kf, dtype), randn_bits(rng, (B, N, H, 128), dtype)
    plan = ops.SparseDecodePlan(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, sink, local, SCALE, G,
                                out_dtype=torch.float16, want_topk=False)
    plan.step()
    torch.cuda.synchronize()
    assert plan.redone_segments() == 1
    out, uidx, ucnt = f32_of(plan.out), plan.union_idx.cpu().numpy(), plan.union_count.cpu().numpy()
    for h in range(H):
        ro, ri, rv, ru = oracle.sparse_decode_step(q[0, h * G:(h + 1) * G], K[0, :, h], V[0, :, h], dtype, G, k, sink, local, SCALE)
        assert ucnt[0, h] == len(ru) and np.array_equal(uidx[0, h, :len(ru)], ru), "union differs (h=%d)" % h
        assert (np.abs(out[0, h * G:(h + 1) * G] - ro) < out_tol(ro, False)).all()


def test_sparse_decode_step_graph_replay():
    """The step captured in a HIP graph and replayed with a new query each time (long segments: the sampled
    thresholds and arrival flags of one replay must never serve the next).  Every replay is compared with the
    eager result for the same query, with eager work in between."""
    from topk_attn_amd import ops
    announce("sparse_decode_step captured in a graph, 3 replays with changing queries (N=70000 k=1024 G=4)")
    rng = np.random.default_rng(77)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 1, 2, 4, 70000, 1024, 16, 128
    Kf = rng.standard_normal((B, N, H, 128))
    Kf[:, rng.permutation(N)[:N // 100]] *= 4.0
    q = to_dev(randn_bits(rng, (B, H * G, 128), dtype), dtype)
    K, V = to_dev(oracle.to_bits(Kf, dtype), dtype), to_dev(randn_bits(rng, (B, N, H, 128), dtype), dtype)
    plan = ops.SparseDecodePlan(q, K, V, k, sink, local, SCALE, G, out_dtype=torch.float16, want_topk=False)
    plan.step()                      # warm-up outside the capture (one-time function attributes)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        plan.step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plan.step()
    torch.cuda.synchronize()
    for it in range(3):
        q.copy_(to_dev(oracle.to_bits(rng.standard_normal((B, H * G, 128)) * (1.0 + 0.5 * it), dtype), dtype))
        plan.step()                  # eager, default stream
        torch.cuda.synchronize()
        want_out, want_idx, want_cnt = plan.out.clone(), plan.union_idx.clone(), plan.union_count.clone()
        plan.out.zero_()
        plan.union_idx.fill_(-7)
        plan.union_count.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(plan.union_count, want_cnt), "replay %d: union counts differ" % it
        assert torch.equal(plan.union_idx, want_idx), "replay %d: union lists differ" % it
        assert torch.equal(plan.out, want_out), "replay %d: outputs differ" % it


def test_sparse_decode_step_graph_replay_cuts_announced_in_the_launch(hooks):
    """The same for a step whose GEMV launch finds the cuts of its segments in its first workgroups and announces them
    to the others (4 x 32768 tokens, output only): a replay brings the same epoch, so the word of one replay must be
    spent before the next.  Top-k and hand-off list (made visible by the hook) bit for bit, output bit for bit, and no
    segment redone."""
    from topk_attn_amd import ops
    announce("sparse_decode_step captured in a graph, 3 replays, cuts announced inside the GEMV launch (4 x 32768, k=2048)")
    hooks(union_handoff_order=1)
    rng = np.random.default_rng(79)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 1, 4, 4, 32768, 2048, 64, 512
    q = to_dev(randn_bits(rng, (B, H * G, 128), dtype), dtype)
    K, V = to_dev(randn_bits(rng, (B, N, H, 128), dtype), dtype), to_dev(randn_bits(rng, (B, N, H, 128), dtype), dtype)
    plan = ops.SparseDecodePlan(q, K, V, k, sink, local, SCALE, G, out_dtype=torch.float16, want_topk=True)
    ops.profile_reset()
    ops.profile_enable(True)
    plan.step()                      # warm-up outside the capture
    torch.cuda.synchronize()
    kernels = ops.profile_read()
    ops.profile_enable(False)
    assert "gemv_cut_slices" in kernels and "cut_sample" not in kernels, sorted(kernels)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        plan.step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plan.step()
    torch.cuda.synchronize()
    for it in range(3):
        q.copy_(to_dev(oracle.to_bits(rng.standard_normal((B, H * G, 128)) * (1.0 + 0.5 * it), dtype), dtype))
        plan.step()                  # eager, default stream
        torch.cuda.synchronize()
        assert plan.redone_segments() == 0
        want = [t.clone() for t in (plan.out, plan.union_idx, plan.union_count, plan.topk_idx, plan.topk_val)]
        plan.out.zero_()
        plan.union_idx.fill_(-7)
        plan.union_count.zero_()
        plan.topk_idx.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert plan.redone_segments() == 0, "replay %d: a segment was redone from the keys" % it
        for got, ref, what in zip((plan.out, plan.union_idx, plan.union_count, plan.topk_idx, plan.topk_val), want,
                                  ("outputs", "hand-off lists", "list counts", "top-k indices", "top-k values")):
            assert torch.equal(got, ref), "replay %d: %s differ" % (it, what)


def test_retrieval_attention_graph_replay():
    """The operator captured in a HIP graph (the batch path: shared-key scoring, small-workgroup selection,
    attention that writes the result itself) and replayed with new queries; every replay is compared with the
    eager result for the same query, with eager work in between."""
    from topk_attn_amd import retrieval_attention_cpp as ra
    announce("retrieval_attention_128 captured in a graph, 3 replays with changing queries (B=6)")
    rng = np.random.default_rng(78)
    dtype, B = oracle.F16, 6
    q = to_dev(randn_bits(rng, (B, 32, 128), dtype, 0.1), dtype)
    K, V = to_dev(randn_bits(rng, (8192, 32, 128), dtype, 0.1), dtype), to_dev(randn_bits(rng, (8192, 32, 128), dtype, 0.1), dtype)
    out = torch.zeros((B, 32, 128), dtype=torch.float16, device="cuda")
    ra.retrieval_attention_128(q, K, V, out)     # warm-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        ra.retrieval_attention_128(q, K, V, out)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            ra.retrieval_attention_128(q, K, V, out)
    torch.cuda.synchronize()
    for it in range(3):
        q.copy_(to_dev(randn_bits(rng, (B, 32, 128), dtype, 0.1 * (1 + it)), dtype))
        ra.retrieval_attention_128(q, K, V, out)
        torch.cuda.synchronize()
        want = out.clone()
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), "replay %d: outputs differ" % it
    ref, _, _ = oracle.retrieval_attention(bits_of(q)[B - 1, 3], bits_of(K)[:, 3], bits_of(V)[:, 3], dtype, 4, 128, 1.0)
    assert np.abs(f32_of(out)[B - 1, 3] - ref).max() < TOL
