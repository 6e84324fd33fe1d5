"""Fused GEMV + top-k: fp32 scores bit-identical to the oracle's canonical order (and within 1e-5 of the
fp64 dot), selected indices bit-identical, for the flat, chunked, grouped, centre-only and two-level forms."""
import numpy as np
import pytest
import torch

import oracle
from tests.util import announce, randn_bits, to_dev

pytestmark = pytest.mark.gpu

SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


def _run_flat(dtype, B, H, G, N, k, seed, shared_kv=False, num_chunks=1, scale=SCALE, levels=False):
    from topk_attn_amd import ops
    rng = np.random.default_rng(seed)
    q = randn_bits(rng, (B, H * G, 128), dtype)
    kshape = (N, H, 128) if shared_kv else (B, N, H, 128)
    if levels:
        lv = np.linspace(-2, 2, 16)
        K = oracle.to_bits(lv[rng.integers(0, 16, kshape)], dtype)
    else:
        K = randn_bits(rng, kshape, dtype)
    idx, val, scores = ops.gemv_topk(to_dev(q, dtype), to_dev(K, dtype), k, group=G, scale=scale,
                                     num_chunks=num_chunks, return_scores=True)
    torch.cuda.synchronize()
    idx, val, scores = idx.cpu().numpy(), val.cpu().numpy(), scores.cpu().numpy()
    chunk = N // num_chunks
    for b in range(B):
        for h in range(H):
            Kh = K[:, h, :] if shared_kv else K[b, :, h, :]
            qf = oracle.group_query(q[b, h * G:(h + 1) * G], dtype, G)
            ref = oracle.scores_canonical(Kh, dtype, qf, scale)
            assert np.array_equal(scores[b, h].view(np.uint32), ref.view(np.uint32)), "scores differ (b=%d h=%d)" % (b, h)
            truth = oracle.scores_f64(Kh, dtype, q[b, h * G:(h + 1) * G], scale)
            assert np.abs(ref.astype(np.float64) - truth).max() < 1e-5 * max(1.0, np.abs(truth).max() / 4)
            for c in range(num_chunks):
                ei, ev = oracle.topk_stable(ref[c * chunk:(c + 1) * chunk], k)
                got = idx[b, h, c * k:(c + 1) * k]
                assert np.array_equal(got, ei + c * chunk), "indices differ (b=%d h=%d c=%d)" % (b, h, c)
                assert np.array_equal(val[b, h, c * k:(c + 1) * k].view(np.uint32), ev.view(np.uint32))


def test_config1_single_head():
    """q fp16 [128], K fp16 [32768,128] N(0,1), scores K.q/sqrt(128), top-2048."""
    announce("gemv_topk config 1: N=32768 k=2048 fp16")
    _run_flat(oracle.F16, 1, 1, 1, 32768, 2048, seed=1)


@pytest.mark.parametrize("dtype", [oracle.F16, oracle.BF16])
def test_small_shapes(dtype):
    announce("gemv_topk small shapes dtype=%d" % dtype)
    _run_flat(dtype, 2, 3, 1, 1000, 100, seed=2)
    _run_flat(dtype, 1, 2, 4, 4099, 257, seed=3)
    _run_flat(dtype, 1, 1, 8, 130, 130, seed=4)


def test_whole_segment_routes_edges():
    """Segments that one workgroup scores itself (up to 2048 rows) or that fit in LDS whole (up to 16384): k = n,
    k = 1, the largest k, odd lengths, chunks, both dtypes."""
    announce("gemv_topk whole-segment routes: edge shapes")
    _run_flat(oracle.BF16, 1, 1, 8, 2048, 2048, seed=40)            # k = n, sorted whole
    _run_flat(oracle.F16, 2, 2, 1, 2047, 1, seed=41)                # k = 1
    _run_flat(oracle.F16, 1, 2, 2, 16384, 8192, seed=42)            # largest segment and k of the LDS route
    _run_flat(oracle.BF16, 1, 3, 4, 6000, 1500, seed=43, num_chunks=3, levels=True)   # chunks of 2000, ties
    _run_flat(oracle.F16, 1, 1, 1, 2049, 700, seed=44)              # first length past the one-launch route


def test_grouped_batched():
    announce("gemv_topk B=2 Hkv=8 G=4 N=16384 k=2048 fp16")
    _run_flat(oracle.F16, 2, 8, 4, 16384, 2048, seed=5)


def test_shared_kv_chunked():
    """The reference op's stage 1: 4 chunks of 2048 keys, top-K per chunk, no scale, KV shared by the batch."""
    announce("gemv_topk chunked N=8192 chunks=4 k=128 shared KV")
    _run_flat(oracle.F16, 2, 4, 1, 8192, 128, seed=6, shared_kv=True, num_chunks=4, scale=1.0)


@pytest.mark.parametrize("B,H", [(2, 32), (3, 22), (5, 13), (8, 8), (9, 8), (17, 4)])
def test_shared_kv_batch_tiles(B, H):
    """Keys shared by the batch are scored for several batch entries per pass (tiles of 2, 4 or 8 entries, with
    a ragged last tile) and the 128 or more short segments are selected by a small workgroup each."""
    announce("gemv_topk shared KV batch tiles B=%d H=%d N=8192 chunks=4 k=128" % (B, H))
    _run_flat(oracle.F16, B, H, 1, 8192, 128, seed=60 + B, shared_kv=True, num_chunks=4, scale=1.0)


@pytest.mark.parametrize("dtype,B,H,N,chunks,k", [(oracle.F16, 2, 3, 4096, 2, 128), (oracle.F16, 17, 2, 4100, 1, 300),
                                                  (oracle.BF16, 32, 2, 8192, 4, 128), (oracle.F16, 33, 1, 4099, 1, 64),
                                                  (oracle.BF16, 9, 4, 2048, 1, 2048)])
def test_matrix_core_scores_shared_kv(dtype, B, H, N, chunks, k):
    """score_mode = TKA_SCORE_MATRIX on a key cache shared by the batch: the scores come from the matrix cores, whose
    order of addition is not the canonical one, so they are held to 1e-5 of the exact dot product (the stated rule
    for fp32 scores), and the selection must be exact ON THOSE SCORES: indices and values are the first k of a
    stable descending sort of the score vector the call returned, chunk by chunk."""
    from topk_attn_amd import _lib as L
    from topk_attn_amd import ops
    announce("gemv_topk on the matrix cores dtype=%d B=%d H=%d N=%d chunks=%d k=%d" % (dtype, B, H, N, chunks, k))
    rng = np.random.default_rng(1000 + B)
    q, K = randn_bits(rng, (B, H, 128), dtype), randn_bits(rng, (N, H, 128), dtype)
    idx, val, scores = ops.gemv_topk(to_dev(q, dtype), to_dev(K, dtype), k, group=1, scale=SCALE, num_chunks=chunks,
                                     return_scores=True, score_mode=L.TKA_SCORE_MATRIX)
    plain = ops.gemv_scores(to_dev(q, dtype), to_dev(K, dtype), group=1, scale=SCALE, score_mode=L.TKA_SCORE_MATRIX)
    torch.cuda.synchronize()
    idx, val, scores, plain = idx.cpu().numpy(), val.cpu().numpy(), scores.cpu().numpy(), plain.cpu().numpy()
    assert np.array_equal(scores.view(np.uint32), plain.view(np.uint32))      # the GEMV-only entry point runs the same kernel
    chunk = N // chunks
    differs = 0
    for b in range(B):
        for h in range(H):
            truth = oracle.scores_f64(K[:, h, :], dtype, q[b, h:h + 1], SCALE)
            assert np.abs(scores[b, h].astype(np.float64) - truth).max() < 1e-5 * max(1.0, np.abs(truth).max() / 4)
            canon = oracle.scores_canonical(K[:, h, :], dtype, oracle.group_query(q[b, h:h + 1], dtype, 1), SCALE)
            differs += int((canon.view(np.uint32) != scores[b, h].view(np.uint32)).sum())
            for c in range(chunks):
                ei, ev = oracle.topk_stable(scores[b, h, c * chunk:(c + 1) * chunk], k)   # (pinned against lexsort / stable sort)
                assert np.array_equal(idx[b, h, c * k:(c + 1) * k], ei + c * chunk), "indices differ (b=%d h=%d c=%d)" % (b, h, c)
                assert np.array_equal(val[b, h, c * k:(c + 1) * k].view(np.uint32), ev.view(np.uint32))
    print("matrix-core scores that differ from the canonical ones in their last bits: %d of %d" % (differs, B * H * N), flush=True)


def test_many_short_segments_routes():
    """128 or more segments of at most 2048 rows: plain scores + a small workgroup per segment; both dtypes, grouped
    queries, odd lengths, ties, keys per sequence and shared."""
    announce("gemv_topk many short segments")
    _run_flat(oracle.BF16, 8, 8, 2, 8000, 500, seed=70, num_chunks=4)                      # per-sequence keys
    _run_flat(oracle.BF16, 6, 11, 4, 4000, 1000, seed=71, shared_kv=True, num_chunks=4, levels=True)   # ties, k = n
    _run_flat(oracle.F16, 16, 16, 1, 1999, 1024, seed=72, shared_kv=True)                  # odd length, largest k
    _run_flat(oracle.F16, 8, 32, 1, 300, 7, seed=73, shared_kv=True)                       # tiny segments
    _run_flat(oracle.F16, 3, 2, 1, 12000, 300, seed=74, shared_kv=True)                    # shared keys, one workgroup per segment


def test_tie_stress_bf16_levels():
    """K quantised to 16 levels: many exact score ties; indices must still match bit for bit."""
    announce("gemv_topk tie stress bf16 N=65536 G=8 k=4096")
    _run_flat(oracle.BF16, 1, 2, 8, 65536, 4096, seed=7, levels=True)


def test_unit_query_reproduces_column():
    """q = e_i makes the score K[:, i] * scale exactly — a check that does not go through the oracle."""
    from topk_attn_amd import ops
    announce("gemv_scores unit query")
    rng = np.random.default_rng(8)
    K = randn_bits(rng, (3000, 2, 128), oracle.F16)
    for i in (0, 7, 64, 127):
        qv = np.zeros((1, 2, 128))
        qv[0, :, i] = 1.0
        s = ops.gemv_scores(to_dev(oracle.to_bits(qv, oracle.F16), oracle.F16), to_dev(K, oracle.F16), scale=0.5)
        torch.cuda.synchronize()
        want = oracle.from_bits(K[:, :, i], oracle.F16).T * np.float32(0.5)
        assert np.array_equal(s[0].cpu().numpy(), want)


def test_center_only_config2_shape():
    """32 heads x 4096 centroids with a per-head mean shift, top-64, expand x64 -> 4096 token ids per head."""
    from topk_attn_amd import ops
    announce("center_topk_expand config 2")
    rng = np.random.default_rng(2)
    H, Cn, top_c, clen = 32, 4096, 64, 64
    cen = rng.standard_normal((H, Cn, 128)) + 0.5 * rng.standard_normal((H, 1, 128))
    cen_b = oracle.to_bits(cen, oracle.F16)
    q_b = randn_bits(rng, (H, 128), oracle.F16)
    out, cids, cval = ops.center_topk_expand(to_dev(q_b, oracle.F16), to_dev(cen_b, oracle.F16), top_c, clen, SCALE)
    torch.cuda.synchronize()
    out, cids, cval = out.cpu().numpy(), cids.cpu().numpy(), cval.cpu().numpy()
    for h in range(H):
        eo, ec, ev = oracle.center_topk_expand(q_b[h], cen_b[h], oracle.F16, top_c, clen, SCALE)
        assert np.array_equal(cids[h], ec) and np.array_equal(out[h], eo)
        assert np.array_equal(cval[h].view(np.uint32), ev.view(np.uint32))
        # closed form of the expansion, independent of the oracle
        assert np.array_equal(out[h].reshape(top_c, clen), cids[h][:, None] * clen + np.arange(clen)[None])


@pytest.mark.parametrize("H,tied_centres", [(4, False), (32, False), (32, True)])
def test_two_level_cluster_reference_shape(H, tied_centres):
    """Reference constants of gemv_topk.cu:21-28: 32 centroids, clusters of 1280 tokens, top-5 clusters, top-512
    inside each.  With all 32 heads (160 segments) the centre stage runs inside the GEMV launch of the token stage;
    with 4 heads it is a launch of its own.  tied_centres: three identical centroids per head, aligned with the
    query so that they take ranks 0-2: equal scores, the lower centroid id must come first."""
    from topk_attn_amd import ops
    announce("cluster_gemv_topk CSZ=32 CLEN=1280 TOPC=5 k=512 H=%d tied_centres=%s" % (H, tied_centres))
    rng = np.random.default_rng(12345)
    CSZ, CLEN, TOPC, K = 32, 1280, 5, 512
    cen = rng.uniform(-0.5, 0.5, (H, CSZ, 128))
    qf = rng.uniform(-0.5, 0.5, (H, 128))
    if tied_centres:
        cen[:, [20, 3, 7]] = 0.9 * qf[:, None, :]
    keys = cen.transpose(1, 0, 2)[:, None, :, :] + 0.05 * rng.standard_normal((CSZ, CLEN, H, 128))
    keys = keys.reshape(CSZ * CLEN, H, 128)
    cen_b, keys_b = oracle.to_bits(cen, oracle.F16), oracle.to_bits(keys, oracle.F16)
    q_b = oracle.to_bits(qf, oracle.F16)
    out = ops.cluster_gemv_topk(to_dev(q_b, oracle.F16), to_dev(cen_b, oracle.F16), to_dev(keys_b, oracle.F16),
                                TOPC, CLEN, K, 1.0)
    torch.cuda.synchronize()
    out = out.cpu().numpy()
    for h in range(H):
        want = oracle.cluster_topk(q_b[h], cen_b[h], keys_b[:, h, :], oracle.F16, TOPC, CLEN, K, 1.0)
        assert np.array_equal(out[h], want)
        if tied_centres:
            assert [int(want[r * K]) // CLEN for r in range(3)] == [3, 7, 20]
        # the reference's own check (gemv_topk.cu:138-170): set equality per (head, rank) slice
        for r in range(TOPC):
            assert set(out[h, r * K:(r + 1) * K]) == set(want[r * K:(r + 1) * K])


# ---- long segments: sampled threshold + candidate slices; a segment they fail is redone from the keys ----

def _mix32(x):
    x &= 0xFFFFFFFF
    x ^= x >> 16; x = (x * 0x7feb352d) & 0xFFFFFFFF
    x ^= x >> 15; x = (x * 0x846ca68b) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def _sampled_positions(seg, n, samples=2048):
    """Token positions the threshold estimate of a long segment looks at: one per stride of n/samples tokens, at a
    hashed offset inside the stride (2048 samples for segments below 512K tokens)."""
    stride = n // samples
    return [i * stride + ((_mix32((seg * 0x9e3779b9 + i) & 0xFFFFFFFF) * stride) >> 32) for i in range(samples)]


def _check_long(K, q, dtype, G, k, scale=SCALE, redone=None, gave_up=None):
    """`redone`: how many segments the selection kernel is expected to redo from the keys (None: not checked);
    `gave_up`: how many candidate slices are expected to come from workgroups whose wait for the threshold ran out."""
    from topk_attn_amd import ops
    plan = ops.GemvTopkPlan(to_dev(q, dtype), to_dev(K, dtype), k, group=G, scale=scale).run()
    torch.cuda.synchronize()
    if redone is not None:
        assert plan.redone_segments() == redone
    if gave_up is not None:
        assert plan.gave_up_slices() == gave_up
    idx, val = plan.idx.cpu().numpy(), plan.val.cpu().numpy()
    B, N, H = K.shape[:3]
    for b in range(B):
        for h in range(H):
            ref = oracle.scores_canonical(K[b, :, h, :], dtype, oracle.group_query(q[b, h * G:(h + 1) * G], dtype, G), scale)
            ei, ev = oracle.topk_stable(ref, k)
            assert np.array_equal(idx[b, h], ei), "indices differ (b=%d h=%d)" % (b, h)
            assert np.array_equal(val[b, h].view(np.uint32), ev.view(np.uint32))


def test_long_segment_candidates():
    announce("gemv_topk long segment N=131072 k=2048 G=4 (candidate lists)")
    rng = np.random.default_rng(31)
    K = randn_bits(rng, (1, 131072, 2, 128), oracle.F16)
    K[0, rng.permutation(131072)[:1300]] = oracle.to_bits(rng.standard_normal((1300, 2, 128)) * 4.0, oracle.F16)
    _check_long(K, randn_bits(rng, (1, 8, 128), oracle.F16), oracle.F16, 4, 2048, redone=0)


def test_mid_segments_large_call_candidates():
    """Segments between 32768 and 65536 tokens take the sampled-threshold path when the call is large (a million
    rows): 4 x 8 segments of 40000 tokens, ragged slices, none redone."""
    announce("gemv_topk mid segments B=4 H=8 N=40000 k=1500 (candidate lists)")
    rng = np.random.default_rng(41)
    K = randn_bits(rng, (4, 40000, 8, 128), oracle.F16)
    _check_long(K, randn_bits(rng, (4, 8, 128), oracle.F16), oracle.F16, 1, 1500, redone=0)


def test_long_segment_all_equal():
    """Every key equal: the sampled threshold is a (key, token) pair, so only the first tokens pass."""
    announce("gemv_topk long segment all keys equal")
    rng = np.random.default_rng(32)
    K = np.broadcast_to(randn_bits(rng, (1, 1, 1, 128), oracle.BF16), (1, 70001, 2, 128)).copy()
    _check_long(K, randn_bits(rng, (1, 2, 128), oracle.BF16), oracle.BF16, 1, 1000, redone=0)


def test_long_segment_sample_hits_only_heavy_tokens_falls_back():
    """Heavy tokens placed exactly where the threshold estimate samples: the threshold lands among them, fewer than
    k tokens pass, and the segment is redone from the keys.  One head is adversarial, the other ordinary."""
    announce("gemv_topk long segment adversarial sample (fallback: too few candidates)")
    rng = np.random.default_rng(33)
    N, k, dtype = 131072, 4096, oracle.F16
    Kf = rng.standard_normal((1, N, 2, 128)) * 0.05
    qf = rng.standard_normal((1, 2, 128))
    pos = _sampled_positions(0, N)                       # segment 0 = (batch 0, head 0)
    Kf[0, pos, 0, :] = qf[0, 0] * rng.uniform(0.5, 1.5, (len(pos), 1))   # large positive scores, all distinct
    _check_long(oracle.to_bits(Kf, dtype), oracle.to_bits(qf, dtype), dtype, 1, k, redone=1)


def test_long_segment_bf16_levels_group8():
    announce("gemv_topk long segment bf16 16-level keys N=262144 k=4096 G=8")
    rng = np.random.default_rng(34)
    K = oracle.to_bits(np.linspace(-2, 2, 16)[rng.integers(0, 16, (1, 262144, 1, 128))], oracle.BF16)
    _check_long(K, randn_bits(rng, (1, 8, 128), oracle.BF16), oracle.BF16, 8, 4096)


@pytest.mark.parametrize("layout", ["spread", "tail", "head", "two_buckets"])
def test_long_segment_heavy_ties(layout):
    """Scores that take three values on a long segment, with the k-th largest inside a bucket of tens of
    thousands of equal scores (a unit query makes the score one key column): the sampled threshold must cut the
    bucket by token, wherever its tokens sit, and the result must be the lowest tokens of the bucket."""
    announce("gemv_topk long segment heavy ties (%s)" % layout)
    rng = np.random.default_rng(37)
    dtype, N, k = oracle.F16, 131072, 2048
    col = np.full(N, -1.0)
    if layout == "spread":
        col[rng.permutation(N)[:60000]] = 0.5
    elif layout == "tail":
        col[N - 60000:] = 0.5
    elif layout == "head":
        col[:60000] = 0.5
    else:
        col[rng.permutation(N)[:40000]] = 0.5                 # the bucket of the k-th
        col[rng.permutation(N)[:30000]] = 0.25                # a second large bucket right below (and over part of it)
    top = rng.permutation(N)[:1000]
    col[top] = 2.0 + rng.random(1000)                         # 1000 distinct scores above the bucket
    Kf = rng.standard_normal((1, N, 2, 128)) * 0.01
    Kf[0, :, 0, 0] = col
    Kf[0, :, 1, 0] = col[::-1]                                # second head: the mirrored layout
    qv = np.zeros((1, 2, 128))
    qv[0, :, 0] = 1.0
    _check_long(oracle.to_bits(Kf, dtype), oracle.to_bits(qv, dtype), dtype, 1, k, scale=1.0, redone=0)


def test_long_segment_chunked_shared_kv():
    """Two chunks of 65536 tokens of a KV cache shared by the batch: per-chunk thresholds, per-chunk top-k."""
    from topk_attn_amd import ops
    announce("gemv_topk long chunks N=131072 chunks=2 k=512 shared KV B=2")
    rng = np.random.default_rng(35)
    dtype, N, k, chunks = oracle.F16, 131072, 512, 2
    K = randn_bits(rng, (N, 2, 128), dtype)
    q = randn_bits(rng, (2, 2, 128), dtype)
    idx, val = ops.gemv_topk(to_dev(q, dtype), to_dev(K, dtype), k, group=1, scale=SCALE, num_chunks=chunks)
    torch.cuda.synchronize()
    idx, val = idx.cpu().numpy(), val.cpu().numpy()
    chunk = N // chunks
    for b in range(2):
        for h in range(2):
            ref = oracle.scores_canonical(K[:, h, :], dtype, oracle.group_query(q[b, h:h + 1], dtype, 1), SCALE)
            for c in range(chunks):
                ei, ev = oracle.topk_stable(ref[c * chunk:(c + 1) * chunk], k)
                assert np.array_equal(idx[b, h, c * k:(c + 1) * k], ei + c * chunk), "indices differ (b=%d h=%d c=%d)" % (b, h, c)
                assert np.array_equal(val[b, h, c * k:(c + 1) * k].view(np.uint32), ev.view(np.uint32))


@pytest.mark.parametrize("dtype,B,H,G,N,k,kind", [
    (oracle.F16, 8, 2, 1, 131072, 2048, "heavy"),      # one tile of eight entries
    (oracle.BF16, 3, 2, 4, 70001, 1000, "levels"),     # a tile of four with one entry missing, grouped queries, ties, ragged slice
    (oracle.F16, 2, 1, 8, 100000, 2048, "normal"),     # a tile of two
    (oracle.F16, 9, 1, 2, 66000, 1024, "equal"),       # two tiles of eight, the second with one entry; every score of an entry ties
    (oracle.BF16, 6, 3, 1, 65536, 512, "normal")])     # 18 segments of 65536 tokens: more than a million rows
def test_long_segment_shared_keys(dtype, B, H, G, N, k, kind):
    """Long segments over a key cache that the batch shares (key_stride_b = 0): one pass over the keys scores a tile of
    batch entries, thresholds and candidate slices are per (entry, head).  Indices and values bit for bit, no segment
    redone, and the kernel that ran."""
    from topk_attn_amd import ops
    announce("gemv_topk long segments, keys shared by the batch: dtype=%d B=%d H=%d G=%d N=%d k=%d %s" % (dtype, B, H, G, N, k, kind))
    rng = np.random.default_rng(B * 1000 + N % 997)
    if kind == "levels":
        K = oracle.to_bits(np.linspace(-2, 2, 16)[rng.integers(0, 16, (N, H, 128))], dtype)
    elif kind == "equal":
        K = np.broadcast_to(randn_bits(rng, (1, 1, 128), dtype), (N, H, 128)).copy()
    else:
        Kf = rng.standard_normal((N, H, 128))
        if kind == "heavy":
            Kf[rng.permutation(N)[:N // 100]] *= 4.0
        K = oracle.to_bits(Kf, dtype)
    q = randn_bits(rng, (B, H * G, 128), dtype)
    plan = ops.GemvTopkPlan(to_dev(q, dtype), to_dev(K, dtype), k, group=G, scale=SCALE)
    ops.profile_reset()
    ops.profile_enable(True)
    plan.run()
    torch.cuda.synchronize()
    ran = ops.profile_read()
    ops.profile_enable(False)
    assert "gemv_candidates_shared" in ran, sorted(ran)
    assert plan.redone_segments() == 0 and plan.gave_up_slices() == 0
    idx, val = plan.idx.cpu().numpy(), plan.val.cpu().numpy()
    for b in range(B):
        for h in range(H):
            ref = oracle.scores_canonical(K[:, h, :], dtype, oracle.group_query(q[b, h * G:(h + 1) * G], dtype, G), SCALE)
            ei, ev = oracle.topk_stable(ref, k)
            assert np.array_equal(idx[b, h], ei), "indices differ (b=%d h=%d)" % (b, h)
            assert np.array_equal(val[b, h].view(np.uint32), ev.view(np.uint32))


def test_long_segment_shared_keys_threshold_withheld(hooks):
    """The same with the thresholds of every third segment withheld: their slices are marked as given up by the
    workgroups that score them for the whole tile, those segments are redone from the keys, the others are not."""
    from topk_attn_amd import ops
    announce("gemv_topk long segments, shared keys, thresholds of segments 1, 4, 7 withheld")
    hooks(tau_spin_limit=64, tau_withhold_mod=3, tau_withhold_rem=1, tau_withhold_mode=0)
    rng = np.random.default_rng(91)
    dtype, B, H, N, k = oracle.F16, 4, 2, 70000, 1024
    K, q = randn_bits(rng, (N, H, 128), dtype), randn_bits(rng, (B, H, 128), dtype)
    plan = ops.GemvTopkPlan(to_dev(q, dtype), to_dev(K, dtype), k, group=1, scale=SCALE).run()
    torch.cuda.synchronize()
    assert plan.redone_segments() == 3
    idx = plan.idx.cpu().numpy()
    for b in range(B):
        for h in range(H):
            ref = oracle.scores_canonical(K[:, h, :], dtype, oracle.group_query(q[b, h:h + 1], dtype, 1), SCALE)
            assert np.array_equal(idx[b, h], oracle.topk_stable(ref, k)[0]), "indices differ (b=%d h=%d)" % (b, h)


def test_long_segment_ragged_length():
    """Segment length that is no multiple of the 256-token slice (nor of 4): the last slice is partial."""
    announce("gemv_topk long segment N=100003 k=1500 bf16 G=2")
    rng = np.random.default_rng(36)
    K = randn_bits(rng, (1, 100003, 2, 128), oracle.BF16)
    _check_long(K, randn_bits(rng, (1, 4, 128), oracle.BF16), oracle.BF16, 2, 1500)


@pytest.mark.parametrize("CSZ,CLEN", [(4, 65536), (3, 131072)])
def test_two_level_long_clusters(CSZ, CLEN):
    """Two-level selection whose clusters are long (cluster ids pick the segments): four segments of 65536 tokens take
    the common-cut route, four of 131072 the sampled-threshold path of the long segments."""
    from topk_attn_amd import ops
    announce("cluster_gemv_topk CSZ=%d CLEN=%d TOPC=2 k=300" % (CSZ, CLEN))
    rng = np.random.default_rng(37)
    H, TOPC, K = 2, 2, 300
    cen = rng.uniform(-0.5, 0.5, (H, CSZ, 128))
    keys = np.empty((CSZ * CLEN, H, 128), dtype=np.float32)
    for c in range(CSZ):
        keys[c * CLEN:(c + 1) * CLEN] = cen[:, c][None] + 0.05 * rng.standard_normal((CLEN, H, 128), dtype=np.float32)
    cen_b, keys_b = oracle.to_bits(cen, oracle.F16), oracle.to_bits(keys, oracle.F16)
    q_b = oracle.to_bits(rng.uniform(-0.5, 0.5, (H, 128)), oracle.F16)
    out = ops.cluster_gemv_topk(to_dev(q_b, oracle.F16), to_dev(cen_b, oracle.F16), to_dev(keys_b, oracle.F16),
                                TOPC, CLEN, K, 1.0)
    torch.cuda.synchronize()
    out = out.cpu().numpy()
    for h in range(H):
        want = oracle.cluster_topk(q_b[h], cen_b[h], keys_b[:, h, :], oracle.F16, TOPC, CLEN, K, 1.0)
        assert np.array_equal(out[h], want)


def test_two_level_long_clusters_redone(hooks):
    """The same with every token-stage segment flagged: the launch that redoes them scores the clusters that the centre
    stage picked (the segments' places come from the cluster ids) and writes global token ids."""
    hooks(force_segment_redo=1)
    test_two_level_long_clusters(3, 131072)


def test_long_segment_plan_reuse():
    """One plan (one workspace) run three times with a new query each time: thresholds of an earlier run must
    never be taken for the current one."""
    from topk_attn_amd import ops
    announce("gemv_topk long segment, plan reused with changing queries")
    rng = np.random.default_rng(38)
    dtype, N, k = oracle.F16, 80000, 1000
    K = randn_bits(rng, (1, N, 1, 128), dtype)
    qd = to_dev(randn_bits(rng, (1, 1, 128), dtype), dtype)
    plan = ops.GemvTopkPlan(qd, to_dev(K, dtype), k, group=1, scale=SCALE)
    for it in range(3):
        q = oracle.to_bits(rng.standard_normal((1, 1, 128)) * (1.0 + it), dtype)
        qd.copy_(to_dev(q, dtype))
        plan.run()
        torch.cuda.synchronize()
        ref = oracle.scores_canonical(K[0, :, 0, :], dtype, oracle.group_query(q[0], dtype, 1), SCALE)
        ei, ev = oracle.topk_stable(ref, k)
        assert np.array_equal(plan.idx[0, 0].cpu().numpy(), ei), "indices differ on run %d" % it
        assert np.array_equal(plan.val[0, 0].cpu().numpy().view(np.uint32), ev.view(np.uint32))


@pytest.fixture
def hooks():
    """Testing hooks of the candidate route, restored to their defaults afterwards."""
    from topk_attn_amd import ops
    yield ops.set_test_hooks
    ops.set_test_hooks()


def test_long_segment_forced_redo(hooks):
    """The force_segment_redo hook sends every long segment through the path that redoes it from the keys — here on
    ordinary data with heavy hitters, in rank mode, with a ragged length."""
    announce("gemv_topk long segment, every segment redone from the keys (N=70001 k=3000 G=4)")
    hooks(force_segment_redo=1)
    rng = np.random.default_rng(39)
    K = randn_bits(rng, (1, 70001, 2, 128), oracle.F16)
    K[0, rng.permutation(70001)[:700]] = oracle.to_bits(rng.standard_normal((700, 2, 128)) * 4.0, oracle.F16)
    _check_long(K, randn_bits(rng, (1, 8, 128), oracle.F16), oracle.F16, 4, 3000, redone=2)


def _redo_keys(rng, N, H, dtype, kind):
    """Keys for the three ways the launch that redoes flagged segments can go on after the bucket of the k-th key is
    known (the query of these cases is the same in all 128 dimensions, so a key row's score is a multiple of its sum)."""
    if kind == "two_values":   # scores +c and -c: with k = number of the larger ones the bucket is taken whole
        rows = np.where(rng.random((1, N, H, 1)) < 0.03, 0.5, -0.5) * np.ones((1, 1, 1, 128))
    elif kind == "equal":      # one score for all tokens: a bucket beyond the LDS whose members only their index tells apart
        rows = np.full((1, N, H, 128), 0.25)
    elif kind == "narrow":     # all scores inside one bucket of the 11 leading key bits, many of them different
        rows = 0.25 + rng.integers(0, 64, (1, N, H, 128)) / 4096.0
    else:                      # "heavy": ordinary data, a few rows four times as long
        rows = rng.standard_normal((1, N, H, 128))
        rows[0, rng.permutation(N)[:N // 100]] *= 4.0
    return oracle.to_bits(rows, dtype)


@pytest.mark.parametrize("kind,N,k", [("heavy", 70001, 3000), ("two_values", 80000, 0), ("equal", 66000, 2000), ("narrow", 131072, 2048),
                                      ("heavy", 300000, 4096)])
def test_long_segment_redo_launch(hooks, kind, N, k):
    """Every segment flagged (force_segment_redo) on the route of the long segments: the launch behind the selection
    redoes them, all workgroups sharing the work, and goes on - by the bucket of the k-th key - with the whole bucket taken,
    with its members gathered and cut, or with one workgroup selecting (a bucket beyond the LDS: narrowed by counting
    passes, or, where all its members carry one key, cut by their rank in index order).  Rank-ordered output."""
    from topk_attn_amd import ops
    announce("gemv_topk long segments, all redone by the launch behind the selection: %s N=%d k=%d" % (kind, N, k))
    hooks(force_segment_redo=1)
    rng = np.random.default_rng(91)
    dtype, H, G = oracle.F16, 2, 2
    K = _redo_keys(rng, N, H, dtype, kind)
    q = randn_bits(rng, (1, H * G, 128), dtype) if kind == "heavy" else oracle.to_bits(np.full((1, H * G, 128), 0.125), dtype)
    if kind == "two_values":   # (head 0's count of the larger score; head 1 then cuts inside its bucket or takes less than it)
        ref = oracle.scores_canonical(K[0, :, 0, :], dtype, oracle.group_query(q[0, 0:G], dtype, G), SCALE)
        k = int((ref > 0).sum())
    ops.profile_reset()
    ops.profile_enable(True)
    _check_long(K, q, dtype, G, k, redone=H)
    ran = ops.profile_read()
    ops.profile_enable(False)
    assert "redo_segments" in ran and "select_finalize_cand" in ran, sorted(ran)


def test_long_segments_sixteen_heads():
    """Sixteen KV heads: the rows of one head lie 4 KB apart, and the streaming workgroups take their slices in units
    that go round the segments instead of segment by segment (137 slices per segment: the last unit of each is short)."""
    announce("gemv_topk long segments, sixteen heads (N=70001 k=2048): slices taken round the segments")
    rng = np.random.default_rng(44)
    K = randn_bits(rng, (1, 70001, 16, 128), oracle.F16)
    _check_long(K, randn_bits(rng, (1, 16, 128), oracle.F16), oracle.F16, 1, 2048, redone=0)


@pytest.mark.parametrize("withheld", [(2, 1), (1, 0)])
def test_long_segment_threshold_never_published(hooks, withheld):
    """The bounded wait of the streaming workgroups runs out: the threshold of one of the two segments (then of
    both) is never published, the spin limit is lowered so that the wait is short, every slice of such a segment
    is marked as given up, and the selection kernel redoes exactly those segments from the keys.  The segment
    that did get its threshold keeps the candidate route.  Every kernel runs to its end."""
    mod, rem = withheld
    announce("gemv_topk long segments, threshold of segments s %% %d == %d withheld for good (N=131072 k=2048)" % (mod, rem))
    hooks(tau_spin_limit=64, tau_withhold_mod=mod, tau_withhold_rem=rem, tau_withhold_mode=0)
    rng = np.random.default_rng(43)
    K = randn_bits(rng, (1, 131072, 2, 128), oracle.F16)
    K[0, rng.permutation(131072)[:1300]] = oracle.to_bits(rng.standard_normal((1300, 2, 128)) * 4.0, oracle.F16)
    affected = 2 // mod
    _check_long(K, randn_bits(rng, (1, 2, 128), oracle.F16), oracle.F16, 1, 2048, redone=affected, gave_up=affected * 256)


# ---- a few segments of middling length: a cut from common sample rows, candidates ranked by counting ----

@pytest.mark.parametrize("dtype,B,H,G,N,k", [(oracle.F16, 1, 1, 1, 32768, 2048), (oracle.BF16, 1, 2, 4, 20011, 1000),
                                             (oracle.F16, 2, 2, 1, 65536, 2048), (oracle.F16, 1, 1, 8, 40000, 1),
                                             (oracle.BF16, 1, 3, 2, 16385, 2048), (oracle.F16, 1, 2, 1, 12000, 400),
                                             (oracle.BF16, 2, 2, 4, 8193, 300),
                                             # more than 65536 rows: the cut from a launch of its own, 512 tokens per GEMV workgroup
                                             (oracle.F16, 1, 4, 1, 32768, 2048), (oracle.BF16, 2, 3, 2, 20001, 1000),
                                             (oracle.F16, 1, 8, 4, 49152, 1500), (oracle.F16, 3, 1, 1, 30000, 7),
                                             # k above n / 14.5 (up to n / 8): slices of 128 tokens
                                             (oracle.F16, 1, 1, 1, 20000, 2048), (oracle.BF16, 2, 1, 2, 16384, 2048),
                                             (oracle.F16, 1, 8, 4, 24577, 2048), (oracle.BF16, 1, 3, 1, 32768, 2048 + 1000),
                                             # segments of 8193 .. 16384 tokens on calls of more than 65536 rows
                                             (oracle.F16, 1, 8, 1, 16384, 1024), (oracle.BF16, 2, 8, 4, 9001, 512),
                                             (oracle.F16, 1, 5, 2, 16384, 2048),
                                             # sixteen heads (rows of a head 4 KB apart) in a number of segments that is no power of two
                                             (oracle.F16, 3, 16, 1, 9000, 500),
                                             # more than 655360 rows (several generations of GEMV workgroups)
                                             (oracle.F16, 3, 8, 1, 32768, 2048), (oracle.BF16, 5, 8, 2, 20000, 1000)])
def test_common_cut_route(dtype, B, H, G, N, k):
    """Calls of up to 1572864 rows with segments of 8193 .. 65536 tokens and
    no score output: the cut of a segment comes from 256 sample rows - every GEMV workgroup derives the same one, or, on
    calls of more than 65536 rows, one workgroup per segment does in a launch before the GEMV - and eight ranking
    workgroups per segment rank the candidates.  Ordinary data with heavy hitters; ragged lengths (an odd number of
    slices of 256 tokens); no segment is redone from the keys."""
    announce("gemv_topk common-cut route dtype=%d B=%d H=%d G=%d N=%d k=%d" % (dtype, B, H, G, N, k))
    rng = np.random.default_rng(51)
    K = randn_bits(rng, (B, N, H, 128), dtype)
    K[:, rng.permutation(N)[:N // 100]] = oracle.to_bits(rng.standard_normal((B, N // 100, H, 128)) * 4.0, dtype)
    _check_long(K, randn_bits(rng, (B, H * G, 128), dtype), dtype, G, k, redone=0)


@pytest.mark.parametrize("heads", [1, 3])
@pytest.mark.parametrize("kind", ["levels", "all_equal", "two_buckets", "ramp", "tail_block"])
def test_common_cut_route_ties_and_clusters(kind, heads):
    """Ties (16-level keys, constant keys, three-valued scores with the k-th inside a bucket of thousands of equal
    scores) and top scores that sit in one place (a ramp over the tokens; all of the top k in the last tokens, so
    that their slices hold more candidates than the ranking kernel reads in its first round trip).  With three heads
    (the same keys in each) the call has more than 65536 rows and finds its cuts in a launch of their own."""
    announce("gemv_topk common-cut route, %s, %d head(s)" % (kind, heads))
    rng = np.random.default_rng(52)
    dtype, N, k = oracle.F16, 32768, 2048
    q = randn_bits(rng, (1, 1, 128), dtype)
    if kind == "levels":
        K = oracle.to_bits(np.linspace(-2, 2, 16)[rng.integers(0, 16, (1, N, 1, 128))], dtype)
    elif kind == "all_equal":
        K = np.broadcast_to(randn_bits(rng, (1, 1, 1, 128), dtype), (1, N, 1, 128)).copy()
    else:
        col = np.full(N, -1.0)
        if kind == "two_buckets":
            col[rng.permutation(N)[:9000]] = 0.5
            col[rng.permutation(N)[:700]] = 2.0
        elif kind == "ramp":
            col = np.linspace(-1.0, 1.0, N) + rng.standard_normal(N) * 0.01
        else:
            col = rng.standard_normal(N) * 0.1
            col[N - 2300:] += 3.0
        Kf = np.zeros((1, N, 1, 128))
        Kf[0, :, 0, 5] = col
        qf = np.zeros((1, 1, 128))
        qf[0, 0, 5] = 1.0            # unit query: the score is one key column
        K, q = oracle.to_bits(Kf, dtype), oracle.to_bits(qf, dtype)
    if heads > 1:
        K, q = np.ascontiguousarray(np.repeat(K, heads, axis=2)), np.ascontiguousarray(np.repeat(q, heads, axis=1))
    _check_long(K, q, dtype, 1, k, scale=1.0, redone=0)


def _cut_sample_positions(seg, n, samples=256):
    """Token positions of the sample rows of a segment on the common-cut route."""
    stride = n // samples
    return [i * stride + (((((i + seg * 0x85ebca6b) & 0xFFFFFFFF) * 0x9e3779b9) & 0xFFFFFFFF) * stride >> 32) for i in range(samples)]


def test_common_cut_route_adversarial_sample_falls_back():
    """Heavy tokens exactly where the cut is sampled: the cut lands among them, fewer than k tokens pass, and the
    segment is redone from the keys by its first ranking workgroup; the other head keeps the route."""
    announce("gemv_topk common-cut route, adversarial sample (fallback)")
    rng = np.random.default_rng(53)
    N, k, dtype = 32768, 2048, oracle.F16
    Kf = rng.standard_normal((1, N, 2, 128)) * 0.05
    qf = rng.standard_normal((1, 2, 128))
    pos = _cut_sample_positions(0, N)
    Kf[0, pos, 0, :] = qf[0, 0] * rng.uniform(0.5, 1.5, (len(pos), 1))
    _check_long(oracle.to_bits(Kf, dtype), oracle.to_bits(qf, dtype), dtype, 1, k, redone=1)


def test_common_cut_route_adversarial_sample_falls_back_on_a_call_that_fills_the_gpu():
    """The same on a call of more than 65536 rows (four heads): the cut of head 2 comes out among the heavy tokens."""
    announce("gemv_topk common-cut route, cuts announced inside the GEMV launch, adversarial sample (fallback)")
    rng = np.random.default_rng(57)
    N, k, dtype = 32768, 2048, oracle.F16
    Kf = rng.standard_normal((1, N, 4, 128)) * 0.05
    qf = rng.standard_normal((1, 4, 128))
    pos = _cut_sample_positions(2, N)
    Kf[0, pos, 2, :] = qf[0, 2] * rng.uniform(0.5, 1.5, (len(pos), 1))
    _check_long(oracle.to_bits(Kf, dtype), oracle.to_bits(qf, dtype), dtype, 1, k, redone=1)


@pytest.mark.parametrize("H,N,k,mod,rem,affected", [(4, 32768, 2048, 1, 0, 4), (4, 32768, 2048, 2, 1, 2), (20, 16384, 1024, 3, 1, 7)])
def test_common_cut_route_cut_never_announced(hooks, H, N, k, mod, rem, affected):
    """Calls of more than 65536 rows find their cuts in the first workgroups of the GEMV launch, and the scoring
    workgroups wait for their segment's word - a bounded wait.  With the word of chosen segments withheld and the wait
    shortened, every slice of those segments is marked and the ranking kernel redoes them from the keys; the others keep
    the route.  Every kernel runs to its end.  The call of twenty heads has more scoring workgroups than run at once:
    there the sampling workgroups score tokens themselves afterwards, and wait like the others."""
    announce("gemv_topk common-cut route, %d x %d tokens, the cut of segments s %% %d == %d is never announced" % (H, N, mod, rem))
    hooks(tau_spin_limit=64, tau_withhold_mod=mod, tau_withhold_rem=rem, tau_withhold_mode=0)
    rng = np.random.default_rng(58)
    K = randn_bits(rng, (1, N, H, 128), oracle.F16)
    _check_long(K, randn_bits(rng, (1, H, 128), oracle.F16), oracle.F16, 1, k, redone=affected, gave_up=affected * (N // 256))


def test_common_cut_route_sample_sits_low():
    """The sampled rows score lower than the rest (their keys shrunk by a fifth): the cut lands low and more tokens pass
    than one ranking workgroup may hold (8192).  No part of the order is that large, so the segment keeps the route."""
    announce("gemv_topk common-cut route, sample below the rest: more than 8192 candidates, none redone")
    rng = np.random.default_rng(56)
    N, k, dtype = 65536, 2048, oracle.F16
    Kf = rng.standard_normal((1, N, 1, 128))
    pos = _cut_sample_positions(0, N)
    Kf[0, pos, 0, :] *= 0.8
    K, q = oracle.to_bits(Kf, dtype), randn_bits(rng, (1, 1, 128), dtype)
    ref = oracle.scores_canonical(K[0, :, 0, :], dtype, oracle.group_query(q[0, 0:1], dtype, 1), SCALE)
    m = 256.0 * k / N
    rank = int(np.ceil(m + 5.5 * np.sqrt(m) + 2.0))
    cut = np.sort(ref[pos])[::-1][rank - 1]
    assert 8192 < int((ref >= cut).sum()) < 16384, "the premise of this test: candidates at or above the rank-%d sample" % rank
    _check_long(K, q, dtype, 1, k, redone=0)


def test_common_cut_route_forced_redo(hooks):
    announce("gemv_topk common-cut route, every segment redone from the keys")
    hooks(force_segment_redo=1)
    rng = np.random.default_rng(54)
    K = randn_bits(rng, (1, 30001, 2, 128), oracle.BF16)
    _check_long(K, randn_bits(rng, (1, 4, 128), oracle.BF16), oracle.BF16, 2, 1500, redone=2)


def test_common_cut_route_chunked():
    """Two chunks of 32768 tokens per head: per-chunk top-k with indices counted over the whole sequence."""
    announce("gemv_topk common-cut route, 2 chunks x 32768")
    from topk_attn_amd import ops
    rng = np.random.default_rng(55)
    dtype, N, k = oracle.F16, 65536, 1024
    K = randn_bits(rng, (1, N, 2, 128), dtype)
    q = randn_bits(rng, (1, 2, 128), dtype)
    idx, val = ops.gemv_topk(to_dev(q, dtype), to_dev(K, dtype), k, scale=SCALE, num_chunks=2)
    torch.cuda.synchronize()
    idx, val = idx.cpu().numpy(), val.cpu().numpy()
    for h in range(2):
        ref = oracle.scores_canonical(K[0, :, h, :], dtype, oracle.group_query(q[0, h:h + 1], dtype, 1), SCALE)
        for c in range(2):
            ei, ev = oracle.topk_stable(ref[c * 32768:(c + 1) * 32768], k)
            assert np.array_equal(idx[0, h, c * k:(c + 1) * k], ei + c * 32768)
            assert np.array_equal(val[0, h, c * k:(c + 1) * k].view(np.uint32), ev.view(np.uint32))


@pytest.mark.parametrize("forced", [0, 1])
def test_long_chunks_route_chunked(hooks, forced):
    """Two chunks of 70 000 tokens per head on the route of the long segments (a chunk is a segment; indices count over the
    whole sequence), from the candidates and with every chunk redone by the launch behind the selection."""
    announce("gemv_topk long segments, 2 chunks x 70000, forced redo %d" % forced)
    from topk_attn_amd import ops
    hooks(force_segment_redo=forced)
    rng = np.random.default_rng(57)
    dtype, C, k, G = oracle.BF16, 70000, 1500, 2
    K = randn_bits(rng, (1, 2 * C, 2, 128), dtype)
    q = randn_bits(rng, (1, 2 * G, 128), dtype)
    plan = ops.GemvTopkPlan(to_dev(q, dtype), to_dev(K, dtype), k, group=G, scale=SCALE, num_chunks=2).run()
    torch.cuda.synchronize()
    assert plan.redone_segments() == (4 if forced else 0)
    idx, val = plan.idx.cpu().numpy(), plan.val.cpu().numpy()
    for h in range(2):
        ref = oracle.scores_canonical(K[0, :, h, :], dtype, oracle.group_query(q[0, h * G:(h + 1) * G], dtype, G), SCALE)
        for c in range(2):
            ei, ev = oracle.topk_stable(ref[c * C:(c + 1) * C], k)
            assert np.array_equal(idx[0, h, c * k:(c + 1) * k], ei + c * C), "indices differ (h=%d chunk %d)" % (h, c)
            assert np.array_equal(val[0, h, c * k:(c + 1) * k].view(np.uint32), ev.view(np.uint32))


# ---- key caches that are views: padded head dimension, head-major storage ----

@pytest.mark.parametrize("layout", ["padded_heads", "head_major"])
@pytest.mark.parametrize("N,k", [(1500, 100), (6000, 300), (20000, 700), (40000, 8000), (70000, 1000)])
def test_key_cache_layouts(layout, N, k):
    """The key strides are arguments: a cache with unused heads on either side of the ones in use (token stride larger
    than the heads in use, base pointer inside a row) and a cache stored head-major (token stride 128, head stride
    N * 128) must give what the contiguous copy gives, on every route (one launch, registers of a workgroup, common
    cut, dense path, candidate slices)."""
    from topk_attn_amd import ops
    announce("gemv_topk key layout %s N=%d k=%d" % (layout, N, k))
    rng = np.random.default_rng(N + k)
    dtype, B, H, G = oracle.F16, 2, 2, 2
    q = randn_bits(rng, (B, H * G, 128), dtype)
    K = randn_bits(rng, (B, N, H, 128), dtype)
    if layout == "padded_heads":
        full = randn_bits(rng, (B, N, H + 3, 128), dtype)
        full[:, :, 1:1 + H] = K
        Kd = to_dev(full, dtype)[:, :, 1:1 + H]
    else:
        Kd = to_dev(np.ascontiguousarray(K.transpose(0, 2, 1, 3)), dtype).permute(0, 2, 1, 3)
    assert not Kd.is_contiguous()
    plan = ops.GemvTopkPlan(to_dev(q, dtype), Kd, k, group=G, scale=SCALE).run()
    torch.cuda.synchronize()
    idx, val = plan.idx.cpu().numpy(), plan.val.cpu().numpy()
    for b in range(B):
        for h in range(H):
            ref = oracle.scores_canonical(K[b, :, h, :], dtype, oracle.group_query(q[b, h * G:(h + 1) * G], dtype, G), SCALE)
            ei, ev = oracle.topk_stable(ref, k)
            assert np.array_equal(idx[b, h], ei), "indices differ (b=%d h=%d)" % (b, h)
            assert np.array_equal(val[b, h].view(np.uint32), ev.view(np.uint32))
