"""Pins the CPU oracle (tka_oracle.c) against evidence that does not come from the oracle itself: numpy / scipy /
torch library routines, closed forms, hand-derived known answers for the reduction order, invariants, brute force."""
import itertools

import numpy as np
import pytest
import scipy.special

import oracle

RNG = np.random.default_rng(20240)
SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


# ---- conversions -----------------------------------------------------------------------------------------

def test_half_to_float_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().orc_half_to_float(int(b)) for b in bits], np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_bf16_to_float_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = (bits.astype(np.uint32) << 16).view(np.float32)
    got = np.array([oracle.lib().orc_bf16_to_float(int(b)) for b in bits], np.float32)
    ok = ~np.isnan(want)   # NaN payloads do not survive the float -> Python float -> float32 round trip
    assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok]) and np.isnan(got[~ok]).all()


def test_to_bits_bf16_round_to_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.14159], np.float32)  # 1+2^-8 ties to even (1.0), 1+3*2^-8 -> up
    import torch
    want = torch.tensor(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.to_bits(x, oracle.BF16), want)


# ---- scores: the canonical 16-lane order -------------------------------------------------------------------

def _one_row(qvals, kvals, dtype=oracle.F16, scale=1.0):
    q = np.zeros((1, 128)); k = np.zeros((1, 128))
    for d, v in qvals.items():
        q[0, d] = v
    for d, v in kvals.items():
        k[0, d] = v
    qb, kb = oracle.to_bits(q, dtype), oracle.to_bits(k, dtype)
    return float(oracle.scores_canonical(kb, dtype, oracle.group_query(qb, dtype, 1), scale)[0])


def test_lane_chain_is_sequential_fma():
    """Inside lane j the eight products are accumulated in ascending d (gemv_topk.cu:320-324).
    Products 2^24, 1, -2^24, 1: the sequential chain loses the first 1 and gives 1; a pairwise tree would give 2."""
    for lane in (0, 5, 15):
        d = 8 * lane
        got = _one_row({d: 4096, d + 1: 1, d + 2: 4096, d + 3: 1}, {d: 4096, d + 1: 1, d + 2: -4096, d + 3: 1})
        assert got == 1.0


def test_butterfly_partner_distances_8_4_2_1():
    """Across lanes the partials are added with partner distance 8 first, then 4, 2, 1 (gemv_topk.cu:325-328).
    One product per lane; each case is arranged so that any other pairing order loses or keeps a different 1."""
    big = (4096, 4096)  # q, k -> product 2^24

    def lanes(assign):
        q, k = {}, {}
        for lane, (qv, kv) in assign.items():
            q[8 * lane], k[8 * lane] = qv, kv
        return _one_row(q, k)

    # distance 8 first: (p0 + p8) cancels exactly, so both ones survive -> 2 (sequential lane order would give 1)
    assert lanes({0: big, 8: (4096, -4096), 4: (1, 1), 12: (1, 1)}) == 2.0
    # distance 4 second: p0 and p4 cancel at the second level, p2 + p6 = 2 is added at the third
    assert lanes({0: big, 4: (4096, -4096), 2: (1, 1), 6: (1, 1)}) == 2.0
    # distance 2 third: p0 and p2 cancel at the third level, p1 + p3 = 2 is added at the last
    assert lanes({0: big, 2: (4096, -4096), 1: (1, 1), 3: (1, 1)}) == 2.0
    # distance 1 last: p0 + p1 is formed only at the very end, after (p0 + p8) absorbed and lost p8 = 1
    assert lanes({0: big, 8: (1, 1), 1: (4096, -4096)}) == 0.0
    # and the mirror: the 1 in lane 9 meets +2^24 of lane 1 first and is lost there as well
    assert lanes({0: (4096, -4096), 1: big, 9: (1, 1)}) == 0.0


def test_scale_is_one_multiply_after_the_sum():
    got = _one_row({0: 3, 1: 5}, {0: 7, 1: 11}, scale=SCALE)
    assert got == float(np.float32(76.0) * np.float32(SCALE))


@pytest.mark.parametrize("dtype", [oracle.F16, oracle.BF16])
def test_scores_close_to_fp64_dot(dtype):
    K = oracle.to_bits(RNG.standard_normal((4000, 128)), dtype)
    q = oracle.to_bits(RNG.standard_normal((4, 128)), dtype)
    for g in (1, 4):
        qf = oracle.group_query(q[:g], dtype, g)
        s = oracle.scores_canonical(K, dtype, qf, SCALE)
        Kf, qfl = oracle.from_bits(K, dtype).astype(np.float64), oracle.from_bits(q[:g], dtype).astype(np.float64)
        truth = (Kf @ qfl.sum(0)) * SCALE
        assert np.abs(s - truth).max() < 1e-5
        assert np.abs(oracle.scores_f64(K, dtype, q[:g], SCALE) - truth).max() < 1e-12


def test_unit_query_reproduces_a_key_column():
    K = oracle.to_bits(RNG.standard_normal((300, 128)), oracle.F16)
    for i in (0, 9, 127):
        q = np.zeros((1, 128)); q[0, i] = 1.0
        s = oracle.scores_canonical(K, oracle.F16, oracle.group_query(oracle.to_bits(q, oracle.F16), oracle.F16, 1), 1.0)
        assert np.array_equal(s, oracle.from_bits(K[:, i], oracle.F16))


def test_strided_rows():
    K = oracle.to_bits(RNG.standard_normal((50, 3, 128)), oracle.F16)
    qf = RNG.standard_normal(128).astype(np.float32)
    a = oracle.scores_canonical(K[:, 1, :], oracle.F16, qf)
    b = oracle.scores_canonical(np.ascontiguousarray(K[:, 1, :]), oracle.F16, qf)
    assert np.array_equal(a, b)


# ---- selection ---------------------------------------------------------------------------------------------

def _lexsort_topk(scores, k):
    s = np.asarray(scores, np.float32).astype(np.float64)
    s = np.where(np.isnan(s), -np.inf, s)                     # NaN sorts below every number ...
    nan_last = np.isnan(np.asarray(scores, np.float32))
    order = np.lexsort((np.arange(len(s)), nan_last, -s))     # ... even below -inf; ties -> lower index
    return order[:k].astype(np.int32)


@pytest.mark.parametrize("n,k", [(1, 1), (10, 10), (1000, 37), (5000, 2048), (70000, 4096)])
def test_topk_matches_stable_sort(n, k):
    import torch
    x = RNG.standard_normal(n).astype(np.float32)
    x[RNG.integers(0, n, n // 3)] = np.float32(0.5)           # plenty of ties
    idx, val = oracle.topk_stable(x, k)
    assert np.array_equal(idx, _lexsort_topk(x, k))
    tv, ti = torch.sort(torch.from_numpy(x), descending=True, stable=True)
    assert np.array_equal(idx, ti[:k].numpy().astype(np.int32)) and np.array_equal(val, tv[:k].numpy())


def test_topk_special_values():
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -0.0, 0.0, np.nan, -1.0], np.float32)
    idx, val = oracle.topk_stable(x, 10)
    assert idx.tolist() == [2, 5, 0, 1, 6, 7, 9, 3, 4, 8]     # +-0 tie by index; NaN last, by index
    assert np.signbit(val[2:6]).sum() == 0                    # -0.0 is returned as +0.0


def test_topk_brute_force_tiny():
    for n in range(1, 7):
        for vals in itertools.product([0.0, 1.0, -1.0], repeat=n):
            x = np.array(vals, np.float32)
            for k in range(1, n + 1):
                idx, _ = oracle.topk_stable(x, k)
                want = sorted(range(n), key=lambda i: (-vals[i], i))[:k]
                assert idx.tolist() == want


def test_score_key_is_monotone():
    x = np.sort(np.concatenate([RNG.standard_normal(2000).astype(np.float32), np.float32([0, -0.0, np.inf, -np.inf, 1e-40, -1e-40])]))
    keys = np.array([oracle.lib().orc_score_key(float(v)) for v in x], np.uint64)
    assert (np.diff(keys.astype(np.int64)) >= 0).all()
    assert np.array_equal(keys.astype(np.uint32), oracle.score_keys(x))
    assert oracle.lib().orc_score_key(float("nan")) == 0
    back = np.array([oracle.lib().orc_key_score(int(k)) for k in keys], np.float32)
    assert np.array_equal(back, x + np.float32(0.0))


def test_rejects_bad_k():
    with pytest.raises(ValueError):
        oracle.topk_stable(np.zeros(4, np.float32), 5)


def test_center_expand_closed_form():
    q = oracle.to_bits(RNG.standard_normal((1, 128)), oracle.F16)
    cen = oracle.to_bits(RNG.standard_normal((500, 128)), oracle.F16)
    out, cids, cval = oracle.center_topk_expand(q[0], cen, oracle.F16, 7, 16, SCALE)
    s = oracle.scores_canonical(cen, oracle.F16, oracle.group_query(q, oracle.F16, 1), SCALE)
    assert np.array_equal(cids, _lexsort_topk(s, 7)) and np.array_equal(cval, s[cids])
    assert np.array_equal(out.reshape(7, 16), cids[:, None] * 16 + np.arange(16)[None])


def test_cluster_topk_composition():
    H, CSZ, CLEN, TOPC, K = 2, 8, 96, 3, 20
    cen = oracle.to_bits(RNG.uniform(-0.5, 0.5, (H, CSZ, 128)), oracle.F16)
    keys = oracle.to_bits(RNG.standard_normal((CSZ * CLEN, H, 128)), oracle.F16)
    q = oracle.to_bits(RNG.uniform(-0.5, 0.5, (H, 128)), oracle.F16)
    for h in range(H):
        got = oracle.cluster_topk(q[h], cen[h], keys[:, h, :], oracle.F16, TOPC, CLEN, K)
        qf = oracle.group_query(q[h:h + 1], oracle.F16, 1)
        top = _lexsort_topk(oracle.scores_canonical(cen[h], oracle.F16, qf), TOPC)
        want = []
        for c in top:
            ts = oracle.scores_canonical(keys[c * CLEN:(c + 1) * CLEN, h, :], oracle.F16, qf)
            want.extend((c * CLEN + _lexsort_topk(ts, K)).tolist())
        assert got.tolist() == want


@pytest.mark.parametrize("k,sink,local,n", [(50, 8, 16, 1000), (10, 0, 0, 20), (30, 40, 40, 60), (5, 100, 100, 50)])
def test_index_union_vs_numpy(k, sink, local, n):
    ids = RNG.choice(n, k, replace=False).astype(np.int32)
    out, cnt = oracle.index_union(ids, sink, local, n)
    want = np.union1d(np.union1d(ids, np.arange(min(sink, n))), np.arange(max(n - local, 0), n))
    assert cnt == len(want) and np.array_equal(out[:cnt], want)


# ---- attention ---------------------------------------------------------------------------------------------

def _np_attention(q, K, V, dtype, idx, scale):
    qf = oracle.from_bits(q, dtype).astype(np.float64)
    Kf = oracle.from_bits(K, dtype).astype(np.float64)[idx]
    Vf = oracle.from_bits(V, dtype).astype(np.float64)[idx]
    x = (Kf @ qf) * scale
    return scipy.special.softmax(x) @ Vf, scipy.special.logsumexp(x)


@pytest.mark.parametrize("dtype", [oracle.F16, oracle.BF16])
def test_attention_vs_scipy(dtype):
    q = oracle.to_bits(RNG.standard_normal(128), dtype)
    K = oracle.to_bits(RNG.standard_normal((700, 128)), dtype)
    V = oracle.to_bits(RNG.standard_normal((700, 128)), dtype)
    out, lse = oracle.attention_f64(q, K, V, dtype, scale=SCALE)
    want, want_lse = _np_attention(q, K, V, dtype, np.arange(700), SCALE)
    assert np.abs(out - want).max() < 1e-12 and abs(lse - want_lse) < 1e-10
    idx = RNG.choice(700, 100, replace=False).astype(np.int32)
    out, _ = oracle.attention_f64(q, K, V, dtype, idx=idx, scale=SCALE)
    assert np.abs(out - _np_attention(q, K, V, dtype, idx, SCALE)[0]).max() < 1e-12
    perm, _ = oracle.attention_f64(q, K, V, dtype, idx=idx[::-1].copy(), scale=SCALE)
    assert np.abs(out - perm).max() < 1e-12                  # order of the selected set is irrelevant


def test_attention_closed_forms():
    dtype = oracle.F16
    V = oracle.to_bits(RNG.standard_normal((64, 128)), dtype)
    K = oracle.to_bits(np.zeros((64, 128)), dtype)
    q = oracle.to_bits(RNG.standard_normal(128), dtype)
    out, lse = oracle.attention_f64(q, K, V, dtype, scale=1.0)
    assert np.abs(out - oracle.from_bits(V, dtype).astype(np.float64).mean(0)).max() < 1e-12   # uniform weights
    assert abs(lse - np.log(64)) < 1e-12
    logit = np.full(64, -50.0, np.float32); logit[17] = 50.0
    out, _ = oracle.attention_f64(q, K, V, dtype, idx=np.arange(64, dtype=np.int32), logit=logit, scale=1.0)
    assert np.abs(out - oracle.from_bits(V[17], dtype)).max() < 1e-12                            # dominant logit
    out, lse = oracle.attention_f64(q, K, V, dtype, idx=np.zeros(0, np.int32), count=0)
    assert (out == 0).all() and lse == -np.inf


def test_lse_combine_split_equals_unsplit():
    dtype = oracle.F16
    q = oracle.to_bits(RNG.standard_normal(128), dtype)
    K = oracle.to_bits(RNG.standard_normal((900, 128)), dtype)
    V = oracle.to_bits(RNG.standard_normal((900, 128)), dtype)
    whole, whole_lse = _np_attention(q, K, V, dtype, np.arange(900), SCALE)
    bounds = [0, 1, 300, 300, 640, 900]                       # includes an empty split
    m, l, acc = [], [], []
    qf, Kf, Vf = (oracle.from_bits(a, dtype).astype(np.float64) for a in (q, K, V))
    for a, b in zip(bounds[:-1], bounds[1:]):
        x = (Kf[a:b] @ qf) * SCALE * np.log2(np.e)
        if b > a:
            mm = x.max(); p = np.exp2(x - mm)
            m.append(mm); l.append(p.sum()); acc.append(p @ Vf[a:b])
        else:
            m.append(-np.inf); l.append(0.0); acc.append(np.zeros(128))
    out, lse = oracle.lse_combine(np.array(m), np.array(l), np.array(acc))
    assert np.abs(out - whole).max() < 1e-5 and abs(lse - whole_lse) < 1e-5     # fp32 partials
    out1, _ = oracle.lse_combine(np.array(m[:1]), np.array(l[:1]), np.array(acc[:1]))
    assert np.abs(out1 - Vf[0]).max() < 1e-6                                     # S = 1
    out0, lse0 = oracle.lse_combine(np.array([-np.inf]), np.array([0.0]), np.zeros((1, 128)))
    assert (out0 == 0).all() and lse0 == -np.inf


def test_retrieval_attention_composition():
    """Per-chunk stable top-k, hand-off slot [c*k + r], softmax over the survivors' fp32 scores, gathered P.V
    (retrieval_attention.cu:1162-1339) re-derived with numpy."""
    dtype, N, chunks, k = oracle.F16, 512, 4, 16
    q = oracle.to_bits(RNG.standard_normal(128) * 0.1, dtype)
    K = oracle.to_bits(RNG.standard_normal((N, 128)) * 0.1, dtype)
    V = oracle.to_bits(RNG.standard_normal((N, 128)) * 0.1, dtype)
    out, idx, val = oracle.retrieval_attention(q, K, V, dtype, chunks, k)
    s = oracle.scores_canonical(K, dtype, oracle.group_query(q[None], dtype, 1))
    want_idx = np.concatenate([c * 128 + _lexsort_topk(s[c * 128:(c + 1) * 128], k) for c in range(chunks)])
    assert np.array_equal(idx, want_idx) and np.array_equal(val, s[want_idx])
    p = np.exp(val.astype(np.float64)); p /= p.sum()          # raw exp, as test_ra.py:137-139
    assert np.abs(out - p @ oracle.from_bits(V, dtype).astype(np.float64)[want_idx]).max() < 1e-12


def test_sparse_decode_step_composition():
    dtype, N, G, k, sink, local = oracle.BF16, 600, 4, 40, 8, 32
    q = oracle.to_bits(RNG.standard_normal((G, 128)), dtype)
    K = oracle.to_bits(RNG.standard_normal((N, 128)), dtype)
    V = oracle.to_bits(RNG.standard_normal((N, 128)), dtype)
    out, tidx, tval, uni = oracle.sparse_decode_step(q, K, V, dtype, G, k, sink, local, SCALE)
    s = oracle.scores_canonical(K, dtype, oracle.group_query(q, dtype, G), SCALE)
    assert np.array_equal(tidx, _lexsort_topk(s, k)) and np.array_equal(tval, s[tidx])
    want_uni = np.union1d(np.union1d(tidx, np.arange(sink)), np.arange(N - local, N))
    assert np.array_equal(uni, want_uni) and len(set(uni.tolist())) == len(uni)   # duplicate-free
    for g in range(G):
        assert np.abs(out[g] - _np_attention(q[g], K, V, dtype, want_uni, SCALE)[0]).max() < 1e-12


def test_cpu_baseline_agrees_with_oracle():
    """The torch-CPU restatement used as the reported baseline selects the same sets on tie-free data."""
    import torch
    from oracle.cpu_baseline import sparse_decode_cpu
    dtype, N, H, G, k = oracle.F16, 2000, 2, 4, 64
    qb = oracle.to_bits(RNG.standard_normal((H * G, 128)), dtype)
    Kb = oracle.to_bits(RNG.standard_normal((N, H, 128)), dtype)
    Vb = oracle.to_bits(RNG.standard_normal((N, H, 128)), dtype)
    t = lambda b: torch.from_numpy(b.view(np.int16)).view(torch.float16)
    out, top = sparse_decode_cpu(t(qb), t(Kb), t(Vb), k, 8, 32, SCALE, G)
    for h in range(H):
        ro, ri, _, _ = oracle.sparse_decode_step(qb[h * G:(h + 1) * G], Kb[:, h], Vb[:, h], dtype, G, k, 8, 32, SCALE)
        assert set(top[h].tolist()) == set(ri.tolist())
        assert np.abs(out[h * G:(h + 1) * G].numpy() - ro).max() < 1e-4
