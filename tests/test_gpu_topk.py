"""Selection phase on caller-supplied fp32 scores: indices must equal the oracle's stable order bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from tests.util import announce

pytestmark = pytest.mark.gpu


def _check(scores_np, k):
    from topk_attn_amd import ops
    scores_np = np.ascontiguousarray(scores_np, np.float32)
    if scores_np.ndim == 1:
        scores_np = scores_np[None]
    s = torch.from_numpy(scores_np).cuda()
    idx, val = ops.topk(s, k)
    torch.cuda.synchronize()
    idx, val = idx.cpu().numpy(), val.cpu().numpy()
    for r in range(scores_np.shape[0]):
        ei, ev = oracle.topk_stable(scores_np[r], k)
        assert np.array_equal(idx[r], ei), "row %d: first mismatch at rank %d" % (r, int(np.argmax(idx[r] != ei)))
        assert np.array_equal(val[r].view(np.uint32), ev.view(np.uint32))


CASES = [(1, 1), (1000, 1), (1000, 1000), (1024, 64), (2048, 1024), (4096, 64), (5000, 777), (32768, 2048),
         (131072, 2048), (100000, 4096), (20000, 8192)]


@pytest.mark.parametrize("n,k", CASES)
def test_random_scores(n, k):
    announce("topk random n=%d k=%d" % (n, k))
    rng = np.random.default_rng(n * 31 + k)
    _check(rng.standard_normal(n).astype(np.float32), k)


@pytest.mark.parametrize("n,k", [(4096, 64), (32768, 2048), (70000, 4096)])
def test_all_equal(n, k):
    announce("topk all-equal n=%d k=%d" % (n, k))
    _check(np.full(n, 1.5, np.float32), k)


@pytest.mark.parametrize("n,k", [(8192, 100), (32768, 2048), (262144, 4096)])
def test_few_levels(n, k):
    """Scores drawn from 16 values: every rank boundary falls inside a large tie bucket."""
    announce("topk 16-level n=%d k=%d" % (n, k))
    rng = np.random.default_rng(7)
    levels = np.linspace(-2, 2, 16).astype(np.float32)
    _check(levels[rng.integers(0, 16, n)], k)


def test_signed_zero_inf_nan():
    announce("topk special values")
    rng = np.random.default_rng(3)
    x = rng.standard_normal(6000).astype(np.float32)
    x[::7] = 0.0
    x[3::7] = -0.0
    x[5::97] = np.inf
    x[11::89] = -np.inf
    x[13::101] = np.nan
    for k in (1, 50, 900, 3000, 6000):
        _check(x, k)


def test_ramps_and_segments():
    announce("topk ramps, several segments")
    n = 10000
    up = np.arange(n, dtype=np.float32)
    down = up[::-1].copy()
    two = np.where(np.arange(n) % 2 == 0, 1.0, -1.0).astype(np.float32)
    _check(np.stack([up, down, two, -up]), 1500)


def test_strided_segments():
    announce("topk strided rows")
    from topk_attn_amd import ops
    rng = np.random.default_rng(11)
    full = rng.standard_normal((5, 9000)).astype(np.float32)
    s = torch.from_numpy(full).cuda()
    idx, _ = ops.topk(s[:, :7000], 300)
    torch.cuda.synchronize()
    for r in range(5):
        ei, _ = oracle.topk_stable(full[r, :7000], 300)
        assert np.array_equal(idx[r].cpu().numpy(), ei)
    # rows that start 4 bytes off a 16-byte boundary (no vector loads), long and short
    for lo, hi, k in ((1, 7001, 300), (3, 1500, 64), (1, 4000, 1000)):
        idx, val = ops.topk(s[:, lo:hi], k)
        torch.cuda.synchronize()
        for r in range(5):
            ei, ev = oracle.topk_stable(full[r, lo:hi], k)
            assert np.array_equal(idx[r].cpu().numpy(), ei)
            assert np.array_equal(val[r].cpu().numpy().view(np.uint32), ev.view(np.uint32))


def _short_segment_rows(rng, n):
    """Rows that stress every radix pass of a short segment: ties in the key, in its leading bits, specials."""
    levels = np.linspace(-2, 2, 16).astype(np.float32)
    tiny = (1.0 + np.arange(n) % 5 * 2.0 ** -23).astype(np.float32)        # keys that differ in the last bits only
    close = (1.0 + rng.integers(0, 1 << 12, n) * 2.0 ** -23).astype(np.float32)
    special = rng.standard_normal(n).astype(np.float32)
    special[::7] = 0.0
    special[3::7] = -0.0
    special[5::97] = np.inf
    special[11::89] = -np.inf
    special[13::101] = np.nan
    wide = (rng.standard_normal(n) * 10.0 ** rng.integers(-30, 30, n)).astype(np.float32)
    return [rng.standard_normal(n).astype(np.float32), np.full(n, -3.25, np.float32), levels[rng.integers(0, 16, n)], tiny,
            close, special, wide, np.arange(n, dtype=np.float32), -np.arange(n, dtype=np.float32),
            np.abs(rng.standard_normal(n)).astype(np.float32), np.full(n, np.nan, np.float32)]


@pytest.mark.parametrize("n,k", [(2048, 128), (2048, 1024), (2048, 2048 // 2 - 1), (2048, 1), (2047, 33), (1024, 64),
                                 (1280, 512), (777, 777), (64, 5), (3, 2), (1, 1), (4096, 64), (4096, 1024), (2049, 1000),
                                 (3000, 7), (4095, 513)])
def test_short_segments(n, k):
    """Segments of at most 4096 scores, many per call (the operator's chunks, the centroids of a head):
    adversarial rows and random ones."""
    announce("topk short segments n=%d k=%d" % (n, k))
    rng = np.random.default_rng(n * 7 + k)
    rows = _short_segment_rows(rng, n)
    rows += [rng.standard_normal(n).astype(np.float32) for _ in range(256)]   # enough segments for the small-workgroup route
    _check(np.stack(rows), k)


@pytest.mark.parametrize("n,k", [(8192, 2048), (5000, 1500), (16384, 100), (12345, 2047), (16384, 2048), (8193, 1), (16383, 999)])
def test_register_resident_segments(n, k):
    """Segments of 4097 to 16384 scores (one 1024-thread workgroup holds the keys in registers), k up to 2048:
    adversarial rows and random ones."""
    announce("topk register-resident segments n=%d k=%d" % (n, k))
    rng = np.random.default_rng(n + k)
    rows = _short_segment_rows(rng, n)
    rows += [rng.standard_normal(n).astype(np.float32) for _ in range(3)]
    _check(np.stack(rows), k)


def test_random_shapes_and_distributions():
    """Eighty seeded (segment length, k, segment count, distribution) draws up to 16384 scores per segment, checked
    against numpy's lexsort on the order-preserving keys (oracle.score_keys is pinned against the C oracle)."""
    from topk_attn_amd import ops
    announce("topk 80 random shapes and distributions")
    rng = np.random.default_rng(2024)
    for it in range(80):
        n = int(rng.choice([rng.integers(1, 65), rng.integers(1, 2049), rng.integers(2049, 4097), rng.integers(4097, 16385)]))
        kmax = min(n, 1024 if n <= 4096 else 2048)
        k = int(rng.choice([1, kmax, rng.integers(1, kmax + 1)]))
        S = int(rng.choice([1, 3, rng.integers(1, 300)]))
        S = max(1, min(S, 2_000_000 // n))
        kind = it % 6
        if kind == 0:
            x = rng.standard_normal((S, n))
        elif kind == 1:
            x = np.linspace(-2, 2, 16)[rng.integers(0, 16, (S, n))]
        elif kind == 2:
            x = 1.0 + rng.integers(0, 1 << int(rng.integers(1, 20)), (S, n)) * 2.0 ** -23
        elif kind == 3:
            x = rng.standard_normal((S, n))
            m = rng.random((S, n))
            x[m < 0.1], x[(m >= 0.1) & (m < 0.2)], x[(m >= 0.2) & (m < 0.22)] = 0.0, -0.0, np.inf
            x[(m >= 0.22) & (m < 0.24)], x[(m >= 0.24) & (m < 0.3)] = -np.inf, np.nan
        elif kind == 4:
            x = np.round(rng.standard_normal((S, n)) * int(rng.integers(1, 6)))
        else:
            x = np.full((S, n), float(rng.standard_normal()))
        x = x.astype(np.float32)
        idx, val = ops.topk(torch.from_numpy(x).cuda(), k)
        torch.cuda.synchronize()
        keys = oracle.score_keys(x).astype(np.int64)
        order = np.lexsort((np.broadcast_to(np.arange(n), x.shape), -keys), axis=1)[:, :k]
        case = "draw %d: n=%d k=%d S=%d kind=%d" % (it, n, k, S, kind)
        assert np.array_equal(idx.cpu().numpy(), order.astype(np.int32)), case
        assert np.array_equal(oracle.score_keys(val.cpu().numpy()), np.take_along_axis(oracle.score_keys(x), order, axis=1)), case


def test_short_segments_many():
    """4096 segments in one call (32 batch entries x 32 heads x 4 chunks of the operator)."""
    announce("topk short segments 4096 x 2048, k=128")
    from topk_attn_amd import ops
    rng = np.random.default_rng(99)
    x = rng.standard_normal((4096, 2048)).astype(np.float32)
    x[:, ::3] = np.round(x[:, ::3], 1)      # ties across the rank boundary
    idx, val = ops.topk(torch.from_numpy(x).cuda(), 128)
    torch.cuda.synchronize()
    idx, val = idx.cpu().numpy(), val.cpu().numpy()
    order = np.lexsort((np.broadcast_to(np.arange(2048), x.shape), -x), axis=1)[:, :128]
    assert np.array_equal(idx, order.astype(np.int32))
    assert np.array_equal(val, np.take_along_axis(x, order, axis=1))


def test_rejects_bad_k():
    from topk_attn_amd import ops, TkaError
    s = torch.zeros(2, 100, device="cuda")
    with pytest.raises(TkaError):
        ops.topk(s, 101)
    with pytest.raises(TkaError):
        ops.topk(s, 0)
