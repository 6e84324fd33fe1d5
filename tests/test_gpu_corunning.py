"""The waits inside the launches of the long-segment routes, with another stream keeping the GPU busy.

Two kinds of wait exist in this library.  Streaming workgroups of the candidate GEMV (and of the common-cut GEMV) wait,
for a bounded number of polls, for a threshold that sampling workgroups of the SAME launch publish; when the wait runs
out they mark their slice and the segment is redone from the keys, exactly.  The workgroups of the launch that redoes
flagged segments wait for items that other workgroups of the launch have drawn.  Neither wait needs all workgroups of
a launch to be resident at once, which is what a second stream's kernels can prevent.  Here a second stream (default
priority) runs dense attention launches over a large cache back to back while the first runs decode steps; the steps
must give, bit for bit, what they give on an idle GPU - whether or not a wait ran out - and the test prints how many
segments were redone and whether the other stream was still busy when the steps had finished."""
import numpy as np
import pytest
import torch

import oracle
from tests.util import announce, randn_bits, to_dev

pytestmark = pytest.mark.gpu

SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


def _plan(rng, B, H, G, N, k, dtype=oracle.F16):
    from topk_attn_amd import ops
    Kf = rng.standard_normal((B, N, H, 128))
    Kf[:, rng.permutation(N)[:N // 100]] *= 4.0
    q, K, V = randn_bits(rng, (B, H * G, 128), dtype), oracle.to_bits(Kf, dtype), randn_bits(rng, (B, N, H, 128), dtype)
    return ops.SparseDecodePlan(to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype), k, 64, 512, SCALE, G,
                                out_dtype=torch.float16, want_topk=False)


def _snapshot(plan):
    return plan.out.clone(), plan.union_idx.clone(), plan.union_count.clone()


def _same(a, b):
    cnt = a[2].flatten().tolist()
    lists = all(torch.equal(x[:c], y[:c]) for x, y, c in zip(a[1].flatten(0, 1), b[1].flatten(0, 1), cnt))
    return torch.equal(a[0], b[0]) and torch.equal(a[2], b[2]) and lists


@pytest.fixture
def hooks():
    from topk_attn_amd import ops
    yield ops.set_test_hooks
    ops.set_test_hooks()


def test_steps_while_another_stream_keeps_the_gpu_busy(hooks):
    from topk_attn_amd import ops
    announce("decode steps (2 x 16384 and 1 x 131072 tokens, 8 KV heads) beside dense attention on a second stream")
    rng = np.random.default_rng(301)
    small = _plan(rng, 2, 8, 4, 16384, 2048)      # the common-cut route: cuts announced inside the GEMV launch
    long_ = _plan(rng, 1, 8, 4, 131072, 2048)     # the candidate route: thresholds published inside the GEMV launch
    # the other stream's work: dense attention over 2 x 131072 tokens (1 GB of cache per launch), 300 launches in a row
    dt = torch.float16
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    bq = torch.randn((2, 32, 128), generator=gen, device="cuda", dtype=dt)
    bK = torch.randn((2, 131072, 8, 128), generator=gen, device="cuda", dtype=dt)
    bV = torch.randn((2, 131072, 8, 128), generator=gen, device="cuda", dtype=dt)
    dense = ops.FlashDecodePlan(bq, bK, bV, SCALE, group=4)
    side = torch.cuda.Stream()                    # (default priority)

    want = {}
    for name, plan in (("small", small), ("long", long_)):
        plan.step()
        torch.cuda.synchronize()
        want[name] = _snapshot(plan)
        assert plan.redone_segments() == 0
    hooks(force_segment_redo=1)
    long_.step()
    torch.cuda.synchronize()
    assert _same(_snapshot(long_), want["long"]) and long_.redone_segments() == 8
    hooks()

    for forced in (0, 1):
        with torch.cuda.stream(side):
            for _ in range(300):
                dense.run()
            side_done = torch.cuda.Event()
            side_done.record()
        redone = {"small": [], "long": []}
        beside = 0   # steps that had finished while the other stream was still at work
        for it in range(6):
            for name, plan in (("small", small), ("long", long_)):
                if forced and name == "long":
                    hooks(force_segment_redo=1)
                plan.step()
                got = _snapshot(plan)
                redone[name].append(plan.redone_segments())
                hooks()
                assert _same(got, want[name]), "%s step %d beside the other stream differs from the idle one" % (name, it)
                beside += 0 if side_done.query() else 1
        torch.cuda.synchronize()
        print("  %s: segments redone per step: small %s, long %s; %d of 12 steps had finished while the other stream was at work" % (
            "every long segment flagged" if forced else "as the data has it", redone["small"], redone["long"], beside), flush=True)
        assert beside >= 6, "the other stream's work ended too early for this test to say anything"
        if forced:
            assert all(r == 8 for r in redone["long"])
