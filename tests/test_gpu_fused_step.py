"""The decode step of a caller that wants the attention output alone, on long segments (up to 131072 tokens; longer ones
run the selection launch as ever and are here for comparison): selection and attention run in ONE launch (every attention workgroup derives the k-th largest composite from the candidates of the GEMV launch and keeps
its share of the token list in LDS), followed by the combine launch that also redoes flagged segments from the keys.
Nothing but the output leaves the step, so the checks are: the output against the fp64 oracle's step (its own exact
selection) at 2e-3, against the step that writes its lists (same library, other kernels), and the kernels that ran."""
import numpy as np
import pytest
import torch

import oracle
from tests.util import announce, bits_of, f32_of, randn_bits, to_dev

pytestmark = pytest.mark.gpu

SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


@pytest.fixture
def hooks():
    """The one-launch form is taken by default from 256 segments on; the cases here have a few segments (the CPU oracle
    checks every one of them) and ask for it through the testing hook, as tests/test_gpu_full_size.py does at 64
    segments of 131072 tokens."""
    from topk_attn_amd import ops

    def set_hooks(**kw):
        kw.setdefault("fused_tail", 1)
        ops.set_test_hooks(**kw)
    set_hooks()
    yield set_hooks
    ops.set_test_hooks()


def _keys(rng, shape, dtype, kind):
    if kind == "levels":      # 16 levels in [-2, 2]: many exact score ties
        return oracle.to_bits(np.linspace(-2, 2, 16)[rng.integers(0, 16, shape)], dtype)
    if kind == "equal":       # every score equal: the cut falls inside one run of ties
        return oracle.to_bits(np.broadcast_to(rng.standard_normal(shape[-1]), shape), dtype)
    x = rng.standard_normal(shape)
    if kind == "heavy":       # 1 % of the keys of every head four times as long
        B, N, H, _ = shape
        for b in range(B):
            for h in range(H):
                x[b, rng.permutation(N)[:N // 100], h] *= 4.0
    if kind == "front":       # the large scores all at the front: slices with hundreds of candidates
        x[:, :shape[1] // 64] *= 3.0
    return oracle.to_bits(x, dtype)


def _run(dtype, B, H, G, N, k, sink, local, kind, out_dtype, seed, expect_redone=0, check_lists=True):
    from topk_attn_amd import ops
    rng = np.random.default_rng(seed)
    q = randn_bits(rng, (B, H * G, 128), dtype)
    K = _keys(rng, (B, N, H, 128), dtype, kind)
    V = randn_bits(rng, (B, N, H, 128), dtype)
    qd, Kd, Vd = to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype)
    plan = ops.SparseDecodePlan(qd, Kd, Vd, k, sink, local, SCALE, G, out_dtype=out_dtype, want_topk=False, want_union=False)
    ops.profile_reset()
    ops.profile_enable(True)
    out = plan.step()
    torch.cuda.synchronize()
    ran = ops.profile_read()
    ops.profile_enable(False)
    redone = plan.redone_segments()
    if N <= 131072:   # up to 256 slices of 512 tokens: one launch selects and attends
        assert "attn_select_mfma" in ran and "lse_combine_redo" in ran and "select_finalize_cand" not in ran, sorted(ran)
    else:             # longer segments keep the selection launch
        assert "select_finalize_cand" in ran and "attn_mfma_indexed" in ran, sorted(ran)
    assert redone == expect_redone, "segments redone from the keys: %d" % redone
    out = f32_of(out)
    bf16_out = out_dtype == torch.bfloat16
    worst = 0.0
    for b in range(B):
        for h in range(H):
            ro, ri, rv, ru = oracle.sparse_decode_step(q[b, h * G:(h + 1) * G], K[b, :, h], V[b, :, h], dtype, G, k, sink,
                                                       local, SCALE)
            tol = 2e-3 + (np.abs(ro) * 2.0 ** -8 if bf16_out else 0.0)
            err = np.abs(out[b, h * G:(h + 1) * G] - ro)
            assert (err < tol).all(), "output against the oracle (b=%d, h=%d): %g" % (b, h, err.max())
            worst = max(worst, float(err.max()))
    if check_lists:   # the step that writes its lists runs other kernels on the same selection
        out2, tidx, tval, uidx, ucnt = ops.sparse_decode_step(qd, Kd, Vd, k, sink, local, SCALE, G, out_dtype=out_dtype)
        torch.cuda.synchronize()
        assert np.abs(f32_of(out2) - out).max() < (1e-3 if not bf16_out else 4e-2)
    print("  worst deviation from the oracle %.2e" % worst, flush=True)
    return plan


@pytest.mark.parametrize("dtype,B,H,G,N,k,sink,local,kind,out_dtype", [
    (oracle.F16, 2, 2, 4, 70000, 2048, 64, 512, "heavy", torch.float16),       # a ragged last slice
    (oracle.F16, 1, 8, 4, 131072, 2048, 64, 512, "heavy", torch.bfloat16),     # the headline shape, one batch entry
    (oracle.BF16, 1, 2, 8, 131072, 4096, 0, 0, "levels", torch.bfloat16),      # ties; no sink range, no window
    (oracle.F16, 1, 2, 2, 70001, 1024, 7, 9, "normal", torch.float16),
    (oracle.BF16, 1, 1, 4, 300000, 2048, 100, 1000, "normal", torch.float16),  # 586 slices: three per thread
    (oracle.F16, 1, 1, 8, 1 << 20, 4096, 64, 512, "levels", torch.float16),    # 2048 slices: eight per thread
    (oracle.F16, 1, 2, 4, 100000, 2048, 64, 512, "equal", torch.float16),      # every token ties: slices filled to the brim
    (oracle.F16, 1, 2, 4, 131072, 2048, 64, 512, "front", torch.float16),      # slices with more candidates than their head holds
    (oracle.F16, 1, 1, 4, 80000, 2048, 30000, 60000, "heavy", torch.float16),  # range and window overlap: nothing in between
    (oracle.F16, 1, 1, 2, 66000, 4000, 0, 1, "normal", torch.float16)])
def test_fused_step_against_oracle(hooks, dtype, B, H, G, N, k, sink, local, kind, out_dtype):
    announce("fused step dtype=%d B=%d H=%d G=%d N=%d k=%d sink=%d local=%d %s" % (dtype, B, H, G, N, k, sink, local, kind))
    _run(dtype, B, H, G, N, k, sink, local, kind, out_dtype, seed=N + k + G)


def test_fused_step_forced_redo(hooks):
    """Every segment flagged (the selection accepts no candidate count): empty partials from the attention launch, all
    rows written by the redo workgroups of the combine launch."""
    announce("fused step, every segment redone from the keys")
    hooks(force_segment_redo=1)
    _run(oracle.F16, 1, 3, 4, 70000, 2048, 64, 512, "heavy", torch.float16, seed=11, expect_redone=3, check_lists=False)
    _run(oracle.BF16, 2, 1, 8, 66000, 1000, 0, 0, "levels", torch.bfloat16, seed=12, expect_redone=2, check_lists=False)


def test_fused_step_threshold_never_published(hooks):
    """The threshold of every other segment is withheld and the wait shortened: the slices of those segments are marked as
    given up, their segments redone from the keys, the others selected inside the attention launch."""
    announce("fused step, thresholds of segments 1, 3 withheld")
    hooks(tau_spin_limit=64, tau_withhold_mod=2, tau_withhold_rem=1, tau_withhold_mode=0)
    _run(oracle.F16, 2, 2, 4, 70000, 2048, 64, 512, "heavy", torch.float16, seed=13, expect_redone=2, check_lists=False)


def test_fused_step_graph_replay(hooks):
    """The step captured in a HIP graph and replayed: the attention launch clears the threshold words and arrival flags
    of its segments, so every replay finds its own."""
    from topk_attn_amd import ops
    announce("fused step in a graph, three replays")
    rng = np.random.default_rng(21)
    dtype, B, H, G, N, k, sink, local = oracle.F16, 1, 2, 4, 70000, 2048, 64, 512
    q = randn_bits(rng, (B, H * G, 128), dtype)
    K = _keys(rng, (B, N, H, 128), dtype, "heavy")
    V = randn_bits(rng, (B, N, H, 128), dtype)
    qd, Kd, Vd = to_dev(q, dtype), to_dev(K, dtype), to_dev(V, dtype)
    plan = ops.SparseDecodePlan(qd, Kd, Vd, k, sink, local, SCALE, G, out_dtype=torch.float16, want_topk=False, want_union=False)
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
        qd.copy_(to_dev(oracle.to_bits(rng.standard_normal((B, H * G, 128)) * (1.0 + 0.5 * it), dtype), dtype))
        plan.step()                  # eager, default stream
        torch.cuda.synchronize()
        want = plan.out.clone()
        plan.out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(plan.out, want), "replay %d: outputs differ" % it
        assert plan.redone_segments() == 0
