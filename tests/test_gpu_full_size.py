"""The configurations the throughput figures are quoted on, at their full sizes, through properties that need no CPU
pass over gigabytes of keys:

* selection: the fused GEMV + top-k (candidate lists, sampled thresholds) must return exactly the first k entries of a
  STABLE descending sort of the plain score vector of the same keys (stable = ties keep the lower index first).  The
  score vector comes from the library's GEMV-only entry point, whose values are pinned bit for bit against the CPU
  oracle in test_gpu_gemv_topk.py at sizes the oracle finishes; the sort is torch's, an independent selection.
* union: ascending, duplicate-free, sink range + selected middle + local window, count = size of that set.
* attention: against a torch fp32 softmax over the union rows of each KV head, within the 2e-3 of the end-to-end
  tests (plus the half-ulp of a bf16 output).
* dense flash-decoding: against torch fp32 attention over all 131 072 tokens, and invariant under the split count.

Beside those properties, two (batch entry, KV head) pairs of every configuration go through the CPU oracle itself at the
full length (a head of 131 072 tokens costs it under a second, one of a million a few): rank-ordered indices and values
and the union list bit for bit, the attention against the fp64 oracle at 2e-3.
"""
import numpy as np
import pytest
import torch

import oracle
from tests.util import announce, bits_of

pytestmark = pytest.mark.gpu

SCALE = float(np.float32(1.0 / np.sqrt(128.0)))


def _randn16(shape, dt, gen, rows_per_chunk=1 << 16):
    """Normal 16-bit tensor [B, N, H, 128] filled chunk by chunk (no fp32 copy of the whole cache)."""
    out = torch.empty(shape, dtype=dt, device="cuda")
    flat = out.view(-1, shape[-2] * shape[-1])
    for r0 in range(0, flat.shape[0], rows_per_chunk):
        r1 = min(r0 + rows_per_chunk, flat.shape[0])
        flat[r0:r1] = torch.randn((r1 - r0, flat.shape[1]), generator=gen, device="cuda").to(dt)
    return out


def _check_selection(scores, idx, val, k):
    """idx/val [B,H,k] against the stable descending sort of scores [B,H,N]; bit-exact."""
    B, H, _ = scores.shape
    for b in range(B):
        sv, si = torch.sort(scores[b], dim=-1, descending=True, stable=True)
        assert torch.equal(idx[b].long(), si[:, :k]), "top-k indices differ from the stable sort (batch entry %d)" % b
        assert torch.equal(val[b].view(torch.int32), sv[:, :k].contiguous().view(torch.int32)), "top-k values differ"


def _oracle_step(q, K, V, b, h, G, dtype, k, sink, local):
    """The CPU oracle's decode step of one (batch entry, KV head) of the GPU tensors q [B,Hq,128], K, V [B,N,H,128]."""
    qb = bits_of(q[b, h * G:(h + 1) * G])
    Kb, Vb = bits_of(K[b, :, h]), bits_of(V[b, :, h])
    return oracle.sparse_decode_step(qb, Kb, Vb, dtype, G, k, sink, local, SCALE)


def _check_against_oracle(pairs, q, K, V, G, dtype, k, sink, local, tidx, tval, uidx, ucnt, outs):
    """Rank-ordered ids and values and the union list bit for bit; every output in `outs` (tensor, tolerance function)."""
    for b, h in pairs:
        announce("  oracle on (batch entry %d, KV head %d), %d tokens" % (b, h, K.shape[1]))
        ro, ri, rv, ru = _oracle_step(q, K, V, b, h, G, dtype, k, sink, local)
        assert np.array_equal(tidx[b, h].cpu().numpy(), ri), "top-k indices differ from the oracle (b=%d, h=%d)" % (b, h)
        assert np.array_equal(tval[b, h].cpu().numpy().view(np.uint32), rv.view(np.uint32)), "top-k values differ from the oracle"
        n = int(ucnt[b, h])
        assert n == len(ru) and np.array_equal(uidx[b, h, :n].cpu().numpy(), ru), "union list differs from the oracle"
        for out, tol in outs:
            got = out[b, h * G:(h + 1) * G].float().cpu().numpy()
            assert (np.abs(got - ro) < tol(ro)).all(), "attention output against the fp64 oracle (b=%d, h=%d): %g" % (
                b, h, np.abs(got - ro).max())


def test_c4_end_to_end_full_size():
    """B=8, 8 KV heads x GQA 4, N=131072 fp16, k=2048, sink 64, local 512, bf16 output; 1% heavy-hitter keys.
    The same step once more with fp16 output, which is held to the 2e-3 without any allowance for the output's rounding."""
    from topk_attn_amd import ops
    B, H, G, N, k, sink, local = 8, 8, 4, 131072, 2048, 64, 512
    announce("full size c4: B=%d Hkv=%d G=%d N=%d k=%d" % (B, H, G, N, k))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(404)
    q = torch.randn((B, H * G, 128), generator=gen, device="cuda").to(torch.float16)
    K = _randn16((B, N, H, 128), torch.float16, gen)
    V = _randn16((B, N, H, 128), torch.float16, gen)
    for b in range(B):
        for h in range(H):
            hh = torch.randperm(N, generator=gen, device="cuda")[:N // 100]
            K[b, hh, h] = (K[b, hh, h].float() * 4.0).to(torch.float16)
    out, tidx, tval, uidx, ucnt = ops.sparse_decode_step(q, K, V, k, sink, local, SCALE, G, out_dtype=torch.bfloat16)
    out16, tidx16, tval16, uidx16, ucnt16 = ops.sparse_decode_step(q, K, V, k, sink, local, SCALE, G, out_dtype=torch.float16)
    # and for a caller that asks for the output alone, with selection and attention in one launch (the rule takes that
    # form from 256 segments on; the hook takes it here)
    plan_out = ops.SparseDecodePlan(q, K, V, k, sink, local, SCALE, G, out_dtype=torch.float16, want_topk=False, want_union=False)
    ops.set_test_hooks(fused_tail=1)
    try:
        ops.profile_reset()
        ops.profile_enable(True)
        out_only = plan_out.step()
        torch.cuda.synchronize()
        ran = ops.profile_read()
        ops.profile_enable(False)
        redone_only = plan_out.redone_segments()
    finally:
        ops.set_test_hooks()
    assert "attn_select_mfma" in ran and "lse_combine_redo" in ran and "select_finalize_cand" not in ran, sorted(ran)
    assert redone_only == 0
    scores = ops.gemv_scores(q, K, group=G, scale=SCALE)
    torch.cuda.synchronize()
    _check_selection(scores, tidx, tval, k)
    assert torch.equal(tidx, tidx16) and torch.equal(uidx, uidx16) and torch.equal(ucnt, ucnt16)
    _check_against_oracle([(0, 0), (B - 1, H - 1)], q, K, V, G, oracle.F16, k, sink, local, tidx, tval, uidx, ucnt,
                          [(out, lambda r: 2e-3 + np.abs(r) * 2.0 ** -8), (out16, lambda r: 2e-3), (out_only, lambda r: 2e-3)])

    lo, hi = sink, N - local
    edge = torch.cat([torch.arange(lo, device="cuda"), torch.arange(hi, N, device="cuda")])
    worst = worst16 = 0.0
    for b in range(B):
        for h in range(H):
            sel = tidx[b, h].long()
            want = torch.unique(torch.cat([edge, sel]))          # sorted ascending, duplicate-free
            n = int(ucnt[b, h])
            assert n == want.numel(), "union count"
            assert torch.equal(uidx[b, h, :n].long(), want), "union list"
            ks, vs = K[b, want, h].float(), V[b, want, h].float()
            logits = (q[b, h * G:(h + 1) * G].float() @ ks.T) * SCALE
            ref = torch.softmax(logits, dim=-1) @ vs
            got = out[b, h * G:(h + 1) * G].float()
            tol = 2e-3 + ref.abs() * 2.0 ** -8                   # bf16 output: its own rounding on top
            assert bool(((got - ref).abs() < tol).all()), "attention output (b=%d, h=%d)" % (b, h)
            worst = max(worst, float((got - ref).abs().max()))
            err16 = float((out16[b, h * G:(h + 1) * G].float() - ref).abs().max())
            assert err16 < 2e-3, "attention output, fp16 (b=%d, h=%d): %g" % (b, h, err16)
            worst16 = max(worst16, err16)
            err_only = float((out_only[b, h * G:(h + 1) * G].float() - ref).abs().max())
            assert err_only < 2e-3, "attention output of the one-launch form (b=%d, h=%d): %g" % (b, h, err_only)
    print("c4 full size: worst attention error %.2e (bf16 output), %.2e (fp16 output, strict 2e-3)" % (worst, worst16), flush=True)


def test_c4_shared_cache_full_size():
    """c4's shapes over ONE cache that the batch shares (kv_stride_b = 0), where one pass over the keys scores the eight
    batch entries: the step must give, bit for bit in its lists and its output, what it gives when every batch entry
    holds its own copy of that cache (the per-entry kernels, pinned above) - and one (batch entry, KV head) pair goes through
    the CPU oracle as well."""
    from topk_attn_amd import ops
    announce("c4 over a shared cache: B=8 Hq=32 Hkv=8 N=131072 fp16 k=2048, against per-entry copies of the cache")
    B, H, G, N, k, sink, local = 8, 8, 4, 131072, 2048, 64, 512
    gen = torch.Generator(device="cuda")
    gen.manual_seed(404)
    dt = torch.float16
    q = torch.randn((B, H * G, 128), generator=gen, device="cuda").to(dt)
    K1 = _randn16((1, N, H, 128), dt, gen)
    V1 = _randn16((1, N, H, 128), dt, gen)
    for h in range(H):
        hh = torch.randperm(N, generator=gen, device="cuda")[:N // 100]
        K1[0, hh, h] = (K1[0, hh, h].float() * 4.0).to(dt)
    shared = ops.SparseDecodePlan(q, K1[0], V1[0], k, sink, local, SCALE, G, out_dtype=torch.float16)
    ops.profile_reset()
    ops.profile_enable(True)
    shared.step()
    torch.cuda.synchronize()
    ran = ops.profile_read()
    ops.profile_enable(False)
    assert "gemv_candidates_shared" in ran, sorted(ran)
    assert shared.redone_segments() == 0
    Kb, Vb = K1.expand(B, N, H, 128).contiguous(), V1.expand(B, N, H, 128).contiguous()
    own = ops.SparseDecodePlan(q, Kb, Vb, k, sink, local, SCALE, G, out_dtype=torch.float16)
    own.step()
    torch.cuda.synchronize()
    assert torch.equal(shared.topk_idx, own.topk_idx) and torch.equal(shared.topk_val.view(torch.int32), own.topk_val.view(torch.int32))
    assert torch.equal(shared.union_count, own.union_count) and torch.equal(shared.union_idx, own.union_idx)
    assert torch.equal(shared.out, own.out), "outputs differ: %g" % (shared.out.float() - own.out.float()).abs().max().item()
    _check_against_oracle([(B - 1, 3)], q, Kb, Vb, G, oracle.F16, k, sink, local, shared.topk_idx, shared.topk_val, shared.union_idx,
                          shared.union_count, [(shared.out, lambda ro: 2e-3)])


def _levels16(shape, dt, gen):
    levels = torch.linspace(-2, 2, 16, device="cuda")
    out = torch.empty(shape, dtype=dt, device="cuda")
    flat = out.view(-1, shape[-2] * shape[-1])
    for r0 in range(0, flat.shape[0], 1 << 16):
        r1 = min(r0 + (1 << 16), flat.shape[0])
        flat[r0:r1] = levels[torch.randint(0, 16, (r1 - r0, flat.shape[1]), generator=gen, device="cuda")].to(dt)
    return out


@pytest.mark.parametrize("pool", [0, 4096])
def test_c5_tie_stress_full_size(pool):
    """8 KV heads x GQA 8, N=1048576 bf16 keys on 16 levels, k=4096, attention over the selected tokens.
    pool=0: every key row drawn independently (exact ties between scores wherever the level sums coincide).
    pool=4096: the rows are drawn from 4096 distinct ones, so every score is shared by about 256 tokens and the cut
    at rank k falls inside a run of equal scores on every head: the lower token index must win throughout."""
    from topk_attn_amd import ops
    H, G, N, k = 8, 8, 1 << 20, 4096
    announce("full size c5: Hkv=%d G=%d N=%d k=%d bf16 levels, row pool %d" % (H, G, N, k, pool))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(505 + pool)
    if pool:
        rows = _levels16((1, pool, H, 128), torch.bfloat16, gen)[0]
        K = rows[torch.randint(0, pool, (N,), generator=gen, device="cuda")].unsqueeze(0).contiguous()
    else:
        K = _levels16((1, N, H, 128), torch.bfloat16, gen)
    V = _randn16((1, N, H, 128), torch.bfloat16, gen)
    q = torch.randn((1, H * G, 128), generator=gen, device="cuda").to(torch.bfloat16)
    plan = ops.SparseDecodePlan(q, K, V, k, 0, 0, SCALE, G, out_dtype=torch.bfloat16)
    out = plan.step()
    scores = ops.gemv_scores(q, K, group=G, scale=SCALE)
    torch.cuda.synchronize()
    _check_selection(scores, plan.topk_idx, plan.topk_val, k)
    _check_against_oracle([(0, 0), (0, H - 1)], q, K, V, G, oracle.BF16, k, 0, 0, plan.topk_idx, plan.topk_val,
                          plan.union_idx, plan.union_count, [(out, lambda r: 2e-3 + np.abs(r) * 2.0 ** -8)])
    kth = plan.topk_val[0, :, k - 1]
    ties = (scores[0] == kth[:, None]).sum(dim=1)
    print("c5 full size (pool %d): tokens sharing the k-th score per head: %s" % (pool, ties.tolist()), flush=True)
    if pool:
        assert bool((ties >= 2).all()), "the cut does not fall inside a run of equal scores"
    for h in range(H):
        want = torch.sort(plan.topk_idx[0, h].long()).values
        assert int(plan.union_count[0, h]) == k and torch.equal(plan.union_idx[0, h, :k].long(), want), "union list"
        logits = (q[0, h * G:(h + 1) * G].float() @ K[0, want, h].float().T) * SCALE
        ref = torch.softmax(logits, dim=-1) @ V[0, want, h].float()
        got = out[0, h * G:(h + 1) * G].float()
        assert bool(((got - ref).abs() < 2e-3 + ref.abs() * 2.0 ** -8).all()), "attention output (h=%d)" % h


def test_threshold_published_late_some_slices_give_up():
    """Four segments of a million tokens (2048 candidate slices each, twice what the GPU holds at once).  The
    threshold of segment 2 is withheld until the first of its streaming workgroups has run out of its (shortened)
    wait: the first slices of the segment are marked as given up, the later ones see the threshold and store
    their candidates - more than k of them, which the selection kernel used to accept.  The marked slices force
    the segment to be redone from the keys; the other three segments keep the candidate route; the result is the
    stable sort's for every segment, and every kernel runs to its end."""
    from topk_attn_amd import ops
    H, N, k = 4, 1 << 20, 4096
    announce("full size: threshold of one of %d segments of %d tokens published late (k=%d)" % (H, N, k))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(606)
    K = _randn16((1, N, H, 128), torch.float16, gen)
    q = torch.randn((1, H, 128), generator=gen, device="cuda").to(torch.float16)
    ops.set_test_hooks(tau_spin_limit=64, tau_withhold_mod=4, tau_withhold_rem=2, tau_withhold_mode=1)
    try:
        plan = ops.GemvTopkPlan(q, K, k, group=1, scale=SCALE).run()
        torch.cuda.synchronize()
        redone, gave_up = plan.redone_segments(), plan.gave_up_slices()
    finally:
        ops.set_test_hooks()
    print("late threshold: %d segment(s) redone, %d of 2048 slices gave up" % (redone, gave_up), flush=True)
    scores = ops.gemv_scores(q, K, group=1, scale=SCALE)
    torch.cuda.synchronize()
    _check_selection(scores, plan.idx, plan.val, k)
    assert redone == 1
    assert 0 < gave_up < 2048, "the case meant here is a segment with SOME slices given up"
    plan.run()                                     # the same plan with the hooks off again: nothing is redone
    torch.cuda.synchronize()
    assert plan.redone_segments() == 0 and plan.gave_up_slices() == 0
    _check_selection(scores, plan.idx, plan.val, k)


def test_c3_dense_flash_decode_full_size():
    """32 query heads over 8 KV heads, N=131072 fp16: against torch fp32 attention, and across split counts."""
    from topk_attn_amd import ops
    B, H, G, N = 1, 8, 4, 131072
    announce("full size c3: Hq=%d Hkv=%d N=%d dense flash-decoding" % (H * G, H, N))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(303)
    q = torch.randn((B, H * G, 128), generator=gen, device="cuda").to(torch.float16)
    K = _randn16((B, N, H, 128), torch.float16, gen)
    V = _randn16((B, N, H, 128), torch.float16, gen)
    out = ops.flash_decode(q, K, V, SCALE, group=G)
    out_1 = ops.flash_decode(q, K, V, SCALE, group=G, num_splits=1)
    out_37 = ops.flash_decode(q, K, V, SCALE, group=G, num_splits=37)
    torch.cuda.synchronize()
    for h in range(H):
        logits = (q[0, h * G:(h + 1) * G].float() @ K[0, :, h].float().T) * SCALE
        ref = torch.softmax(logits, dim=-1) @ V[0, :, h].float()
        for o in (out, out_1, out_37):
            assert float((o[0, h * G:(h + 1) * G].float() - ref).abs().max()) < 2e-3
    for h in (0, H - 1):       # the fp64 oracle on two KV heads, all 131072 tokens
        announce("  oracle on KV head %d, %d tokens" % (h, N))
        Kb, Vb = bits_of(K[0, :, h]), bits_of(V[0, :, h])
        for g in range(G):
            ref, _ = oracle.attention_f64(bits_of(q[0, h * G + g]), Kb, Vb, oracle.F16, scale=SCALE)
            for o in (out, out_1, out_37):
                assert np.abs(o[0, h * G + g].float().cpu().numpy() - ref).max() < 2e-3


def test_dense_flash_decode_sixteen_heads_full_size():
    """Sixteen KV heads over 131072 tokens: a head's rows lie 4 KB apart and the cache of one batch entry is half a
    gigabyte, so the matrix-core kernel's grid counts the heads in x and the splits in y.  Against torch fp32
    attention (tolerance 2e-3), and across split counts."""
    from topk_attn_amd import ops
    B, H, G, N = 1, 16, 2, 131072
    announce("full size: Hq=%d Hkv=%d N=%d dense flash-decoding, heads in the grid's x" % (H * G, H, N))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(304)
    q = torch.randn((B, H * G, 128), generator=gen, device="cuda").to(torch.float16)
    K = _randn16((B, N, H, 128), torch.float16, gen)
    V = _randn16((B, N, H, 128), torch.float16, gen)
    out = ops.flash_decode(q, K, V, SCALE, group=G)
    out_5 = ops.flash_decode(q, K, V, SCALE, group=G, num_splits=5)
    torch.cuda.synchronize()
    for h in range(H):
        logits = (q[0, h * G:(h + 1) * G].float() @ K[0, :, h].float().T) * SCALE
        ref = torch.softmax(logits, dim=-1) @ V[0, :, h].float()
        for o in (out, out_5):
            assert float((o[0, h * G:(h + 1) * G].float() - ref).abs().max()) < 2e-3
