#!/usr/bin/env python3
"""Benchmark of the sparse-decode path on one MI355X.

A step = one pass of the hot path over one batch of seeded synthetic input, inputs resident in HBM.
The default workload is the one the headline metric is quoted on:

  c4  end-to-end decode at 128k: batch 8, 32 query / 8 KV heads, head_dim 128, KV length 131072 fp16 N(0,1)
      with 1% of the keys per head scaled x4; fused GEMV + top-2048 per KV head -> union with 64 sink + 512
      local tokens -> gathered attention -> LSE combine; bf16 output.

The other workloads time one stage each at the sizes of the remaining configurations (c1 single-head
GEMV + top-k, c2 centre-only top-k, c3 dense flash-decoding, c5 one-million-token tie stress); `ra` times
the reference's operator at its own test shape (--batch, --topk).

Prints ONE JSON line.  `value` is algorithmic bytes per step / step time (GB/s); `roofline` is the dominant
kernel timed with HIP events on its launch stream; `cpu_baseline` is the torch-CPU restatement of the same
step timed on this machine's host cores on a bounded sample (c4 only).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
SCALE = 0.08838834764831845  # fl32(1/sqrt(128)) as Python float


def randn16(torch, shape, dt, g, dev, chunk_dim0=True):
    """N(0,1) tensor of a 16-bit type, generated slice by slice to bound the fp32 temporaries."""
    out = torch.empty(shape, device=dev, dtype=dt)
    if len(shape) >= 3 and shape[0] > 1 and chunk_dim0:
        for i in range(shape[0]):
            out[i] = torch.randn(shape[1:], generator=g, device=dev, dtype=torch.float32).to(dt)
    else:
        step = max(1, (1 << 26) // max(1, int(out[0].numel()))) if out.dim() > 1 else out.numel()
        if out.dim() == 1:
            out.copy_(torch.randn(shape, generator=g, device=dev, dtype=torch.float32).to(dt))
        else:
            for i in range(0, shape[0], step):
                j = min(shape[0], i + step)
                out[i:j] = torch.randn((j - i,) + tuple(shape[1:]), generator=g, device=dev, dtype=torch.float32).to(dt)
    return out


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def levels16(torch, shape, dt, g, dev):
    """[B, N, H, 128] tensor whose entries take 16 uniform levels in [-2, 2], generated in slices of 131072 tokens."""
    out = torch.empty(shape, device=dev, dtype=dt)
    lv = torch.linspace(-2.0, 2.0, 16, device=dev)
    for b in range(shape[0]):
        for t0 in range(0, shape[1], 131072):
            t1 = min(shape[1], t0 + 131072)
            ids = torch.randint(0, 16, (t1 - t0,) + tuple(shape[2:]), generator=g, device=dev)
            out[b, t0:t1] = lv[ids].to(dt)
    return out


class SparseDecode:
    """c4 (and a small variant): the end-to-end step."""

    def __init__(self, torch, ops, dev, batch=8, hkv=8, group=4, seq_len=131072, k=2048, sink=64, local=512,
                 dtype="float16", out_dtype="bfloat16", heavy=0.01, seed=4, name="c4", num_splits=0, levels=False,
                 want_union=True, shared=False):
        self.torch, self.name = torch, name
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        dt = getattr(torch, dtype)
        B, H, G, N = batch, hkv, group, seq_len
        self.B, self.H, self.G, self.N, self.k, self.sink, self.local = B, H, G, N, k, sink, local
        self.q = randn16(torch, (B, H * G, 128), dt, g, dev, chunk_dim0=False)
        self.shared = shared
        KB = 1 if shared else B       # shared: one cache [N, H, 128] for all batch entries (kv_stride_b = 0)
        if levels:  # 16 uniform levels in [-2, 2]: many exact score ties
            self.K = levels16(torch, (KB, N, H, 128), dt, g, dev)
        else:
            self.K = randn16(torch, (KB, N, H, 128), dt, g, dev)
        self.V = randn16(torch, (KB, N, H, 128), dt, g, dev)
        n_heavy = int(N * heavy)
        for b in range(KB):
            for h in range(H):
                hh = torch.randperm(N, generator=g, device=dev)[:n_heavy]
                self.K[b, hh, h] = (self.K[b, hh, h].float() * 4.0).to(dt)
        if shared:
            self.K, self.V = self.K[0], self.V[0]
        # production configuration: the attention consumes the union list; the optional rank-ordered top-k
        # output (a sort per KV head) is not requested
        self.plan = ops.SparseDecodePlan(self.q, self.K, self.V, k, sink, local, SCALE, G,
                                         out_dtype=getattr(torch, out_dtype), num_splits=num_splits, want_topk=False)
        self.selected = None
        if not want_union:
            # the caller that only wants the attention output: the step hands its token list on in the order of its route;
            # the size of the list (for the byte count) comes from one step of the plan above
            self.plan.step()
            self.selected = int(self.plan.union_count.sum().item())
            self.plan = ops.SparseDecodePlan(self.q, self.K, self.V, k, sink, local, SCALE, G, out_dtype=getattr(torch, out_dtype),
                                             num_splits=num_splits, want_topk=False, want_union=False)
        self.desc = "%s: B=%d Hq=%d Hkv=%d D=128 N=%d %s k=%d sink=%d local=%d out=%s" % (
            name, B, H * G, H, N, dtype, k, sink, local, out_dtype)
        self.dominant = "gemv_scores"
        self.hooks = {}            # testing hooks the workload runs under (kept when the worst case adds its own)
        self.make_rank_plan = None
        if want_union:             # the same step with the rank-ordered top-k output as well (a sort per KV head)
            self.make_rank_plan = lambda: ops.SparseDecodePlan(self.q, self.K, self.V, k, sink, local, SCALE, G,
                                                               out_dtype=getattr(torch, out_dtype), num_splits=num_splits, want_topk=True)

    def step(self):
        self.plan.step()

    def redone_segments(self):
        return self.plan.redone_segments()

    def bytes(self):
        sel = self.selected if self.selected is not None else int(self.plan.union_count.sum().item())
        gemv = (1 if self.shared else self.B) * self.N * self.H * 128 * 2   # a shared cache is streamed once for the batch
        sparse = sel * 128 * 2 * 2 + sel * 4 * 2          # gathered K and V rows, index lists written + read
        qo = self.B * self.H * self.G * 128 * 4           # q read, out written (2 bytes each)
        return gemv + sparse + qo, gemv, {"selected_tokens": sel}

    def cpu_baseline(self, runs):
        torch = self.torch
        from oracle.cpu_baseline import sparse_decode_cpu
        # bounded sample: batch entry 0 (1/B of the step); the step is B independent copies of it
        qc, Kc, Vc = self.q[0].cpu(), (self.K if self.shared else self.K[0]).cpu(), (self.V if self.shared else self.V[0]).cpu()
        times = []
        for r in range(runs + 2):   # two warm-ups, then the timed runs
            c0 = time.perf_counter()
            ref_out, ref_top = sparse_decode_cpu(qc, Kc, Vc, self.k, self.sink, self.local, SCALE, self.G)
            c1 = time.perf_counter()
            if r >= 2:
                times.append(c1 - c0)
        times.sort()
        cpu_s = times[len(times) // 2] * self.B
        # sanity (not the parity oracle): same selected sets, outputs close
        N, H = self.N, self.H
        lo, hi = min(self.sink, N), max(N - self.local, min(self.sink, N))
        same_sets = None   # (a plan that is not asked for the list has none to compare)
        for h in range(H if self.plan.union_idx is not None else 0):
            want = set(range(lo)) | set(range(hi, N)) | set(ref_top[h].tolist())
            got = self.plan.union_idx[0, h, :int(self.plan.union_count[0, h])].tolist()
            same_sets = same_sets is not False and got == sorted(want)
        max_err = (self.plan.out[0].float().cpu() - ref_out).abs().max().item()
        return cpu_s, {"cores": torch.get_num_threads(), "host_cpus": os.cpu_count(), "cpu_model": cpu_model(), "kind": "port",
                       "sample": "batch entry 0 of %d (all %d KV heads, full N=%d), median of %d runs, scaled x%d" % (
                           self.B, H, N, runs, self.B),
                       "union_sets_equal_gpu": same_sets, "out_max_abs_diff_vs_gpu": round(max_err, 5)}


class GemvTopk:
    """c1 / c5: fused GEMV + top-k alone."""

    def __init__(self, torch, ops, dev, batch, hkv, group, seq_len, k, dtype, seed, name, levels=False, rotate=0):
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        dt = getattr(torch, dtype)
        self.B, self.H, self.G, self.N, self.k = batch, hkv, group, seq_len, k
        self.q = randn16(torch, (batch, hkv * group, 128), dt, g, dev, chunk_dim0=False)
        if levels:  # 16 uniform levels in [-2, 2]: many exact score ties
            self.K = levels16(torch, (batch, seq_len, hkv, 128), dt, g, dev)
        else:
            self.K = randn16(torch, (batch, seq_len, hkv, 128), dt, g, dev)
        # rotate > 0: that many copies of the keys, one plan each, taken in turn, so that a key set much smaller
        # than the Infinity Cache is read from HBM every step
        self.plans = [ops.GemvTopkPlan(self.q, self.K, k, group=group, scale=SCALE)]
        self.copies = [self.K.clone() for _ in range(max(rotate - 1, 0))]
        self.plans += [ops.GemvTopkPlan(self.q, Kc, k, group=group, scale=SCALE) for Kc in self.copies]
        self.turn = 0
        self.desc = "%s: B=%d Hkv=%d G=%d D=128 N=%d %s k=%d (GEMV + top-k only)%s" % (
            name, batch, hkv, group, seq_len, dtype, k, ", %d rotating key sets" % rotate if rotate > 1 else "")
        self.dominant = "gemv_scores"
        self.hooks = {}

    def step(self):
        self.plans[self.turn % len(self.plans)].run()
        self.turn += 1

    def redone_segments(self):
        return self.plans[(self.turn - 1) % len(self.plans)].redone_segments()

    def bytes(self):
        gemv = self.B * self.N * self.H * 128 * 2
        return gemv + self.B * self.H * self.G * 128 * 2 + self.B * self.H * self.k * 8, gemv, {}


class CenterTopk:
    """c2: centre-only top-k with expansion."""

    def __init__(self, torch, ops, dev, centroids=4096, expand=64, rotate=0):
        g = torch.Generator(device=dev)
        g.manual_seed(2)
        H, Cn = 32, centroids
        self.ops, self.H, self.Cn, self.top_c, self.clen = ops, H, Cn, 64, expand
        cen = torch.randn((H, Cn, 128), generator=g, device=dev) + 0.5 * torch.randn((H, 1, 128), generator=g, device=dev)
        self.cen = cen.half()
        self.q = torch.randn((H, 128), generator=g, device=dev).half()
        self.plans = [ops.CenterTopkPlan(self.q, self.cen, self.top_c, self.clen, SCALE)]
        self.copies = [self.cen.clone() for _ in range(max(rotate - 1, 0))]
        self.plans += [ops.CenterTopkPlan(self.q, c, self.top_c, self.clen, SCALE) for c in self.copies]
        self.turn = 0
        self.desc = "c2: 32 heads x %d centroids fp16, top-64, expand x%d%s" % (
            Cn, expand, ", %d rotating centroid sets" % rotate if rotate > 1 else "")
        self.dominant = "gemv_scores"

    def step(self):
        self.plans[self.turn % len(self.plans)].run()
        self.turn += 1

    def bytes(self):
        gemv = self.H * self.Cn * 128 * 2
        return gemv + self.H * 128 * 2 + self.H * self.top_c * self.clen * 4, gemv, {}


class FlashDecode:
    """c3: dense split-K flash-decoding."""

    def __init__(self, torch, ops, dev, num_splits=0):
        g = torch.Generator(device=dev)
        g.manual_seed(3)
        self.H, self.G, self.N = 8, 4, 131072
        self.q = randn16(torch, (1, 32, 128), torch.float16, g, dev, chunk_dim0=False)
        self.K = randn16(torch, (self.N, 8, 128), torch.float16, g, dev, chunk_dim0=False)
        self.V = randn16(torch, (self.N, 8, 128), torch.float16, g, dev, chunk_dim0=False)
        self.plan = ops.FlashDecodePlan(self.q, self.K, self.V, SCALE, group=4, num_splits=num_splits)
        self.desc = "c3: dense flash-decoding B=1 Hq=32 Hkv=8 D=128 N=131072 fp16, splits=%s" % (num_splits or "auto")
        self.dominant = "attn_mfma_dense"

    def step(self):
        self.plan.run()

    def bytes(self):
        kv = 2 * self.N * self.H * 128 * 2
        return kv + 2 * 32 * 128 * 2, kv, {}


class RetrievalOp:
    """ra: the reference's operator at its own test shape (test_ra.py:162-172: 32 heads, 8192 keys shared by the
    batch, 4 chunks of 2048, top-K per chunk), batch entries and K selectable."""

    def __init__(self, torch, dev, batch=4, topk=128, rotate=0, score_mode=0):
        from topk_attn_amd import retrieval_attention_cpp as ra
        g = torch.Generator(device=dev)
        g.manual_seed(6)
        self.B, self.topk = batch, topk
        self.q = (torch.randn((batch, 32, 128), generator=g, device=dev) * 0.1).half()
        K = (torch.randn((8192, 32, 128), generator=g, device=dev) * 0.1).half()
        V = (torch.randn((8192, 32, 128), generator=g, device=dev) * 0.1).half()
        # rotate > 1: that many copies of the caches taken in turn, so that they come from HBM, not the Infinity Cache
        self.kv = [(K, V)] + [(K.clone(), V.clone()) for _ in range(max(rotate - 1, 0))]
        self.turn = 0
        self.out = torch.zeros((batch, 32, 128), dtype=torch.float16, device=dev)
        self.score_mode = score_mode
        self.fn = lambda q, K, V, out: ra.retrieval_attention(q, K, V, out, topk, score_mode=score_mode)
        self.desc = "ra: retrieval_attention_%d, B=%d, 32 heads, 8192 keys fp16 shared by the batch%s%s" % (
            topk, batch, ", %d rotating cache copies" % rotate if rotate > 1 else "",
            ", scores on the matrix cores" if score_mode else "")
        self.dominant = ("gemv_scores_mfma" if score_mode else "gemv_scores_shared") if batch >= 2 else "gemv_scores"

    def step(self):
        K, V = self.kv[self.turn % len(self.kv)]
        self.turn += 1
        self.fn(self.q, K, V, self.out)

    def bytes(self):
        keys = 8192 * 32 * 128 * 2                               # read once for the whole batch
        rows = self.B * 32 * 4 * self.topk * 128 * 2             # gathered V rows
        return keys + rows + 2 * self.B * 32 * 128 * 2, keys, {}


class PlainCopy:
    """Calibration workload for the HBM traffic counters: a device-to-device copy of known size."""

    def __init__(self, torch, dev, nbytes=1 << 30):
        self.src = torch.ones(nbytes // 2, dtype=torch.float16, device=dev)
        self.dst = torch.empty_like(self.src)
        self.nbytes = nbytes
        self.desc = "copy: %d bytes read + %d bytes written per step" % (nbytes, nbytes)
        self.dominant = "(torch copy kernel)"

    def step(self):
        self.dst.copy_(self.src)

    def bytes(self):
        return 2 * self.nbytes, 2 * self.nbytes, {}


class ReadProbes:
    """probe-stream / probe-gather: kernels that only read, in the access patterns of the two kernels that carry the
    bytes of the c4 step (the long-segment GEMV: rows of 256 B of one head per workgroup; the gathered attention: the K
    and V rows of 2624 tokens per (batch entry, KV head) at random places)."""

    def __init__(self, torch, ops, dev, kind, threads, rounds):
        g = torch.Generator(device=dev)
        g.manual_seed(8)
        B, N, H = 8, 131072, 8
        self.K = torch.ones((B, N, H, 128), dtype=torch.float16, device=dev)
        if kind == "gather":
            self.V = torch.ones((B, N, H, 128), dtype=torch.float16, device=dev)
            L = 2624
            idx = torch.stack([torch.randperm(N, generator=g, device=dev)[:L] for _ in range(B * H)]).view(B, H, L)
            idx = idx.sort(dim=-1).values.to(torch.int32).contiguous()       # ascending, like the union list
            self.probe = ops.ReadProbe(self.K, self.V, idx, tokens_per_wg=256)
            self.nbytes = B * H * L * 512
            self.desc = "probe-gather: K and V rows of %d tokens per (batch entry, KV head), B=%d Hkv=%d N=%d" % (L, B, H, N)
            self.dominant = "probe_gather"
        else:
            self.probe = ops.ReadProbe(self.K, threads=threads, rounds=rounds)
            self.nbytes = B * N * H * 256
            self.desc = "probe-stream: B=%d N=%d Hkv=%d, %d threads x %d rounds of 8 loads per lane" % (B, N, H, threads, rounds)
            self.dominant = "probe_stream"

    def step(self):
        self.probe.run()

    def bytes(self):
        return self.nbytes, self.nbytes, {}


def build_workload(name, torch, ops, dev, args):
    if name == "probe-stream":
        return ReadProbes(torch, ops, dev, "stream", args.probe_threads, args.probe_rounds)
    if name == "probe-gather":
        return ReadProbes(torch, ops, dev, "gather", 0, 0)
    if name == "copy":
        return PlainCopy(torch, dev)
    if name == "c4":
        return SparseDecode(torch, ops, dev, num_splits=args.splits)
    if name == "c4-shared":     # the same shapes over ONE cache that the batch shares (a common prefix: kv_stride_b = 0)
        return SparseDecode(torch, ops, dev, num_splits=args.splits, name="c4-shared", shared=True)
    if name == "c4-out":        # the same step for a caller that wants the output alone
        return SparseDecode(torch, ops, dev, num_splits=args.splits, name="c4-out", want_union=False)
    if name == "c4-one-launch":  # ... with selection and attention in one launch (the library takes that form from 256 segments on)
        ops.set_test_hooks(fused_tail=1)
        w = SparseDecode(torch, ops, dev, num_splits=args.splits, name="c4-one-launch", want_union=False)
        w.hooks = {"fused_tail": 1}
        return w
    if name == "c4-small":
        return SparseDecode(torch, ops, dev, batch=2, seq_len=16384, name="c4-small")
    if name == "c4-b1-32k":     # one sequence of 32768 tokens on one GPU (all 8 KV heads), output only
        return SparseDecode(torch, ops, dev, batch=1, seq_len=32768, name="c4-b1-32k", want_union=False)
    if name == "c4-share32k":   # one GPU's share of an 8-way head-sharded model, one sequence of 32768 tokens, output only
        return SparseDecode(torch, ops, dev, batch=1, hkv=1, group=8, seq_len=32768, name="c4-share32k", want_union=False)
    if name == "c4-b1-16k":     # the same at 16384 tokens: segments that would also fit the registers of one workgroup
        return SparseDecode(torch, ops, dev, batch=1, seq_len=16384, k=1024, name="c4-b1-16k", want_union=False)
    if name == "c1":
        return GemvTopk(torch, ops, dev, 1, 1, 1, 32768, 2048, "float16", 1, "c1", rotate=args.rotate)
    if name == "c1-8x16k":      # rank-ordered top-k of eight heads of 16384 keys
        return GemvTopk(torch, ops, dev, 1, 8, 1, 16384, 1024, "float16", 1, "c1-8x16k", rotate=args.rotate)
    if name == "c2":
        return CenterTopk(torch, ops, dev, rotate=args.rotate)
    if name == "c2-ref":   # the problem of the reference's recorded latencies (center_only_topk/gemv_topk.cu:2-7)
        return CenterTopk(torch, ops, dev, centroids=1024, expand=128, rotate=args.rotate)
    if name == "c3":
        return FlashDecode(torch, ops, dev, args.splits)
    if name == "ra":
        return RetrievalOp(torch, dev, batch=args.batch, topk=args.topk, rotate=args.rotate, score_mode=args.score_mode)
    if name == "c5":       # the tie-stress step: selection under exact ties at 1M tokens, attention over the selected tokens
        return SparseDecode(torch, ops, dev, batch=1, hkv=8, group=8, seq_len=1048576, k=4096, sink=0, local=0,
                            dtype="bfloat16", heavy=0.0, seed=5, name="c5", levels=True)
    if name == "c5-out":   # the same step for a caller that wants the output alone
        return SparseDecode(torch, ops, dev, batch=1, hkv=8, group=8, seq_len=1048576, k=4096, sink=0, local=0,
                            dtype="bfloat16", heavy=0.0, seed=5, name="c5-out", levels=True, want_union=False)
    if name == "c5-topk":  # its selection stage alone, rank-ordered output
        return GemvTopk(torch, ops, dev, 1, 8, 8, 1048576, 4096, "bfloat16", 5, "c5-topk", levels=True)
    raise ValueError(name)


# HBM bytes per launch of the dominant kernel, from rocprofv3 counter runs of this file's default configurations
# (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, the factors a plain copy of known size gives on this part).
# The counters cannot be read from inside the process, so the figures are recorded here with the file that holds
# the counter run and the digest of the kernel's source at the time of that run: a figure is only reported
# while the source still has that digest.
RECORDED_TRAFFIC = {
    ("c4", "gemv_candidates"): {"bytes": 2189277696,   # 2 x 1066292.4 KiB + 5381.7 KiB
                                "source": "profiles/gemv_candidates_c4.md",
                                "kernel_source": "topk_attn_amd/csrc/gemv_scores.hip",
                                "kernel_source_sha16": "74ccf271f9b5266a"},
}


def recorded_traffic(workload, kernel):
    """(bytes or None, note) for roofline.traffic / roofline.traffic_source."""
    import hashlib
    rec = RECORDED_TRAFFIC.get((workload, kernel))
    if rec is None:
        return None, None
    try:
        with open(os.path.join(ROOT, rec["kernel_source"]), "rb") as f:
            sha = hashlib.sha256(f.read()).hexdigest()[:16]
    except OSError:
        sha = None
    if sha != rec["kernel_source_sha16"]:
        return None, "%s is older than the kernel's source (recorded for %s, now %s): not reported" % (
            rec["source"], rec["kernel_source_sha16"], sha)
    return rec["bytes"], "%s (rocprofv3 counter runs, recorded; kernel source %s)" % (rec["source"], sha)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c4", choices=["c1", "c1-8x16k", "c2", "c2-ref", "c3", "c4", "c4-out", "c4-one-launch", "c4-shared", "c4-small", "c4-b1-32k", "c4-b1-16k", "c4-share32k", "c5", "c5-out", "c5-topk", "ra", "copy",
                                                       "probe-stream", "probe-gather"])
    ap.add_argument("--batch", type=int, default=4, help="ra: batch entries")
    ap.add_argument("--topk", type=int, default=128, choices=[32, 128, 256, 512, 1024], help="ra: K per chunk")
    ap.add_argument("--score-mode", type=int, default=0, choices=[0, 1],
                    help="ra: 1 = scores on the matrix cores (tka_score_mode), 0 = the canonical order")
    ap.add_argument("--splits", type=int, default=0, help="c3, c4: split count of the attention (0 = library default)")
    ap.add_argument("--rotate", type=int, default=0,
                    help="c1, c2, c2-ref, ra: number of key sets taken in turn (working set beyond the Infinity Cache)")
    ap.add_argument("--probe-threads", type=int, default=512, choices=[256, 512], help="probe-stream: threads per workgroup")
    ap.add_argument("--probe-rounds", type=int, default=2, help="probe-stream: rounds of eight loads per lane (512 x 2 = the GEMV's shape)")
    ap.add_argument("--force-redo", action="store_true",
                    help="every step with every long segment redone from the keys (the library's testing hook): the worst case of the "
                         "step, for a kernel trace of it; the line says so in config.forced_redo")
    ap.add_argument("--settle", type=int, default=30,
                    help="untimed steps run as part of the set-up, before the warm-up steps (reported as settle_steps)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-runs", type=int, default=5)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no sharding, no collectives); run with --gpus 1",
              file=sys.stderr)
        return 2

    import torch
    from topk_attn_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = build_workload(args.workload, torch, ops, dev, args)
    if args.force_redo:
        if not hasattr(w, "hooks"):
            print("bench.py: --force-redo applies to the workloads that select (c1, c4*, c5*)", file=sys.stderr)
            return 2
        w.hooks = dict(w.hooks, force_segment_redo=1)
        ops.set_test_hooks(**w.hooks)

    # Set-up, before the W warm-up steps and the K timed ones: a card that has idled while the host built the workload
    # takes some 10 ms of work to settle (the first 25 steps of c4 after an idle gap run 1.5 % slower than all later ones,
    # by GPU-side events as well as by the wall clock); the line says how many steps were run for that.
    for _ in range(args.settle):
        w.step()
    torch.cuda.synchronize()

    for _ in range(args.warmup):
        w.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        w.step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    step_bytes, dom_bytes, extra = w.bytes()
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # every step once more between its own pair of HIP events, recorded on the stream the library launches on
    # (torch's current stream): median and minimum, next to the mean of the back-to-back loop above
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for e0, e1 in pairs:
        e0.record()
        w.step()
        e1.record()
    torch.cuda.synchronize()
    per_step_us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in pairs)
    us_median, us_min = per_step_us[len(per_step_us) // 2], per_step_us[0]

    # per-kernel times from HIP events recorded by the library on the launch stream (second timed loop: the
    # event pairs add a few microseconds per kernel, so they stay out of the loop that `value` comes from)
    # the same loop also asks after every step how many segments the selection had to redo from the keys (a
    # redone segment costs about a millisecond: a run that hit one must say so)
    ops.profile_reset()
    ops.profile_enable(True)
    redone = 0 if hasattr(w, "redone_segments") else None
    for _ in range(args.steps):
        w.step()
        if redone is not None:
            redone += w.redone_segments()
    torch.cuda.synchronize()
    prof = ops.profile_read()
    ops.profile_enable(False)
    kern = {name: ms / max(n, 1) * 1e3 for name, (ms, n) in prof.items()}  # us per launch
    dominant = w.dominant
    if dominant == "gemv_scores" and "gemv_candidates_shared" in kern:
        dominant = "gemv_candidates_shared"             # ... over keys that the batch shares
    if dominant == "gemv_scores" and "gemv_candidates" in kern:
        dominant = "gemv_candidates"                    # long segments run the candidate-mode GEMV
    if dominant == "gemv_scores" and "gemv_cut" in kern:
        dominant = "gemv_cut"                           # a few segments of middling length: the common-cut GEMV
    if dominant == "gemv_scores" and "gemv_cut_slices" in kern:
        dominant = "gemv_cut_slices"                    # the same route on calls that fill the GPU
    dom_us = kern.get(dominant, ms_per_step * 1e3)     # a workload with one foreign kernel: the step itself
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9
    traffic, traffic_source = recorded_traffic(args.workload, dominant) if not args.splits else (None, None)

    def median_us(step, n):
        """Median over n steps, each between its own pair of events (two untimed steps first)."""
        step()
        step()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for e0, e1 in ev:
            e0.record()
            step()
            e1.record()
        torch.cuda.synchronize()
        return sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in ev)[n // 2]

    # The step when EVERY segment is redone from its keys (the testing hook makes the selection refuse every candidate
    # count): the bound on what a step can cost whatever the data does.
    worst_us = worst_redone = None
    if hasattr(w, "hooks") and hasattr(w, "redone_segments") and not args.force_redo:
        ops.set_test_hooks(force_segment_redo=1, **w.hooks)
        worst_us = median_us(w.step, min(args.steps, 10))
        worst_redone = w.redone_segments()
        ops.set_test_hooks(**w.hooks)
        w.step()
        torch.cuda.synchronize()
        assert w.redone_segments() == 0 or redone, "segments still redone after the hook was cleared"
    rank_us = None
    if getattr(w, "make_rank_plan", None):
        rank_plan = w.make_rank_plan()
        rank_us = median_us(rank_plan.step, min(args.steps, 20))
        del rank_plan

    out = {
        "metric": "us/decode-step + achieved HBM GB/s (% of peak), GEMV+top-k+sparse attn @128k",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_steps": args.settle, "ms_per_step": round(ms_per_step, 5), "us_per_step": round(ms_per_step * 1e3, 2),
        "us_per_step_median": round(us_median, 2), "us_per_step_min": round(us_min, 2),
        "redone_segments": redone,
        "worst_case_us_per_step": None if worst_us is None else round(worst_us, 2), "worst_case_redone_segments": worst_redone,
        "us_per_step_with_rank_order": None if rank_us is None else round(rank_us, 2),
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded torch generator on the GPU)",
        "config": dict({"workload": w.desc, "algorithmic_bytes_per_step": step_bytes}, **dict(extra, **({"forced_redo": True} if args.force_redo else {}))),
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "algorithmic_bytes_per_launch": dom_bytes, "avg_launch_us": round(dom_us, 2)},
        "kernels_us": {k_: round(v, 2) for k_, v in sorted(kern.items())},
    }
    if not args.no_cpu and hasattr(w, "cpu_baseline"):
        cpu_s, info = w.cpu_baseline(args.cpu_runs)
        out["cpu_baseline"] = dict({"value": round(step_bytes / cpu_s / 1e9, 3), "unit": "GB/s",
                                    "us_per_step": round(cpu_s * 1e6, 1)}, **info)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
