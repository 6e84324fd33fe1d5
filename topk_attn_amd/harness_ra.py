"""Harness for the operator in the shape of the reference's own (test_ra.py:162-358): for every K per chunk and
every variant name it runs the op, checks the output against a torch model of the op computed here, prints
PASSED / FAILED per variant and, at the end, the performance table built from the timing line the op prints
(retrieval_attention.cu:1586-1612 prints that line on every call; here the op is silent unless asked to).

    python -m topk_attn_amd.harness_ra [--batch 4] [--topk 32 128 ...] [--tol 1e-2] [--binding ctypes|extension]

--binding extension calls the ops of the compiled PyTorch extension module (csrc/torch_ext.cpp, the counterpart of the
module that test_ra.py:80-85 loads) instead of the ctypes binding; both end in the same C entry point.

The model (test_ra.py:88-160 restated): per head and per 2048-key chunk the K largest q.k (no 1/sqrt(d)),
softmax over the 4K survivors with raw exp, weighted sum of their V rows.  It runs in fp32 on the GPU with
``torch.sort(stable=True)``, so ties resolve to the lower index as in the op.  Exit status 1 if anything failed.
"""
import argparse
import ctypes
import os
import re
import sys
import tempfile

import torch

from . import _lib as L
from . import retrieval_attention_cpp as ra

VARIANT_LABELS = {"": "DSM", "_global": "Global", "_pipelined_global": "Pipelined Global", "_pipelined": "Pipelined",
                  "_two_kernels": "Two Kernels", "_gather_baseline": "TopK+Attn"}   # labels of test_ra.py's table


class CaptureStdout:
    """Collects what C code writes to file descriptor 1 while the block runs (the op prints with printf)."""

    def __enter__(self):
        sys.stdout.flush()
        self._saved = os.dup(1)
        self._tmp = tempfile.TemporaryFile(mode="w+b")
        os.dup2(self._tmp.fileno(), 1)
        self.text = ""
        return self

    def __exit__(self, *exc):
        sys.stdout.flush()
        ctypes.CDLL(None).fflush(None)
        os.dup2(self._saved, 1)
        os.close(self._saved)
        self._tmp.seek(0)
        self.text = self._tmp.read().decode(errors="replace")
        self._tmp.close()
        sys.stdout.write(self.text)
        return False


def model(q, k, v, topk, num_chunks=ra.NUM_CHUNKS):
    """fp32 torch model of the op: q [B,H,D], k/v [N,H,D] -> [B,H,D] (fp32)."""
    qf, kf, vf = q.float(), k.float(), v.float()
    n = kf.shape[0]
    chunk = n // num_chunks
    scores = torch.einsum("bhd,nhd->bhn", qf, kf)                       # [B,H,N]
    parts_s, parts_i = [], []
    for c in range(num_chunks):
        s, i = torch.sort(scores[:, :, c * chunk:(c + 1) * chunk], dim=-1, descending=True, stable=True)
        parts_s.append(s[:, :, :topk])
        parts_i.append(i[:, :, :topk] + c * chunk)
    s, i = torch.cat(parts_s, -1), torch.cat(parts_i, -1)               # [B,H,4K]
    p = torch.exp(s)
    p = p / p.sum(-1, keepdim=True)
    vh = vf.permute(1, 0, 2).contiguous()                               # [H,N,D]
    out = torch.empty_like(qf)
    for b in range(q.shape[0]):
        rows = torch.gather(vh, 1, i[b].unsqueeze(-1).expand(-1, -1, vf.shape[-1]))    # [H,4K,D]
        out[b] = torch.einsum("hk,hkd->hd", p[b], rows)
    return out


def run(topk, batch, tol, results, mod=ra):
    print("\nTesting with TOPK=%d, BATCH_SIZE=%d..." % (topk, batch))
    torch.manual_seed(0)
    dev = torch.device("cuda")
    q = torch.randn(batch, ra.NUM_HEADS, ra.HEAD_DIM, device=dev, dtype=torch.float16) * 0.1
    k = torch.randn(ra.SEQ_LEN, ra.NUM_HEADS, ra.HEAD_DIM, device=dev, dtype=torch.float16) * 0.1
    v = torch.randn(ra.SEQ_LEN, ra.NUM_HEADS, ra.HEAD_DIM, device=dev, dtype=torch.float16) * 0.1
    want = model(q, k, v, topk)
    ok = True
    for variant in L.RA_VARIANTS:
        label = VARIANT_LABELS.get(variant, variant)
        out = torch.zeros(batch, ra.NUM_HEADS, ra.HEAD_DIM, device=dev, dtype=torch.float16)
        torch.cuda.nvtx.range_push("retrieval_attention%s_%d" % (variant, topk))    # (roctx ranges on ROCm)
        print("Running %s Kernel..." % label)
        with CaptureStdout() as cap:
            getattr(mod, "retrieval_attention%s_%d" % (variant, topk))(q, k, v, out)
            torch.cuda.synchronize()
        torch.cuda.nvtx.range_pop()
        m = re.search(r"Avg time:\s+([\d\.]+)\s+ms,\s+Throughput:\s+([\d\.]+)\s+iter/s", cap.text)
        if m:
            results.append((topk, label, float(m.group(1)), float(m.group(2))))
        diff = (out.float() - want).abs()
        print("%s Kernel - Max diff: %g" % (label, diff.max().item()))
        print("%s Kernel - Mean diff: %g" % (label, diff.mean().item()))
        passed = diff.max().item() < tol
        print("%s Kernel: %s" % (label, "PASSED" if passed else "FAILED"))
        ok = ok and passed
    return ok


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--topk", type=int, nargs="*", default=list(L.RA_TOPKS))
    ap.add_argument("--tol", type=float, default=1e-2, help="max-abs tolerance (test_ra.py:202 uses 1e-2)")
    ap.add_argument("--binding", choices=["ctypes", "extension"], default="ctypes")
    args = ap.parse_args(argv)
    mod = ra
    if args.binding == "extension":
        from . import load_torch_extension
        mod = load_torch_extension()
    if not torch.cuda.is_available():
        print("harness_ra: no GPU visible", file=sys.stderr)
        return 2
    results, ok = [], True
    before = os.environ.get("TKA_BENCH_PRINT")
    os.environ["TKA_BENCH_PRINT"] = "1"          # the named ops then time themselves and print the reference's line
    try:
        for topk in args.topk:
            ok = run(topk, args.batch, args.tol, results, mod) and ok
    finally:
        if before is None:
            del os.environ["TKA_BENCH_PRINT"]
        else:
            os.environ["TKA_BENCH_PRINT"] = before
    print("\nPerformance Results (Batch Size = %d):" % args.batch)
    print("| %-5s | %-20s | %-15s | %-20s |" % ("TopK", "Kernel Type", "Avg Time (ms)", "Throughput (iter/s)"))
    print("|%s|%s|%s|%s|" % ("-" * 7, "-" * 22, "-" * 17, "-" * 22))
    for topk, label, ms, thr in results:
        print("| %-5d | %-20s | %-15.3f | %-20.2f |" % (topk, label, ms, thr))
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
