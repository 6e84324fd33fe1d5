"""torch-CPU restatement of the sparse-decode step — the reported CPU baseline.  TEST/BENCH INFRASTRUCTURE.

Same three stages as the reference's PyTorch model (baseline_1.py:71-110): fp32 GEMV on widened 16-bit
inputs, ``torch.topk``, gathered ``softmax(q.k/sqrt(d))`` attention in fp32; extended with the group-summed
selection score and the sink/local union that the GPU path uses.  ``torch.topk`` does not define a tie
order, so this is a timing baseline and a sanity check, not the bit-exact oracle (that is tka_oracle.c).
"""
import torch


def sparse_decode_cpu(q, keys, values, k, sink, local, scale, group):
    """q [Hq,128], keys/values [N,Hkv,128] (CPU, fp16/bf16).  Returns (out fp32 [Hq,128], topk idx [Hkv,k])."""
    n, hkv, d = keys.shape
    qf = q.float()
    kf = keys.float()                                                    # widen, as baseline_1.py:73-74
    qsum = qf.view(hkv, group, d).sum(1)                                 # selection score = sum over the group
    scores = torch.einsum("nhd,hd->hn", kf, qsum) * scale                # baseline_1.py:76
    top = torch.topk(scores, k, dim=1, largest=True, sorted=True).indices  # baseline_1.py:77
    out = torch.empty((hkv * group, d), dtype=torch.float32)
    lo = min(sink, n)
    hi = max(n - local, lo)
    for h in range(hkv):
        mid = top[h][(top[h] >= lo) & (top[h] < hi)]
        ids = torch.cat([torch.arange(lo), torch.sort(mid).values, torch.arange(hi, n)])
        ks = kf[ids, h]                                                  # gather, baseline_1.py:101-103
        vs = values[ids, h].float()
        logits = (qf[h * group:(h + 1) * group] @ ks.T) * scale          # baseline_1.py:105
        w = torch.softmax(logits, dim=-1)                                # baseline_1.py:106
        out[h * group:(h + 1) * group] = w @ vs                          # baseline_1.py:107
    return out, top
