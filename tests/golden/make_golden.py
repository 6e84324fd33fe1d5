#!/usr/bin/env python3
"""Writes tests/golden/sparse_decode_small.npz, retrieval_op_small.npz and cluster_small.npz: seeded inputs (bit patterns)
and the oracle's outputs for one small end-to-end case, one small call of the operator, and one small two-level /
centre-only selection per element type.
The reference repository holds no vectors of its own (all its data is generated at run time), so these fixtures
freeze the oracle instead: a change in tka_oracle.c that alters any result fails tests/test_golden.py.
Run from the repository root:  python tests/golden/make_golden.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402


def main():
    out = {}
    scale = float(np.float32(1.0 / np.sqrt(128.0)))
    for tag, dtype, seed in (("f16", oracle.F16, 11), ("bf16", oracle.BF16, 12)):
        rng = np.random.default_rng(seed)
        N, H, G, k, sink, local = 128, 2, 4, 24, 4, 8
        Kf = rng.standard_normal((N, H, 128))
        Kf[rng.permutation(N)[:8]] *= 4.0                       # a few heavy hitters
        levels = np.linspace(-2, 2, 16)
        Kf[64:96] = levels[rng.integers(0, 16, (32, H, 128))]    # a stretch of 16-level keys: exact ties
        q = oracle.to_bits(rng.standard_normal((H * G, 128)), dtype)
        K = oracle.to_bits(Kf, dtype)
        V = oracle.to_bits(rng.standard_normal((N, H, 128)), dtype)
        outs, tidx, tval, unis, cnts = [], [], [], [], []
        for h in range(H):
            o, ti, tv, u = oracle.sparse_decode_step(q[h * G:(h + 1) * G], K[:, h], V[:, h], dtype, G, k, sink, local, scale)
            outs.append(o); tidx.append(ti); tval.append(tv)
            unis.append(np.pad(u, (0, k + sink + local - len(u)), constant_values=-1)); cnts.append(len(u))
        out.update({tag + "_q": q, tag + "_K": K, tag + "_V": V, tag + "_out": np.stack(outs), tag + "_topk_idx": np.stack(tidx),
                    tag + "_topk_val": np.stack(tval), tag + "_union": np.stack(unis), tag + "_union_count": np.array(cnts)})
    out["params"] = np.array([128, 2, 4, 24, 4, 8], np.int64)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "sparse_decode_small.npz"), **out)

    # The operator (test_ra.py:88-160 in small): caches shared by a batch of 16, 2 heads, 4 chunks of 64 keys,
    # 8 survivors per chunk, raw-exp softmax, no scale.  128 segments: enough for the batch route of the library.
    op = {}
    B, N, H, chunks, topk = 16, 256, 2, 4, 8
    for tag, dtype, seed in (("f16", oracle.F16, 21), ("bf16", oracle.BF16, 22)):
        rng = np.random.default_rng(seed)
        q = oracle.to_bits(rng.standard_normal((B, H, 128)) * 0.1, dtype)
        Kf = rng.standard_normal((N, H, 128)) * 0.1
        Kf[100:140] = Kf[100]                                    # forty equal keys: ties inside and across chunks
        K = oracle.to_bits(Kf, dtype)
        V = oracle.to_bits(rng.standard_normal((N, H, 128)) * 0.1, dtype)
        outs = np.empty((B, H, 128))
        idx = np.empty((B, H, chunks * topk), np.int32)
        val = np.empty((B, H, chunks * topk), np.float32)
        for b in range(B):
            for h in range(H):
                outs[b, h], idx[b, h], val[b, h] = oracle.retrieval_attention(q[b, h], K[:, h], V[:, h], dtype, chunks, topk, 1.0)
        op.update({tag + "_q": q, tag + "_K": K, tag + "_V": V, tag + "_out": outs, tag + "_idx": idx, tag + "_val": val})
    op["params"] = np.array([B, N, H, chunks, topk], np.int64)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "retrieval_op_small.npz"), **op)

    # Two-level and centre-only selection (gemv_topk.cu:75-135, center_only_topk/gemv_topk.cu:82-119 in small):
    # 12 centroids, clusters of 16 tokens, top 8 clusters, top 6 tokens of each.  fp16 with 16 heads (128 segments:
    # the library ranks the centroids inside the token launch), bf16 with 2 heads (a launch of its own).  Three
    # centroids per head are identical and aligned with the query, so ranks 0-2 are a tie that the lower id must
    # win, and every cluster holds four equal rows.
    cl = {}
    CSZ, CLEN, TOPC, KC = 12, 16, 8, 6
    for tag, dtype, seed, Hc in (("f16", oracle.F16, 31, 16), ("bf16", oracle.BF16, 32, 2)):
        rng = np.random.default_rng(seed)
        cen = rng.uniform(-0.5, 0.5, (Hc, CSZ, 128))
        qf = rng.uniform(-0.5, 0.5, (Hc, 128))
        cen[:, [9, 3, 7]] = 0.9 * qf[:, None, :]
        keys = cen.transpose(1, 0, 2)[:, None, :, :] + 0.05 * rng.standard_normal((CSZ, CLEN, Hc, 128))
        keys[:, 4:8] = keys[:, 4:5]
        keys = keys.reshape(CSZ * CLEN, Hc, 128)
        q, cen_b, keys_b = oracle.to_bits(qf, dtype), oracle.to_bits(cen, dtype), oracle.to_bits(keys, dtype)
        two = np.stack([oracle.cluster_topk(q[h], cen_b[h], keys_b[:, h, :], dtype, TOPC, CLEN, KC, 1.0) for h in range(Hc)])
        exp = [oracle.center_topk_expand(q[h], cen_b[h], dtype, TOPC, CLEN, 1.0) for h in range(Hc)]
        cl.update({tag + "_q": q, tag + "_centers": cen_b, tag + "_keys": keys_b, tag + "_two_level": two,
                   tag + "_expand": np.stack([e[0] for e in exp]), tag + "_center_ids": np.stack([e[1] for e in exp]),
                   tag + "_center_val": np.stack([e[2] for e in exp])})
    cl["params"] = np.array([CSZ, CLEN, TOPC, KC], np.int64)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "cluster_small.npz"), **cl)


if __name__ == "__main__":
    main()
