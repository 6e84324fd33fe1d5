"""tka_standalone, the command-line counterpart of the reference's stand-alone programs (gemv_topk.cu,
center_only_topk/gemv_topk.cu, baseline_1.cu, flash_decoding.cu, retrieval_attention.cu mains): argument handling without a GPU, and on a GPU
every subcommand with --verify, whose CPU check is computed inside the program."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "topk_attn_amd", "lib", "tka_standalone")


def _run(*args, timeout=180):
    return subprocess.run([BIN, *args], capture_output=True, text=True, timeout=timeout)


def test_usage_and_bad_arguments():
    assert os.path.exists(BIN), "tka_standalone is not built (make -C topk_attn_amd/csrc)"
    for args in ([], ["no_such_program"], ["gemv_topk", "--iters"], ["gemv_topk", "--iters", "0"], ["center_only", "--frobnicate"]):
        r = _run(*args)
        assert r.returncode == 64 and "usage:" in r.stderr, args


@pytest.mark.gpu
@pytest.mark.parametrize("args,lines", [
    (["gemv_topk", "--verify", "2"], ["Fused kernel latency:", "✓ GPU indices match CPU reference", "✓ rank order"]),
    (["center_only", "--verify", "4"], ["Fused kernel latency:", "✓ GPU indices match CPU reference", "✓ rank order"]),
    (["center_only", "--centroids", "4096", "--cluster-len", "64", "--topc", "64", "--verify"],
     ["✓ GPU indices match CPU reference", "Done: computed 32 x 4096 indices"]),
    (["baseline_1", "--verify", "2"], ["gemv_topk (indices build) latency:", "flash decode latency:",
                                       "gemv_topk + flash decode latency:", "✓ GPU indices match", "✓ attention output"]),
    (["flash_decoding", "--verify", "2"], ["flash decode latency:", "✓ attention output"]),
    (["flash_decoding", "--dense", "--verify", "1"], ["flash decode latency:", "✓ attention output"]),
    (["retrieval_attention", "--batch", "3", "--verify", "2"],
     ["Baseline Attention - Avg time:", "=== Running Retrieval Attention (Global Memory, TOPK=1024 per block) ===",
      "Retrieval Attention - Avg time:", "✓ output vs CPU", "Sample output values (head 0, first 8 dims):", "Done!"]),
])
def test_subcommands_verify(args, lines):
    from tests.util import announce
    announce("tka_standalone " + " ".join(args))
    r = _run(*args, "--iters", "5", "--warmup", "2")
    print(r.stdout[-2000:], r.stderr[-2000:], flush=True)
    assert r.returncode == 0
    for want in lines:
        assert want in r.stdout, want
    assert "✗" not in r.stdout
