"""What the compiler reports for every kernel of the library (hipcc's kernel-resource-usage remarks, no GPU needed).

A kernel that spills registers, or that needs a stack, gets scratch memory set up at every launch; the short kernels of
this library are a few microseconds long and feel it.  And the GEMV kernel of the common-cut route on calls that fill the
GPU runs two workgroups of 1024 threads per CU only while it stays within 64 registers per lane."""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "topk_attn_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
SOURCES = ["gemv_scores.hip", "gemv_cut.hip", "gemv_scores_mfma.hip", "topk_select.hip", "select_wave.hip", "attention.hip",
           "attention_mfma.hip", "attention_select.hip"]


def _remarks(source):
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wno-unused-function", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage", "-c", "-o", os.devnull, source]
    done = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-2000:]
    kernels, name = {}, None
    for line in done.stderr.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z /\[\]]+?): (\S+) \[-Rpass", line)
        if m and name:
            kernels[name][m.group(1).strip()] = m.group(2)
    return kernels


@pytest.fixture(scope="module")
def resources():
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    with ThreadPoolExecutor(max_workers=4) as pool:
        per_file = list(pool.map(_remarks, SOURCES))
    merged = {}
    for kernels in per_file:
        merged.update(kernels)
    assert len(merged) > 50
    return merged


def test_no_kernel_needs_scratch_memory(resources):
    bad = {name: r for name, r in resources.items() if "_kernel" in name and
           (r.get("ScratchSize [bytes/lane]") != "0" or r.get("VGPRs Spill") != "0" or r.get("Dynamic Stack") != "False")}
    assert not bad, bad


def test_slices_kernel_runs_two_workgroups_per_cu(resources):
    slices = {name: r for name, r in resources.items() if "gemv_cut_slices_kernel" in name}
    assert len(slices) == 4
    for name, r in slices.items():
        assert int(r["VGPRs"]) <= 64 and r["Occupancy [waves/SIMD]"] == "8", (name, r)
