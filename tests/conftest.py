import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """What is built is used as it is; only when the library, the command-line program or the PyTorch extension is missing are they made."""
    lib = os.path.join(ROOT, "topk_attn_amd", "lib")
    if not all(os.path.exists(os.path.join(lib, f)) for f in ("libtka.so", "tka_standalone", "retrieval_attention_cpp.so")):
        import topk_attn_amd
        topk_attn_amd.build(force=False)


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
