"""topk_attn_amd — MI355X (gfx950) sparse-decode path: fused GEMV + exact top-k, gathered retrieval
attention, split-K flash-decoding with LSE combine.  Hand-written HIP behind a C ABI (include/topk_attn.h);
this package is the thin Python host side."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(force=True, jobs=8):
    """Compile libtka.so for gfx950 with hipcc (no GPU needed)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return os.path.join(_HERE, "lib", "libtka.so")


from . import _lib  # noqa: E402
from ._lib import TkaError, LibraryMissing  # noqa: E402,F401
