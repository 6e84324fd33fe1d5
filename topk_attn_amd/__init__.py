"""topk_attn_amd — MI355X (gfx950) sparse-decode path: fused GEMV + exact top-k, gathered retrieval
attention, split-K flash-decoding with LSE combine.  Hand-written HIP behind a C ABI (include/topk_attn.h);
this package is the thin Python host side."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


TORCH_EXT_PATH = os.path.join(_HERE, "lib", "retrieval_attention_cpp.so")


STAMP_PATH = os.path.join(_HERE, "lib", "BUILD_STAMP")
ARTEFACTS = ("libtka.so", "tka_standalone", "tka_bind_link_check", "retrieval_attention_cpp.so")


def source_digest():
    """SHA-256 over the names and contents of everything the built artefacts are made from."""
    import hashlib
    h = hashlib.sha256()
    roots = [os.path.join(_HERE, "csrc"), os.path.join(_HERE, "..", "include")]
    for root in roots:
        for name in sorted(os.listdir(root)):
            path = os.path.join(root, name)
            if os.path.isfile(path):
                h.update(name.encode() + b"\0")
                with open(path, "rb") as f:
                    h.update(f.read())
    return h.hexdigest()


def is_built():
    """True when every artefact exists and was built from the sources as they are now (by content, not by time)."""
    lib = os.path.join(_HERE, "lib")
    if not all(os.path.exists(os.path.join(lib, f)) for f in ARTEFACTS) or not os.path.exists(STAMP_PATH):
        return False
    with open(STAMP_PATH) as f:
        return f.read().strip() == source_digest()


def build(force=True, jobs=8):
    """Compile libtka.so for gfx950, tka_standalone and tka_bind_link_check with hipcc, and the PyTorch extension
    module retrieval_attention_cpp with g++ (no GPU needed).  force=False makes only what is missing or out of date.
    Raises when any compile fails; on success records the digest of the sources next to the artefacts."""
    if os.path.exists(STAMP_PATH):
        os.remove(STAMP_PATH)
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    build_torch_extension(force)
    with open(STAMP_PATH, "w") as f:
        f.write(source_digest() + "\n")
    return os.path.join(_HERE, "lib", "libtka.so")


def build_torch_extension(force=True):
    """csrc/torch_ext.cpp -> lib/retrieval_attention_cpp.so: host C++ only (pybind11 + the C ABI), so one g++ call
    against the headers and libraries of the installed torch."""
    src = os.path.join(_HERE, "csrc", "torch_ext.cpp")
    deps = [src, os.path.join(_HERE, "..", "include", "topk_attn.h"), os.path.join(_HERE, "lib", "libtka.so")]
    if not force and os.path.exists(TORCH_EXT_PATH) and all(os.path.getmtime(TORCH_EXT_PATH) >= os.path.getmtime(d) for d in deps):
        return TORCH_EXT_PATH
    import sysconfig

    import torch
    from torch.utils import cpp_extension
    lib = os.path.join(_HERE, "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__",
           "-DTORCH_EXTENSION_NAME=retrieval_attention_cpp", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for name in ("COMPILER_TYPE", "STDLIB", "BUILD_ABI"):   # pybind11 ABI tags of the torch build, where it states them
        tag = getattr(torch._C, "_PYBIND11_" + name, None)
        if tag is not None:
            cmd.append('-DPYBIND11_%s="%s"' % (name, tag))
    cmd += ["-I" + os.path.join(_HERE, "..", "include"), "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-isystem" + p for p in cpp_extension.include_paths()]
    cmd += [src, "-o", TORCH_EXT_PATH, "-L" + lib, "-ltka"]
    cmd += ["-L" + p for p in cpp_extension.library_paths()]
    cmd += ["-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python", "-Wl,-rpath,$ORIGIN"]
    subprocess.check_call(cmd)
    return TORCH_EXT_PATH


def load_torch_extension():
    """The compiled extension module `retrieval_attention_cpp` (same name and ops as the reference's bind.cpp
    module).  No fallback: raises LibraryMissing when it has not been built."""
    import importlib.util

    import torch  # noqa: F401  (the module links against torch's libraries)
    if not os.path.exists(TORCH_EXT_PATH):
        raise LibraryMissing("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'`" % TORCH_EXT_PATH)
    spec = importlib.util.spec_from_file_location("retrieval_attention_cpp", TORCH_EXT_PATH)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


from . import _lib  # noqa: E402
from ._lib import TkaError, LibraryMissing  # noqa: E402,F401
