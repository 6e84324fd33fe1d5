"""topk_attn_amd — MI355X (gfx950) sparse-decode path: fused GEMV + exact top-k, gathered retrieval
attention, split-K flash-decoding with LSE combine.  Hand-written HIP behind a C ABI (include/topk_attn.h);
this package is the thin Python host side."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


TORCH_EXT_PATH = os.path.join(_HERE, "lib", "retrieval_attention_cpp.so")


def build(force=True, jobs=8):
    """Compile libtka.so for gfx950 and tka_standalone with hipcc, and the PyTorch extension module
    retrieval_attention_cpp with g++ (no GPU needed).  force=False makes only what is missing or out of date."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    build_torch_extension(force)
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
