"""Builds libtbe_hip.so (the C-ABI library declared in include/tbe_hip.h) for gfx950, and
table_batched_embeddings_cpp.so, the pybind11 module over it (host code, compiled with g++
against PyTorch's headers).

Run as a script (`python build.py`) or call `build()`.  Each .hip file is
compiled to an object in parallel and the objects are linked into one shared
library next to this file, so the library ships with the source tree.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libtbe_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
BINDING_NAME = "table_batched_embeddings_cpp"
BINDING_PATH = os.path.join(HERE, BINDING_NAME + ".so")
BINDING_SOURCE = "table_batched_embeddings_binding.cpp"
SOURCES = ["tbe_api.hip", "tbe_forward.hip", "tbe_sort.hip", "tbe_update.hip", "tbe_backward.hip",
           "tbe_cache.hip", "tbe_mixed.hip", "tbe_approx.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the TBE library needs the ROCm toolchain")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass prints one harmless line per file about the packed-fp32 feature
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False):
    """Compiles every HIP source and links LIB_PATH.  Always recompiles."""
    hipcc = _hipcc()
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    sources = list(SOURCES)
    missing = [s for s in sources if not os.path.exists(os.path.join(CSRC, s))]
    if missing:  # a library linked without one of its files would only fail at symbol lookup
        raise RuntimeError("missing HIP sources under %s: %s" % (CSRC, ", ".join(missing)))
    objects = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in sources]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    workers = min(len(sources), max(1, min(8, os.cpu_count() or 1)))
    with concurrent.futures.ThreadPoolExecutor(workers) as pool:
        for out in pool.map(compile_one, zip(sources, objects)):
            if verbose and out.strip():
                print(out)
    tmp = LIB_PATH + ".tmp"
    out = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objects)
    os.replace(tmp, LIB_PATH)
    if verbose and out.strip():
        print(out)
    build_binding(verbose)
    return LIB_PATH


def build_binding(verbose=False):
    """Compiles the pybind11 module (BINDING_SOURCE) and links it against LIB_PATH and PyTorch.
    It finds the library next to itself (rpath $ORIGIN)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    source = os.path.join(CSRC, BINDING_SOURCE)
    if not os.path.exists(source):
        raise RuntimeError("missing source %s" % source)
    gxx = shutil.which("g++")
    if gxx is None:
        raise RuntimeError("g++ not found; the pybind11 module needs a host C++ compiler")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = [os.path.join(os.path.dirname(HERE), "include")] + cpp_extension.include_paths() + \
        ["/opt/rocm/include", sysconfig.get_paths()["include"]]
    tmp = BINDING_PATH + ".tmp"
    cmd = [gxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=" + BINDING_NAME, "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-w"]
    cmd += ["-I" + d for d in includes]
    cmd += [source, "-o", tmp, "-L" + torch_lib, "-L" + HERE, "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10",
            "-lc10_hip", "-ltorch_hip", "-ltbe_hip", "-Wl,-rpath,$ORIGIN"]
    out = _run(cmd)
    os.replace(tmp, BINDING_PATH)
    if verbose and out.strip():
        print(out)
    return BINDING_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
