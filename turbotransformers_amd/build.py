"""In-tree build of the native parts.

  libttmi.so                 HIP kernels + C ABI (hipcc, gfx950 only)
  turbo_transformers_cxx.so  host C++ layers + pybind11 module (g++), links libttmi.so

Run as ``python turbotransformers_amd/build.py [device|host|all]``.  Outputs land next to
the package so that they travel with the source tree; nothing is installed.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(PKG_DIR, "build")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
CXX = os.environ.get("CXX", "g++")

DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-I", INCLUDE,
    # A "#pragma unroll" the optimizer gives up on (the unrolled body grew past its size limit) leaves register
    # arrays indexed at run time: slow, and wrong where accumulators are pinned by inline asm.  Fail the build instead.
    "-Werror=pass-failed",
]
# Per-file additions.  attention.hip: maxima over MFMA results would otherwise be preceded by one
# canonicalising v_max per operand (signalling-NaN quieting), a tenth of the softmax's VALU work.
DEVICE_FILE_FLAGS = {"attention.hip": ["-fno-honor-nans"], "gemm.hip": ["-mllvm", "-pragma-unroll-threshold=65536"]}


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def device_lib_path():
    return os.path.join(LIB_DIR, "libttmi.so")


def host_module_path():
    ext = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(PKG_DIR, "turbo_transformers_cxx" + ext)


def _stale(obj, sources):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(s) > t for s in sources)


def build_device(jobs=8, verbose=True, force=True):
    """force=False recompiles only objects older than their source or any header."""
    src_dir = os.path.join(CSRC, "device")
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(f for f in os.listdir(src_dir) if f.endswith(".hip"))
    objs = []

    headers = [os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith(".h")]
    headers.append(os.path.join(INCLUDE, "ttmi.h"))

    def compile_one(name):
        obj = os.path.join(OBJ_DIR, name[:-4] + ".o")
        if not force and not _stale(obj, [os.path.join(src_dir, name)] + headers):
            return obj
        out = _run([HIPCC] + DEVICE_FLAGS + DEVICE_FILE_FLAGS.get(name, []) + ["-c", os.path.join(src_dir, name), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, sources))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", device_lib_path()] + objs)
    if verbose:
        print("built", device_lib_path())
    return device_lib_path()


def build_host(jobs=8, verbose=True):
    import pybind11
    src_dir = os.path.join(CSRC, "host")
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = []
    for base, _, files in os.walk(src_dir):
        sources += [os.path.join(base, f) for f in files if f.endswith(".cpp")]
    sources.sort()
    flags = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
             "-I", INCLUDE, "-I", src_dir, "-I", pybind11.get_include(),
             "-I", sysconfig.get_paths()["include"]]

    def compile_one(path):
        rel = os.path.relpath(path, src_dir).replace(os.sep, "_")
        obj = os.path.join(OBJ_DIR, "host_" + rel[:-4] + ".o")
        out = _run([CXX] + flags + ["-c", path, "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, sources))
    _run([CXX, "-shared", "-o", host_module_path()] + objs +
         ["-L", LIB_DIR, "-lttmi", "-Wl,-rpath,$ORIGIN/lib", "-lpthread", "-lz"])
    if verbose:
        print("built", host_module_path())
    return host_module_path()


def build_all(verbose=True):
    build_device(verbose=verbose)
    build_host(verbose=verbose)


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    incremental = "--incremental" in sys.argv
    if what in ("device", "all"):
        build_device(force=not incremental)
    if what in ("host", "all"):
        build_host()
