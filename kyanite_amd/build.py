"""Build libknhip.so (host runtime + ahead-of-time gfx950 kernels) in-tree with hipcc.

Usage: python kyanite_amd/build.py [--force]  (run as a script: importing the package needs the built library)
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(HERE, "libknhip.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HOST_SOURCES = [
    "dtype.cpp", "graph.cpp", "serialize.cpp", "const_eval.cpp", "optimizer.cpp", "strided_shape.cpp",
    "kernels.cpp", "fused_graph.cpp", "rtc.cpp", "gemm_plan.cpp", "planner.cpp", "executor.cpp", "capi.cpp", "standalone.cpp",
]
DEVICE_SOURCES = ["kern/mfma_kernels.hip", "kern/mfma_f16_kernels.hip", "kern/attention_kernels.hip", "kern/attention_f16_kernels.hip",
                  "kern/static_scratch.hip"]

COMMON_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-D__HIP_PLATFORM_AMD__",
                f"-I{ROCM}/include"]
# packed f32 instructions stay off for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument"]


def _hipcc():
    return os.path.join(ROCM, "bin", "hipcc")


def _headers_digest():
    h = hashlib.sha256()
    for root, _, files in os.walk(CSRC):
        for name in sorted(files):
            if name.endswith(".h"):
                with open(os.path.join(root, name), "rb") as f:
                    h.update(f.read())
    with open(os.path.join(HERE, "..", "include", "knhip.h"), "rb") as f:
        h.update(f.read())
    return h.hexdigest()


def _compile(src, force, headers):
    path = os.path.join(CSRC, src)
    obj = os.path.join(BUILD_DIR, src.replace("/", "_") + ".o")
    stamp = obj + ".stamp"
    with open(path, "rb") as f:
        digest = hashlib.sha256(f.read() + headers.encode()).hexdigest()
    if not force and os.path.exists(obj) and os.path.exists(stamp) and open(stamp).read() == digest:
        return obj
    if src.endswith(".hip"):
        cmd = [_hipcc(), "-c", path, "-o", obj] + COMMON_FLAGS + DEVICE_FLAGS
    else:
        cmd = ["g++", "-c", path, "-o", obj] + COMMON_FLAGS
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"compiling {src} failed:\n{' '.join(cmd)}\n{res.stdout}\n{res.stderr}")
    with open(stamp, "w") as f:
        f.write(digest)
    return obj


def build(force=False, verbose=False):
    """Compile every source (always relinks); returns the path of the shared library."""
    os.makedirs(BUILD_DIR, exist_ok=True)
    headers = _headers_digest()
    sources = HOST_SOURCES + DEVICE_SOURCES
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(lambda s: _compile(s, force, headers), sources))
    cmd = [_hipcc(), "-shared", "-o", LIB_PATH] + objs + ["--offload-arch=gfx950", f"-L{ROCM}/lib", "-lhiprtc",
                                                          "-lamdhip64", "-ldl", f"-Wl,-rpath,{ROCM}/lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"linking libknhip.so failed:\n{' '.join(cmd)}\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
