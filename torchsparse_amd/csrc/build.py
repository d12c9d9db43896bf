"""Compile the HIP sources of this directory for gfx950 into torchsparse_amd/libtsmi.so.

  python torchsparse_amd/csrc/build.py [-v]

hipcc cross-compiles without a GPU; the shared object stays in-tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, "libtsmi.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = [
    "common.cpp",
    "kmap.hip",
    "sort.hip",
    "pointops.hip",
    "norm.hip",
    "conv_api.cpp",
    "launch_thread.cpp",
    "conv_igemm_f16.hip",
    "conv_igemm_bf16.hip",
    "conv_igemm_f32.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# ASAN=1 (or SANITIZE=address) in the environment: the host passes of the sources without device
# code (argument checks, plans, dispatch) are compiled with AddressSanitizer into libtsmi_asan.so,
# which the package then loads; device code is never instrumented.  For CPU runs of the host
# logic (python started with the sanitizer runtime preloaded), not for the GPU.
SANITIZE = os.environ.get("ASAN", "0") not in ("", "0") or os.environ.get("SANITIZE") == "address"
HOST_ONLY = ("common.cpp", "conv_api.cpp", "launch_thread.cpp")
HOST_SANITIZE = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-shared-libasan",
                 "-Xarch_host", "-fno-omit-frame-pointer", "-Xarch_host", "-g"]
if SANITIZE:
    OUT = os.path.join(PKG, "libtsmi_asan.so")
    OBJ_DIR = os.path.join(HERE, "build_asan")


def _compile(src, verbose):
    obj = os.path.join(OBJ_DIR, src.rsplit(".", 1)[0] + ".o")
    flags = FLAGS + (HOST_SANITIZE if SANITIZE and src in HOST_ONLY else [])
    cmd = [HIPCC] + flags + ["-x", "hip", "-c", os.path.join(HERE, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if verbose and err.strip():
        print(err)
    return obj


def build(verbose: bool = False, jobs: int = 8) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
    if SANITIZE:
        cmd += ["-fno-gpu-sanitize", "-fsanitize=address", "-shared-libasan"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
