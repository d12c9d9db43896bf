"""Build the CPU oracle (test infrastructure, not the product).

  python oracle/build.py          builds oracle/liboracle.so from oracle/oracle.c
  python oracle/build.py --ref    additionally compiles the reference's own CPU
                                  sources (where they lie under /root/reference)
                                  into oracle/_ref/, when that tree is present.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE_BACKEND = "/root/reference/torchsparse/backend"
REF_MODULE = "tsref_cpu"


# ASAN=1 (or SANITIZE=address) in the environment: the oracle is built with AddressSanitizer and
# UndefinedBehaviorSanitizer into liboracle_asan.so, by the clang that also builds the host side
# of libtsmi_asan.so (one process can hold one sanitizer runtime), and oracle.lib() loads that
# file.  Host code only.  To run the CPU tests under it:
#   ASAN=1 python oracle/build.py && ASAN=1 python torchsparse_amd/csrc/build.py
#   ASAN=1 ASAN_OPTIONS=detect_leaks=0 LD_PRELOAD=$(python oracle/build.py --asan-runtime) \
#       python -m pytest tests -q -m "not gpu"
SANITIZE = os.environ.get("ASAN", "0") not in ("", "0") or os.environ.get("SANITIZE") == "address"
CLANG = os.environ.get("HOST_CLANG", "/opt/rocm/lib/llvm/bin/clang")


def asan_runtime() -> str:
    """Path of the shared sanitizer runtime that has to be loaded before python itself."""
    return subprocess.check_output([CLANG, "-print-file-name=libclang_rt.asan-x86_64.so"], text=True).strip()


def build_oracle(verbose: bool = False) -> str:
    src = os.path.join(HERE, "oracle.c")
    if SANITIZE:
        out = os.path.join(HERE, "liboracle_asan.so")
        cmd = [CLANG, "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-shared-libasan",
               "-fopenmp", "-fPIC", "-shared", "-std=c11", "-fvisibility=hidden", src, "-o", out, "-lm"]
    else:
        out = os.path.join(HERE, "liboracle.so")
        cmd = ["gcc", "-O3", "-march=native", "-fopenmp", "-fPIC", "-shared", "-std=c11",
               "-fvisibility=hidden", src, "-o", out, "-lm"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return out


def build_ref(verbose: bool = False):
    """Compile the reference's CPU sources (gather-scatter convolution, hash, count,
    voxelize, devoxelize) behind oracle/ref_bind.cpp.  Returns the path of the built module or None
    when the reference tree is absent."""
    if not os.path.isdir(REFERENCE_BACKEND):
        return None
    from torch.utils import cpp_extension

    out_dir = os.path.join(HERE, "_ref")
    os.makedirs(out_dir, exist_ok=True)
    cpp_extension.load(
        name=REF_MODULE,
        sources=[
            os.path.join(HERE, "ref_bind.cpp"),
            os.path.join(REFERENCE_BACKEND, "convolution", "convolution_gather_scatter_cpu.cpp"),
            os.path.join(REFERENCE_BACKEND, "hash", "hash_cpu.cpp"),
            os.path.join(REFERENCE_BACKEND, "others", "count_cpu.cpp"),
            os.path.join(REFERENCE_BACKEND, "voxelize", "voxelize_cpu.cpp"),
            os.path.join(REFERENCE_BACKEND, "devoxelize", "devoxelize_cpu.cpp"),
        ],
        extra_include_paths=[REFERENCE_BACKEND],
        extra_cflags=["-O3", "-fopenmp"],
        extra_ldflags=["-lgomp"],
        build_directory=out_dir,
        verbose=verbose,
        is_python_module=False,
    )
    # keep only the shared object; the intermediate files are not needed
    for f in os.listdir(out_dir):
        if not f.endswith(".so"):
            os.remove(os.path.join(out_dir, f))
    return os.path.join(out_dir, REF_MODULE + ".so")


if __name__ == "__main__":
    if "--asan-runtime" in sys.argv:
        print(asan_runtime())
        sys.exit(0)
    print(build_oracle(verbose=True))
    if "--ref" in sys.argv:
        print(build_ref(verbose=True))
