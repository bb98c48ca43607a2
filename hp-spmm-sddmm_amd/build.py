"""In-tree build of the native libraries (no cmake: a few compiler lines).

  libhpspmm.so           HIP kernels + C ABI (include/hpspmm.h), hipcc, gfx950
  libhpspmm_graphgen.so  seeded synthetic graph generators, g++ / OpenMP
  libhpspmm_host.so      C++ host layer with the reference's entry-point shapes
  spmm_test_all          command-line driver with the reference's argv

Run as a script (`python hp-spmm-sddmm_amd/build.py`) or call build_all().
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
CXX = os.environ.get("CXX") or "g++"
ROCM = os.environ.get("ROCM_PATH") or "/opt/rocm"

# packed FP32 VALU ops are disabled for all device code in this build
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
CXX_FLAGS = ["-O3", "-march=x86-64-v2", "-std=c++17", "-fPIC", "-fopenmp", "-Wall", "-Wextra"]


def _run(cmd, verbose):
    if verbose:
        print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels(verbose=False):
    """libhpspmm.so from csrc/*.hip: one object per translation unit (compiled side by side), one link.
    Only the entry points of include/hpspmm.h are exported."""
    from concurrent.futures import ThreadPoolExecutor
    out = os.path.join(HERE, "libhpspmm.so")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    objs = [os.path.join(objdir, f[:-4] + ".o") for f in srcs]

    def compile_one(pair):
        src, obj = pair
        _run([HIPCC, *HIP_FLAGS, "-fvisibility=hidden", "-c", "-I", INCLUDE, "-I", CSRC,
              os.path.join(CSRC, src), "-o", obj], verbose)

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out], verbose)
    return out


def build_graphgen(verbose=False):
    out = os.path.join(HERE, "libhpspmm_graphgen.so")
    _run([CXX, *CXX_FLAGS, "-shared", os.path.join(CSRC, "graphgen.cpp"), "-o", out], verbose)
    return out


def build_host(verbose=False):
    """C++ host layer + CLI driver + CPU self-test (needs libhpspmm.so and libhpspmm_graphgen.so)."""
    srcs = sorted(os.path.join(HOST, "src", f) for f in os.listdir(os.path.join(HOST, "src"))
                  if f.endswith(".cpp"))
    lib = os.path.join(HERE, "libhpspmm_host.so")
    common = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-I", INCLUDE,
              "-I", os.path.join(HOST, "include")]
    link = ["-L", HERE, "-lhpspmm", "-lhpspmm_graphgen", "-L", os.path.join(ROCM, "lib"), "-lrocsparse",
            "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    _run([HIPCC, *common, "-shared", *srcs, "-o", lib, *link], verbose)
    for name in ("test_all", "host_selftest"):
        exe = os.path.join(HERE, "spmm_" + name)
        _run([HIPCC, *common, os.path.join(HOST, name + ".cpp"), "-o", exe, "-L", HERE, "-lhpspmm_host",
              *link], verbose)
    return lib


def build_all(verbose=False):
    build_kernels(verbose)
    build_graphgen(verbose)
    build_host(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    sys.exit(0)
