"""Builds libcatcoc_hip.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc."""
import glob
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
LIB = os.path.join(PKG, "libcatcoc_hip.so")
HOST_EXAMPLE = os.path.join(PKG, "catcoc_quant_rs_host")   # C++ host driving the library through its C ABI alone
FACADE_EXAMPLE = os.path.join(PKG, "catcoc_facade_host")  # C++ host written against the template facade (catcoc_hip/dgemm.hpp)
OBJ_DIR = os.path.join(PKG, "csrc", "build")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(PKG, "csrc", "*.hip")))


def build(verbose=False, extra=(), jobs=8):
    """Compile every HIP source of the package and link libcatcoc_hip.so.  Always compiles."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(PKG, "csrc")]

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *extra, *inc, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr))
        if verbose and r.stderr:
            print(r.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, sources()))
    # Link WITHOUT naming a HIP runtime: the library binds to the libamdhip64 its host process has
    # already loaded (a C/C++ host links it itself; a torch process carries its own copy, and a second
    # runtime in one process cannot open the device).
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    # the stand-alone C++ host: plain g++, links the HIP runtime itself and the library beside it
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [cxx, "-O2", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(rocm, "include"),
           os.path.join(PKG, "csrc", "host_quant_rs.cpp"), "-o", HOST_EXAMPLE, "-L", PKG, "-lcatcoc_hip",
           "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    # the host written against the reference's kernel-template names (include/catcoc_hip/dgemm.hpp), also plain g++
    cmd = [cxx, "-O2", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(rocm, "include"),
           os.path.join(PKG, "csrc", "host_facade.cpp"), "-o", FACADE_EXAMPLE, "-L", PKG, "-lcatcoc_hip",
           "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    import sys
    build(verbose=True, extra=tuple(sys.argv[1:]))
