"""In-tree build of the two shared libraries, without cmake or a JIT cache.

  libtde_hip.so          hipcc, gfx950 only: the HIP kernels and the C ABI (include/tde_abi.h)
  libtorch_dist_ext.so   host compiler only: the torch operator/class registration, linked against
                         libtde_hip.so.  Name and place are the reference loader's (torch_dist_ext/__init__.py:8-12:
                         `<parent of the package directory>/lib<package>.so`), i.e. the repository root.

libtde_hip.so lands next to this file, libtorch_dist_ext.so one level up; both travel with the source tree.
Run as `python torch_dist_ext_amd/_build.py` (by path: importing the package needs the libraries
this script produces).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OBJ_DIR = os.path.join(PKG_DIR, "build")
HIP_LIB = os.path.join(PKG_DIR, "libtde_hip.so")
TORCH_LIB = os.path.join(ROOT, "libtorch_dist_ext.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["tde_abi.hip", "tde_rows_bf16.hip", "tde_rows_f16.hip", "tde_rows_f32.hip", "tde_rows_f64.hip", "tde_probe.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # keep fp32 arithmetic scalar: packed fp32 forms are not used on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no v_fma_mix*: the compiler folds "multiply in fp32, then convert to fp16" into v_fma_mixlo_f16, which rounds the
    # exact product once; the operator's contract is the two roundings of the eager composition
    "-Xclang", "-target-feature", "-Xclang", "-fma-mix-insts",
    # the kernels fix their own instruction order around the loads (scheduling barriers); the SLP vectorizer
    # regroups the element-wise arithmetic across them, which costs registers and the overlap with the loads
    "-fno-slp-vectorize",
    "-Wno-unused-command-line-argument",
]


def _run(cmd, quiet_substr=None):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = proc.stdout or ""
    if quiet_substr:
        out = "\n".join(l for l in out.splitlines() if quiet_substr not in l)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip(verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.path.join(ROCM, "bin", "hipcc")

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc] + HIP_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        out = _run(cmd, quiet_substr="packed-fp32-ops")
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=6) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES))
    # only the C ABI is exported: a second copy of this library in the process (another version, a build under test)
    # then runs its own launchers and kernels, not the first one's
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--version-script=" + os.path.join(CSRC, "tde_exports.map"),
          "-o", HIP_LIB] + objs)
    return HIP_LIB


def build_torch(verbose=False):
    import torch
    from torch.utils import cpp_extension

    torch_lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-deprecated-declarations",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
        "-I", INCLUDE, "-isystem", os.path.join(ROCM, "include"),
    ] + inc + [
        os.path.join(CSRC, "tde_torch.cpp"), "-o", TORCH_LIB,
        "-L", PKG_DIR, "-ltde_hip", "-L", torch_lib_dir, "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
        "-Wl,-rpath,$ORIGIN/torch_dist_ext_amd", "-Wl,-rpath," + torch_lib_dir, "-Wl,--no-as-needed",
    ]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return TORCH_LIB


def build_all(verbose=False):
    build_hip(verbose)
    build_torch(verbose)
    return HIP_LIB, TORCH_LIB


if __name__ == "__main__":
    libs = build_all(verbose="-v" in sys.argv)
    print("built:", *libs)
