"""Builds tests/native/unit_test_abi: a C++ program that drives the C ABI (libtde_hip.so) without Python or torch
in the process and checks it against the oracle's C restatement, which is linked in as the checker.

    python tests/native/build_native.py
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def build(verbose=False):
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    src = os.path.join(HERE, "unit_test_abi.cpp")
    out = os.path.join(HERE, "unit_test_abi")
    oracle_dir = os.path.join(ROOT, "oracle")
    pkg_dir = os.path.join(ROOT, "torch_dist_ext_amd")
    subprocess.run(["make", "-C", oracle_dir, "libtde_oracle.so"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    cmd = [hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "include"), src, "-o", out,
           "-L", pkg_dir, "-ltde_hip", "-L", oracle_dir, "-ltde_oracle",
           "-Wl,-rpath,$ORIGIN/../../torch_dist_ext_amd", "-Wl,-rpath,$ORIGIN/../../oracle"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    if verbose and proc.stdout.strip():
        print(proc.stdout)
    return out


if __name__ == "__main__":
    print("built:", build(verbose="-v" in sys.argv))
