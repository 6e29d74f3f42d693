"""Builds libkvcm_hip.so (gfx950) in-tree with hipcc. `python -m tair_kvcache_amd.build` or build_library()."""
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libkvcm_hip.so")
SOURCES = ["kvcm_copy.hip", "kvcm_hash.hip", "kvcm_select.hip", "kvcm_file.hip"]


def hipcc_command(out=LIB_PATH):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    return [
        hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
        # keep the compiler from forming packed-FP32 instructions anywhere in device code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
        "-o", out,
    ] + [os.path.join(CSRC, s) for s in SOURCES]


def build_library(verbose=False):
    """Compiles every HIP source of the package into libkvcm_hip.so. Raises on failure."""
    cmd = hipcc_command()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
