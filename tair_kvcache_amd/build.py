"""Builds libkvcm_hip.so (gfx950) in-tree with hipcc. `python -m tair_kvcache_amd.build` or build_library().

Every source is compiled to an object of its own, the objects in parallel, then linked. build_library() also builds
tests/libkvcm_hash_general_loader.so: the block-key entry points compiled with KVCM_TEST_FORCE_GENERAL_LOADER, so that
the parity tests can run the loader form that a workgroup spanning 4 GiB of tokens takes without allocating 4 GiB --
a library of its own, because the shipped one has no switch for it -- and the small CPython extension
_kvcm_pylist (gcc) that packs Python index lists."""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libkvcm_hip.so")
TEST_HOOK_LIB_PATH = os.path.join(ROOT, "tests", "libkvcm_hash_general_loader.so")
SOURCES = ["kvcm_copy.hip", "kvcm_hash.hip", "kvcm_select.hip", "kvcm_file.hip", "kvcm_host.hip"]
OBJ_DIR = os.path.join(PKG_DIR, "build")
# CPython extension (host code, gcc): Python index lists -> packed int32 in one C loop
PYLIST_PATH = os.path.join(PKG_DIR, "_kvcm_pylist" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def _hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def compile_flags():
    return [
        "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
        # keep the compiler from forming packed-FP32 instructions anywhere in device code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    ]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + out)
    return out


def build_library(verbose=False):
    """Compiles every HIP source of the package into libkvcm_hip.so, and the test-only general-loader build of the
    block-key entry points into tests/. Raises on failure."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = [(os.path.join(CSRC, s), os.path.join(OBJ_DIR, s.replace(".hip", ".o")), []) for s in SOURCES]
    hook_obj = os.path.join(OBJ_DIR, "kvcm_hash_general_loader.o")
    jobs.append((os.path.join(CSRC, "kvcm_hash.hip"), hook_obj, ["-DKVCM_TEST_FORCE_GENERAL_LOADER=1"]))
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
        outs = list(pool.map(lambda j: _run([_hipcc()] + compile_flags() + j[2] + ["-c", "-o", j[1], j[0]]), jobs))
    link = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC"]
    outs.append(_run(link + ["-o", LIB_PATH] + [j[1] for j in jobs[:len(SOURCES)]]))
    outs.append(_run(link + ["-o", TEST_HOOK_LIB_PATH, hook_obj]))
    outs.append(_run([os.environ.get("CC", "gcc"), "-O2", "-shared", "-fPIC", "-Wall", "-Wextra",
                      "-I" + sysconfig.get_paths()["include"], "-o", PYLIST_PATH, os.path.join(CSRC, "kvcm_pylist.c")]))
    if verbose:
        text = "\n".join(o for o in outs if o.strip())
        if text:
            print(text)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
