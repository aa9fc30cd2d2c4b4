"""Compile the gfx950 kernels into mindformers_amd/lib/libmf_decode.so with hipcc.

hipcc cross-compiles for gfx950 without a GPU present.  Objects go to mindformers_amd/csrc/build/ and the
shared library stays in-tree so that it travels with the source tree to the machine that runs it.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmf_decode.so")

SOURCES = ["errors.cpp", "kv_cache.hip", "paged_attention.hip", "prefill_attention.hip", "elementwise.hip", "w8a16_gemm.hip",
           "w8a8_gemm.hip", "moe.hip", "mla_attention.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 VALU forms are switched off for device code (they have produced silent wrong results on
# this hardware pool); the host pass does not know the feature and says so, which is harmless.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{out}")
    return out


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if src.endswith(".hip"):
        cmd = [HIPCC, *DEVICE_FLAGS, "-c", path, "-o", obj]
    else:
        cmd = [HIPCC, "-O2", "-std=c++17", "-fPIC", "-x", "c++", "-c", path, "-o", obj]
    _run(cmd)
    return obj


def build(verbose=True, jobs=None):
    """Compile every source and link the shared library (always recompiles)."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(8, len(SOURCES))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
