"""Compile the hand-written gfx950 kernels into one C-ABI shared library, in-tree.

    python fms-acceleration_amd/build_hip.py

hipcc cross-compiles for gfx950 without a GPU.  Each translation unit is compiled to an object
in parallel and the objects are linked into ``lib/libfmsa_hip.so`` next to this file; the
Python side loads that file with ctypes and never builds at import time.  The measurement probe
(``csrc/probe.hip``, what ``bench.py --yardsticks`` times) is not part of the product: it becomes a
library of its own, ``lib/libfmsa_probe.so``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfmsa_hip.so")

SOURCES = ["api.hip", "dequant.hip", "gemm_fwd.hip", "gemm_bwd.hip", "gemm_bwd_t.hip", "lora_skinny.hip", "elementwise.hip", "nf4.hip", "norm_rope.hip"]
PROBE_SOURCE = "probe.hip"
PROBE_LIB_PATH = os.path.join(LIB_DIR, "libfmsa_probe.so")

# -packed-fp32-ops is switched off on purpose: the packed fp32 VALU forms are not trusted on the
# target machines, so fp32 math is emitted as scalar-per-lane instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 kernels cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile every source unconditionally and link the library.  Returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = _hipcc()
    objs = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        out = _run(cmd)
        if verbose and out.strip():
            print(out)
        return obj

    probe_obj = os.path.join(OBJ_DIR, PROBE_SOURCE.replace(".hip", ".o"))
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + 1)) as pool:
        list(pool.map(compile_one, list(zip(SOURCES, objs)) + [(PROBE_SOURCE, probe_obj)]))
    for path, members in ((LIB_PATH, objs), (PROBE_LIB_PATH, [probe_obj])):
        tmp = path + ".tmp"
        # --no-undefined: a kernel whose host stub was not emitted must fail the link, not the first call
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--no-undefined", "-o", tmp, *members])
        os.replace(tmp, path)
        if verbose:
            print("built", path)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
