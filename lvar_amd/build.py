"""Build the C-ABI shared library ``lvar_amd/liblvar_sparse_attn.so`` for gfx950 with hipcc.

    python -m lvar_amd.build

hipcc cross-compiles without a GPU.  The library is built in-tree so that it travels with
the source tree; nothing is installed into site-packages.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "liblvar_sparse_attn.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["attn_fwd.hip", "colsum.hip", "masklist.hip", "listbuild.hip", "windowscore.hip", "capi.hip"]
ARCH = "gfx950"
# -packed-fp32-ops is switched off: hipcc must not form v_pk_{add,mul,fma}_f32 from float code
# -fno-honor-nans -mno-amdgpu-ieee: max/min map to single v_max/v_max3 without NaN-quieting copies
HIPCC_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-fno-honor-nans", "-mno-amdgpu-ieee",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build lvar_amd")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(verbose: bool = False) -> str:
    """Compile every HIP translation unit and link the shared library.  Always rebuilds."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        outs = list(ex.map(compile_one, zip(SOURCES, objs)))
    tmp = LIB_PATH + ".tmp"
    outs.append(_run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]))
    os.replace(tmp, LIB_PATH)
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build_library(verbose=True)
    sys.exit(0)
