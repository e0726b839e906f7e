"""Build the C-ABI shared library ``lvar_amd/liblvar_sparse_attn.so`` for gfx950 with hipcc, and the
compiled torch binding ``lvar_amd/_lvar_torch.so`` (host code only, g++ against the torch headers).

    python -m lvar_amd.build

hipcc cross-compiles without a GPU.  Both are built in-tree so that they travel with the source tree;
nothing is installed into site-packages.
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


PROBE_PATH = os.path.join(HERE, "liblvar_bench_probe.so")


def build_bench_probe(verbose: bool = False) -> str:
    """Compile ``csrc/mfma_probe.hip`` (the sustained-MFMA-rate probe that ``bench.py`` times beside the
    attention kernels) into its own small shared library.  Always rebuilds."""
    tmp = PROBE_PATH + ".tmp"
    out = _run([_hipcc(), *HIPCC_FLAGS, "-shared", os.path.join(CSRC, "mfma_probe.hip"), "-o", tmp])
    os.replace(tmp, PROBE_PATH)
    if verbose:
        if out.strip():
            print(out)
        print("built", PROBE_PATH)
    return PROBE_PATH


BINDING_NAME = "_lvar_torch"
BINDING_PATH = os.path.join(HERE, BINDING_NAME + ".so")


def build_torch_binding(verbose: bool = False) -> str:
    """Compile ``csrc/torch_binding.cpp`` (the compiled fast path of ``dense_attn``) into a Python extension
    module.  Host code only: g++ with torch's include paths; the module receives the address of the C-ABI
    entry point at run time, so it does not link the HIP library.  Always rebuilds."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    cxx = shutil.which("g++")
    if cxx is None:
        raise RuntimeError("g++ not found; it is needed for the torch binding")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(rocm, "include")]
    tmp = BINDING_PATH + ".tmp"
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", f"-DTORCH_EXTENSION_NAME={BINDING_NAME}", "-D__HIP_PLATFORM_AMD__",
           "-DUSE_ROCM", "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           *["-I" + i for i in inc], os.path.join(CSRC, "torch_binding.cpp"), "-o", tmp,
           "-L" + tlib, "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python", "-Wl,-rpath," + tlib]
    out = _run(cmd)
    os.replace(tmp, BINDING_PATH)
    if verbose:
        if out.strip():
            print(out)
        print("built", BINDING_PATH)
    return BINDING_PATH


if __name__ == "__main__":
    build_library(verbose=True)
    build_torch_binding(verbose=True)
    build_bench_probe(verbose=True)
    sys.exit(0)
