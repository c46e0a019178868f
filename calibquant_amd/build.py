"""Build the C-ABI HIP library in-tree: calibquant_amd/lib/libcalibquant_hip.so.

Run `python -m calibquant_amd.build`.  hipcc cross-compiles for gfx950 without
a GPU.  The built library is git-ignored and is loaded by `calibquant_amd._lib`.
The second product is the host shim `_cq_torch_step.so` (C++ over torch's headers,
host compiler), which the eager decode step of the attention patch calls.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBPATH = os.path.join(LIBDIR, "libcalibquant_hip.so")
SOURCES = ["cq_core.hip", "cq_quantize.hip", "cq_lutvecmat.hip", "cq_decode.hip", "cq_rope.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # keep the compiler from emitting packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]
# per-source additions.  The decode kernels are bound by vector-instruction issue: the
# ILP-first machine scheduler measures 1-3 % faster there (same register counts, no scratch).
EXTRA_FLAGS = {
    "cq_decode.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"],
}


def build(verbose: bool = True, jobs: int = 4) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    objs, procs = [], []
    for src in SOURCES:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIBPATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIBPATH


SHIM_SRC = os.path.join(CSRC, "cq_torch_step.cpp")
SHIM_NAME = "_cq_torch_step"
SHIMPATH = os.path.join(LIBDIR, SHIM_NAME + ".so")


def build_torch_shim(verbose: bool = True) -> str:
    """The host shim between PyTorch and the C-ABI library (`calibquant_amd/lib/_cq_torch_step.so`): plain
    C++ over torch's headers, no kernels, so the host compiler builds it; it links the HIP library beside
    it (run-path $ORIGIN) and the torch libraries of the interpreter that builds it."""
    import sysconfig

    import torch
    tdir = os.path.dirname(torch.__file__)
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-DTORCH_EXTENSION_NAME=" + SHIM_NAME, "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(ROOT, "include"),
           SHIM_SRC, "-o", SHIMPATH,
           "-L" + os.path.join(tdir, "lib"), "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
           "-ltorch_python", "-L" + LIBDIR, "-lcalibquant_hip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return SHIMPATH


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        # hipcc's host pass warns that it does not know the packed-fp32 feature; harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip():
            print(out)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}")


PHASES_LIBPATH = os.path.join(LIBDIR, "libcalibquant_hip_phases.so")


def build_phase_stops(verbose: bool = True) -> str:
    """The profiling build of the decode source (`-DCQ_PHASE_STOPS`: only the headline instantiation, with
    early-exit points at the phase boundaries selected by the environment variable CQ_DECODE_PHASE_STOP)
    as a library of its own, `lib/libcalibquant_hip_phases.so`; `CALIBQUANT_HIP_LIBRARY` makes
    `calibquant_amd._lib` load it instead of the shipped one.  Used for the per-phase instruction counts
    under profiles/."""
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    for src in SOURCES:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".phases.o" if src == "cq_decode.hip" else ".o"))
        if src == "cq_decode.hip" or not os.path.exists(obj):
            extra = EXTRA_FLAGS.get(src, []) + (["-DCQ_PHASE_STOPS"] if src == "cq_decode.hip" else [])
            cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            p = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            _drain([(src, p)])
        objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PHASES_LIBPATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return PHASES_LIBPATH


if __name__ == "__main__":
    if "--phase-stops" in sys.argv[1:]:
        print(build_phase_stops())
        sys.exit(0)
    print(build())
    print(build_torch_shim())
    sys.exit(0)
