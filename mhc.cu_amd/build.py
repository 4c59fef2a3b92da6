"""Builds libmhc_hip.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc.

    python mhc.cu_amd/build.py [--jobs N] [--profile | --tuning] [--no-ext]

hipcc cross-compiles for gfx950 without a GPU.  The library lands in mhc.cu_amd/mhc/ next to
the Python package that loads it; object files go to mhc.cu_amd/build/.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "mhc", "libmhc_hip.so")

SOURCES = ["capi.hip", "proj_fwd.hip", "gemm_f32.hip", "proj_bwd.hip", "proj_bwd_addx.hip", "proj_bwd_large.hip", "bwd_slab.hip", "coef_fwd.hip", "mix_fwd.hip", "layer_fwd_onepass.hip", "mix_bwd_reduce.hip",
           "bwd_resident.hip", "mix_bwd_dx.hip", "param_grads.hip", "pack_params.hip", "ops.hip"]

# -packed-fp32-ops off: v_pk_*_f32 forms are not trusted on this hardware pool.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


PROFILE_LIB = os.path.join(HERE, "mhc", "libmhc_hip_profile.so")
TUNING_LIB = os.path.join(HERE, "mhc", "libmhc_hip_tuning.so")


def _compile(src, extra=(), suffix=""):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".o")
    cmd = [_hipcc(), *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "packed-fp32-ops" not in l)
    return src, obj, p.returncode, err


def build(jobs: int = 8, verbose: bool = True, profile: bool = False, tuning: bool = False):
    """profile=True builds libmhc_hip_profile.so instead: the same library with the in-kernel phase
    profiler compiled in (csrc/phase_profiler.h), the extra entry point mhc_phase_read and the
    launch-heuristic overrides of the tuning build.
    tuning=True builds libmhc_hip_tuning.so instead: the same library with the launch-heuristic
    overrides of csrc/tuning.h and their setter mhc_tuning_set, for experiments and for the tests that
    compare two launch paths on the same inputs; the product library has neither."""
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    extra, suffix, lib = ((("-DMHC_PHASE_PROFILE", "-DMHC_TUNING", "-fgpu-rdc"), "_prof", PROFILE_LIB) if profile
                          else ((("-DMHC_TUNING",), "_tune", TUNING_LIB) if tuning else ((), "", LIB)))
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, err in ex.map(lambda s_: _compile(s_, extra, suffix), SOURCES):
            if err.strip() and verbose:
                print(f"[{src}]\n{err}", file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}")
            objs.append(obj)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *(["-fgpu-rdc"] if profile else []), "-o", lib, *objs]
    subprocess.check_call(cmd)
    if verbose:
        print("built", lib)
    return lib


PROBE_LIB = os.path.join(HERE, "mhc", "libmhc_probe.so")


def build_probe(verbose: bool = True):
    """libmhc_probe.so: the plain streaming kernels of csrc/stream_probe.hip (measured bandwidth ceilings
    and launch floor for bench.py --stream-probe).  Deliberately not part of libmhc_hip.so."""
    cmd = [_hipcc(), *FLAGS, "-shared", os.path.join(CSRC, "stream_probe.hip"), "-o", PROBE_LIB]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed on stream_probe.hip:\n" + p.stderr)
    if verbose:
        print("built", PROBE_LIB)
    return PROBE_LIB


EXT_SRC = os.path.join(HERE, "torch_ext", "mhc_torch_ext.cpp")
EXT_NAME = "mhc_torch_ext"


def ext_path():
    import sysconfig
    return os.path.join(HERE, "mhc", EXT_NAME + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_torch_ext(verbose: bool = True):
    """Compiles the PyTorch-ROCm extension (torch_ext/mhc_torch_ext.cpp: host C++ only, it calls the
    C ABI of libmhc_hip.so) with g++ against the installed torch headers and links it next to the
    library.  Needs libmhc_hip.so (build() above)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(OBJ, exist_ok=True)
    obj = os.path.join(OBJ, EXT_NAME + ".o")
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include"]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", f"-DTORCH_EXTENSION_NAME={EXT_NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-DUSE_ROCM=1", "-D__HIP_PLATFORM_AMD__=1", "-DHIPBLAS_V2",
           f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-Wno-deprecated-declarations", *inc, "-c", EXT_SRC, "-o", obj]
    subprocess.check_call(cmd)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = ext_path()
    cmd = [cxx, "-shared", obj, "-o", out, f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
           "-ltorch_python", f"-L{os.path.join(HERE, 'mhc')}", "-lmhc_hip", "-Wl,-rpath,$ORIGIN",
           f"-Wl,-rpath,{tlib}"]
    subprocess.check_call(cmd)
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    ap.add_argument("--profile", action="store_true", help="build libmhc_hip_profile.so (in-kernel phase profiler)")
    ap.add_argument("--tuning", action="store_true", help="build libmhc_hip_tuning.so (launch-heuristic overrides)")
    ap.add_argument("--no-ext", action="store_true", help="skip the PyTorch extension (about a minute of g++)")
    a = ap.parse_args()
    build(a.jobs, profile=a.profile, tuning=a.tuning)
    if not a.profile and not a.tuning:
        build_probe()
    if not a.profile and not a.tuning and not a.no_ext:
        build_torch_ext()
