"""Builds the native pieces in-tree with hipcc / g++ (no JIT cache, no cmake).

  libeppgcn_hip.so      HIP kernels + C ABI (no torch dependency)      -> eppgcn_amd/lib/
  GNNAdvisor*.so        pybind11/torch binding over the C ABI           -> eppgcn_amd/

``python -m eppgcn_amd.build`` builds both; ``build_all(force=True)`` recompiles
even when the outputs are newer than the sources.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "csrc", "_obj")
HIP_LIB = os.path.join(LIB_DIR, "libeppgcn_hip.so")
HIP_SOURCES = ["aggregate.hip", "stream.hip", "prepare.hip", "schedule.hip", "update.hip", "capi.hip"]
HIP_HEADERS = ["common.hpp", os.path.join(ROOT, "include", "eppgcn_hip.h"),
               os.path.join(ROOT, "include", "eppgcn_hip_tuning.h")]
ARCH = "gfx950"

# packed fp32 instructions are switched off for every device compile
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wall", "-Wno-unused-function"]


def _hipcc() -> str:
    return os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")


def _newer(target: str, deps) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout)
    return proc.stdout


def build_hip_library(force: bool = False, verbose: bool = False) -> str:
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES]
    hdrs = [h if os.path.isabs(h) else os.path.join(CSRC, h) for h in HIP_HEADERS]
    if not force and _newer(HIP_LIB, srcs + hdrs):
        return HIP_LIB
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, os.path.basename(s) + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        return _run([_hipcc(), *HIPCC_FLAGS, "-c", src, "-o", obj])

    with concurrent.futures.ThreadPoolExecutor(max_workers=len(srcs)) as pool:
        outs = list(pool.map(compile_one, zip(srcs, objs)))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    _run([_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", HIP_LIB, *objs])
    return HIP_LIB


def binding_path() -> str:
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(HERE, "GNNAdvisor" + suffix)


def build_binding(force: bool = False, verbose: bool = False) -> str:
    """pybind11 module ``GNNAdvisor`` (host C++ only; links libeppgcn_hip.so and libtorch)."""
    import torch
    from torch.utils import cpp_extension

    src = os.path.join(CSRC, "gnnadvisor_binding.cpp")
    out = binding_path()
    hdr = os.path.join(ROOT, "include", "eppgcn_hip.h")
    if not force and _newer(out, [src, hdr, HIP_LIB]):
        return out
    build_hip_library(force=False)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    inc = []
    for p in cpp_extension.include_paths() + [os.path.join(rocm, "include"), sysconfig.get_paths()["include"],
                                             os.path.join(ROOT, "include")]:
        inc += ["-I", p]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=GNNAdvisor",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *inc, src, "-o", out,
           "-L", torch_lib, "-L", LIB_DIR, "-L", os.path.join(rocm, "lib"),
           "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python", "-lamdhip64",
           "-leppgcn_hip", f"-Wl,-rpath,{torch_lib}", "-Wl,-rpath,$ORIGIN/lib", f"-Wl,-rpath,{os.path.join(rocm, 'lib')}"]
    log = _run(cmd)
    if verbose and log.strip():
        print(log)
    return out


def build_all(force: bool = False, verbose: bool = False):
    lib = build_hip_library(force, verbose)
    ext = build_binding(force, verbose)
    return lib, ext


if __name__ == "__main__":
    force = "--force" in sys.argv
    only_hip = "--hip-only" in sys.argv
    print(build_hip_library(force, verbose=True))
    if not only_hip:
        print(build_binding(force, verbose=True))
