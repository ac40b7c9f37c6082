"""Builds the native libraries in-tree with hipcc for gfx950.

    python -m raf_amd.build            # build everything
    python -m raf_amd.build --check    # exit 1 if a library is missing or older than its sources

Three shared objects land in raf_amd/lib/:
  libraf_hip_optim.so    HIP kernels + the C ABI declared in include/rafhip_optim.h
  libraf_hip_dialect.so  C++ host layer: OpEnv / dialect registry mirror + the `hip` dialect ops
  _torch_glue.so         CPython module that reads lists of torch tensors for the Python front end
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "raf_amd" / "csrc"
LIB = ROOT / "raf_amd" / "lib"
INCLUDE = ROOT / "include"

ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32.
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]

OPTIM_SOURCES = ["status.hip", "sgd.hip", "lans_kernels.hip", "lans_plan.hip", "l2norm.hip", "fuse_tensor.hip",
                 "device_rt.hip"]
DIALECT_SOURCES = ["dialect/registry.cc", "dialect/device_api.cc", "dialect/memory_pool.cc", "dialect/hip_dialect.cc",
                   "dialect/raf_ir.cc", "dialect/hip_fusion.cc", "dialect/c_api.cc"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP libraries cannot be built")
    return exe


def _run(cmd):
    print("+", " ".join(str(c) for c in cmd), flush=True)
    subprocess.run([str(c) for c in cmd], check=True, cwd=ROOT)


def optim_lib() -> Path:
    return LIB / "libraf_hip_optim.so"


def dialect_lib() -> Path:
    return LIB / "libraf_hip_dialect.so"


def build_optim() -> Path:
    LIB.mkdir(parents=True, exist_ok=True)
    out = optim_lib()
    srcs = [CSRC / s for s in OPTIM_SOURCES]
    _run([hipcc(), *HIP_FLAGS, "-shared", f"-I{INCLUDE}", f"-I{CSRC}", "-o", out, *srcs])
    return out


def build_dialect() -> Path:
    LIB.mkdir(parents=True, exist_ok=True)
    out = dialect_lib()
    srcs = [CSRC / s for s in DIALECT_SOURCES]
    # Host-only C++ that reaches the kernels through the C ABI alone: no HIP headers needed.
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-shared",
          f"-I{INCLUDE}", f"-I{CSRC / 'dialect'}", "-o", out, *srcs, f"-L{LIB}", "-lraf_hip_optim",
          "-Wl,-rpath,$ORIGIN"])
    return out


def glue_lib() -> Path:
    return LIB / "_torch_glue.so"


def build_glue() -> Path:
    """The only piece that sees torch's headers: host C++ built with the host compiler against the
    installed torch (its C++ ABI setting included) and this interpreter's headers."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    LIB.mkdir(parents=True, exist_ok=True)
    out = glue_lib()
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    incs = [f"-I{p}" for p in cpp_extension.include_paths()] + [f"-I{sysconfig.get_paths()['include']}"]
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
          f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", f"-I{INCLUDE}", *incs,
          "-o", out, CSRC / "torch_glue.cpp", f"-L{torch_lib}", "-ltorch_python", "-ltorch_cpu", "-lc10",
          f"-Wl,-rpath,{torch_lib}"])
    return out


def build_all() -> None:
    build_optim()
    build_dialect()
    build_glue()


def stale() -> list:
    """Libraries that are missing or older than any of their sources."""
    bad = []
    deps = {
        optim_lib(): [CSRC / s for s in OPTIM_SOURCES] + list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h")),
        dialect_lib(): [CSRC / s for s in DIALECT_SOURCES] + list((CSRC / "dialect").glob("*.h")) + list(INCLUDE.glob("*.h")),
        glue_lib(): [CSRC / "torch_glue.cpp", INCLUDE / "rafhip_dialect.h"],
    }
    for lib, srcs in deps.items():
        if not lib.exists() or any(s.stat().st_mtime > lib.stat().st_mtime for s in srcs if s.exists()):
            bad.append(lib)
    return bad


if __name__ == "__main__":
    if "--check" in sys.argv:
        bad = stale()
        for b in bad:
            print("stale or missing:", b)
        sys.exit(1 if bad else 0)
    build_all()
