"""Builds the gfx950 shared library of this package with hipcc, in-tree.

    python -m ramtorch_amd.build

hipcc cross-compiles for gfx950 without a GPU.  The library lands next to the
sources as ``ramtorch_amd/_lib/libramtorch_sr_adamw.so`` and is loaded with
ctypes (see ``_native.py``); nothing is installed outside the tree.  A second,
optional artefact is a small CPython extension built with g++ (``build_gather``).
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libramtorch_sr_adamw.so")

SOURCES = ["api.hip"]
HEADERS = ["kernels.h", "device_types.h", "copy_pool.h", os.path.join("..", "..", "include", "ramtorch_sr_adamw.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # Never let the compiler form packed-fp32 instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # The rounding sequence is part of the contract: no implicit contraction
    # (kernels.h repeats this as a pragma), IEEE-correct division and sqrt.
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False, extra_flags=()) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc(), *HIPCC_FLAGS, *extra_flags, "-o", LIB_PATH] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know -packed-fp32-ops; harmless.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


# ---- optional CPython helper (plain g++; links against the installed torch) -------------------
GATHER_SRC = os.path.join(CSRC, "host_gather.cpp")


def gather_path() -> str:
    import sysconfig
    return os.path.join(LIB_DIR, "_rt_gather" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_gather(verbose: bool = False) -> str:
    """Compiles csrc/host_gather.cpp, the descriptor gatherer AdamW.step uses for
    parameter sets with many tensors.  It reads tensors through torch's C++ API, so it
    is tied to the installed torch build."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    os.makedirs(LIB_DIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-I" + i for i in cpp_extension.include_paths()]
    cmd += [GATHER_SRC, "-o", gather_path(), "-L" + torch_lib, "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10",
            "-Wl,-rpath," + torch_lib, "-pthread"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building the gather helper failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    return gather_path()


def is_stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC, s) for s in SOURCES] + [os.path.normpath(os.path.join(CSRC, h)) for h in HEADERS]
    return any(os.path.getmtime(d) > t for d in deps)


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_gather(verbose=True))
