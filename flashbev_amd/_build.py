"""In-tree build of the two native units.

  libflashbev_hip.so   hipcc, gfx950 only: the kernels and the C ABI (include/flashbev_hip.h)
  flashbevpool_ext.so  host C++: thin torch/pybind glue that validates tensors, picks up
                       PyTorch's current HIP stream and calls the C ABI

Both land in ``flashbev_amd/lib/`` so that they travel with the source tree.  Nothing is
built implicitly at import time unless no library exists at all.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
INCLUDE = os.path.join(ROOT, "include")
HIP_LIB = os.path.join(LIBDIR, "libflashbev_hip.so")
EXT_LIB = os.path.join(LIBDIR, "flashbevpool_ext.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",            # geometry must round every operation (bit-exact masks)
    "-munsafe-fp-atomics",          # hardware fp32 atomic add for the gradient scatter
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter",
]


def _run(cmd):
    print("[flashbev_amd build]", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_hip(verbose: bool = True) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = ["hipcc"] + HIPCC_FLAGS + ["-I", INCLUDE, "-o", HIP_LIB,
                                     os.path.join(CSRC, "fbev_kernels.hip")]
    _run(cmd)
    return HIP_LIB


def build_ext(verbose: bool = True) -> str:
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(LIBDIR, exist_ok=True)
    inc = []
    for p in ce.include_paths() + [sysconfig.get_paths()["include"], INCLUDE,
                                   os.path.join(ROCM, "include")]:
        inc += ["-isystem" if "torch" in p or "rocm" in p else "-I", p]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cxx11 = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=flashbevpool_ext",
           f"-D_GLIBCXX_USE_CXX11_ABI={cxx11}"] + inc + [
        "-o", EXT_LIB, os.path.join(CSRC, "fbev_torch_ext.cpp"),
        "-L", LIBDIR, "-lflashbev_hip", "-Wl,-rpath,$ORIGIN",
        "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python",
        "-Wl,-rpath," + torch_lib,
        "-L", os.path.join(ROCM, "lib"), "-lamdhip64",
    ]
    _run(cmd)
    return EXT_LIB


def build_all() -> None:
    build_hip()
    build_ext()


def have_libs() -> bool:
    return os.path.exists(HIP_LIB) and os.path.exists(EXT_LIB)


def stale() -> bool:
    """True when a source under csrc/ or the public header is newer than a built library.  Where the
    sources do not travel with the libraries (no csrc/ directory) nothing is stale."""
    if not have_libs() or not os.path.isdir(CSRC):
        return False
    built = min(os.path.getmtime(HIP_LIB), os.path.getmtime(EXT_LIB))
    srcs = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(INCLUDE, "flashbev_hip.h")]
    return any(os.path.exists(f) and os.path.getmtime(f) > built for f in srcs)


def header_abi_version():
    """FBEV_ABI_VERSION as include/flashbev_hip.h declares it (None without the header)."""
    import re
    try:
        text = open(os.path.join(INCLUDE, "flashbev_hip.h")).read()
    except OSError:
        return None
    m = re.search(r"#define\s+FBEV_ABI_VERSION\s+(\d+)", text)
    return int(m.group(1)) if m else None


if __name__ == "__main__":
    build_all()
    sys.exit(0)
