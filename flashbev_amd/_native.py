"""Loader of the native units.  There is no CPU or pure-PyTorch fallback: if the HIP library
or the torch extension cannot be loaded, importing the operator fails loudly."""
from __future__ import annotations

import importlib.util
import os
import shutil
import sys
import warnings

from . import _build

_ext = None


def load_ext():
    """Return the ``flashbevpool_ext`` module (built in-tree under ``flashbev_amd/lib``)."""
    global _ext
    if _ext is not None:
        return _ext
    import torch  # noqa: F401  (libtorch must be loaded before the extension)

    if not _build.have_libs():
        if shutil.which("hipcc") is None:
            raise ImportError(
                "flashbev_amd: native libraries are missing (expected %s and %s) and hipcc is not "
                "available to build them; run `python -m flashbev_amd._build` on a machine with ROCm"
                % (_build.HIP_LIB, _build.EXT_LIB))
        _build.build_all()
    elif _build.stale():
        # what is built is what runs (file times do not survive every way of copying a tree, so this
        # is a warning; a library that no longer fits the header is an error, below)
        warnings.warn("flashbev_amd: a source under csrc/ is newer than the built libraries; "
                      "run `python -m flashbev_amd._build`", RuntimeWarning, stacklevel=2)
    spec = importlib.util.spec_from_file_location("flashbevpool_ext", _build.EXT_LIB)
    if spec is None or spec.loader is None:
        raise ImportError("flashbev_amd: cannot load %s" % _build.EXT_LIB)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    want = _build.header_abi_version()
    if want is not None and mod.abi_version() != want:
        raise ImportError("flashbev_amd: %s implements ABI version %d but include/flashbev_hip.h declares %d; "
                          "rebuild with `python -m flashbev_amd._build`" % (_build.HIP_LIB, mod.abi_version(), want))
    # same module name as the reference's extension, so `import flashbevpool_ext` keeps working
    sys.modules.setdefault("flashbevpool_ext", mod)
    # the reference keeps its PillarPool baseline in a second extension module; here one module serves both
    sys.modules.setdefault("sampling_vt_ext", mod)
    _ext = mod
    return mod


def lib_paths():
    return {"hip": _build.HIP_LIB, "ext": _build.EXT_LIB}


def is_built() -> bool:
    return os.path.exists(_build.HIP_LIB) and os.path.exists(_build.EXT_LIB)
