"""fla_hip - MI355X (gfx950) linear-attention operators behind the operator API of
``fla_npu.ops.ascendc``.

The package is a thin ctypes front end over ``libfla_hip.so`` (hand-written HIP
kernels).  There is no CPU or eager fallback: if the shared library cannot be
loaded every operator call raises.

Counterpart of torch_custom/fla_npu/fla_npu/__init__.py:120-150 (library
location + ``ctypes.CDLL``), without the CANN environment probing.
"""
from __future__ import annotations

import ctypes
import os
from pathlib import Path
from typing import Optional

__all__ = ["load_library", "library_path", "is_library_loaded", "__version__"]
__version__ = "0.1.0"

_LIB: Optional[ctypes.CDLL] = None
_LIB_PATH: Optional[str] = None
ABI_VERSION = 1


def library_path() -> str:
    """Resolution order: ``FLA_HIP_LIB`` (explicit file), then the in-tree build."""
    env = os.environ.get("FLA_HIP_LIB")
    if env:
        return env
    return str(Path(__file__).resolve().parent / "lib" / "libfla_hip.so")


def load_library() -> ctypes.CDLL:
    """Load ``libfla_hip.so`` once and check its ABI version."""
    global _LIB, _LIB_PATH
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"fla_hip: {path} not found. Build it with `make -C flash-linear-attention-npu_amd/csrc` "
            "(or __graft_entry__.build()), or point FLA_HIP_LIB at a built libfla_hip.so. "
            "There is no fallback implementation."
        )
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    lib.fla_abi_version.restype = ctypes.c_int
    lib.fla_last_error.restype = ctypes.c_char_p
    got = lib.fla_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"fla_hip: {path} has ABI version {got}, this wrapper needs {ABI_VERSION}.")
    _LIB, _LIB_PATH = lib, path
    return lib


def is_library_loaded() -> bool:
    return _LIB is not None
