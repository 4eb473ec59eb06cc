"""ctypes binding of libfsgs_hip.so. Prototypes are read from include/fsgs.h so the header is the single source of truth.

The product path has no CPU fallback: if the shared object is missing, loading fails loudly.
"""
from __future__ import annotations

import ctypes
import re
from pathlib import Path
from typing import Dict, List, Tuple

import torch

PKG_DIR = Path(__file__).resolve().parent
HEADER = PKG_DIR.parent / "include" / "fsgs.h"
DEBUG_HEADER = PKG_DIR.parent / "include" / "fsgs_debug.h"  # measurement / verification aids
LIB_PATH = PKG_DIR / "libfsgs_hip.so"

_SCALARS = {
    "int": ctypes.c_int, "int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64, "size_t": ctypes.c_size_t,
    "double": ctypes.c_double, "float": ctypes.c_float, "uint32_t": ctypes.c_uint32,
}


def parse_prototypes(header_text: str, prefix: str) -> Dict[str, Tuple[object, List[object]]]:
    """Returns {name: (restype, [argtypes])} for every `prefix*` function declared in a C header."""
    text = re.sub(r"/\*.*?\*/", " ", header_text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^[ \t]*#[^\n]*", " ", text, flags=re.M)  # preprocessor lines
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(" + prefix + r"\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()

        def ctype(decl: str):
            decl = decl.strip()
            if "*" in decl:
                return ctypes.c_void_p  # device / host addresses travel as plain integers
            return _SCALARS[decl.replace("const", "").split()[0]]

        restype = ctypes.c_char_p if "char" in ret else _SCALARS[ret.replace("const", "").split()[0]]
        argtypes = [] if args in ("", "void") else [ctype(a) for a in args.split(",")]
        protos[name] = (restype, argtypes)
    return protos


_lib = None
_protos = None


def prototypes():
    global _protos
    if _protos is None:
        _protos = parse_prototypes(HEADER.read_text() + "\n" + DEBUG_HEADER.read_text(), "fsgs_")
    return _protos


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP library first (python -m fast_sp_gs_amd.build). "
                "There is no CPU fallback for these operators.")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in prototypes().items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib


def ptr(t):
    """Device (or host) address of a tensor, NULL for None."""
    if t is None:
        return None
    return t.data_ptr()


def current_stream() -> int:
    """Raw handle of torch's current stream on the current device. The operators ask for it on every call, so it is read
    through torch's C accessor (a fraction of a microsecond) rather than through `torch.cuda.current_stream()`, which
    builds a Python Stream object (about 10 us, a dozen times per training step)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().fsgs_last_error()
        raise RuntimeError(f"{what}: {msg.decode() if msg else 'error'} (status {rc})")


def require_cuda(what: str, **tensors) -> None:
    """Mirrors the reference's CHECK_INPUT (fast_2d_gs/_C/include/common.hpp:25-35): device tensor, contiguous."""
    for name, t in tensors.items():
        if t is None:
            continue
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(f"{what}: {name} must be a Tensor")
        if not t.is_cuda:
            raise RuntimeError(f"{what}: {name} must be a CUDA tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{what}: {name} must be contiguous")


def require_shape(what: str, name: str, t: torch.Tensor, *shape) -> None:
    if tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"{what}: {name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def require_dtype(what: str, name: str, t: torch.Tensor, dtype) -> None:
    if t.dtype != dtype:
        raise RuntimeError(f"{what}: {name} must have dtype {dtype}, got {t.dtype}")
