"""Operator boundary: same surface as the reference's `fast_2d_gs/_C/__init__.py` (get_C_function,
have_C_functions, try_use_C_extension, get_python_function; reference lines 10-49), backed by the hand-written HIP
library through its C ABI instead of a pybind module.

Differences that are deliberate:
  * there is no silent Python fallback: if libfsgs_hip.so is missing, importing this package raises;
  * names without a counterpart in the reference (`knn_topk`, `lbs_blend`) are additive.
"""
from __future__ import annotations

import warnings
from typing import Callable, Union

from .. import lib as _lib

_lib.load()  # fail loudly at import time, before any wrapper class captures a callable

from . import _ops  # noqa: E402

_py_functions = {}

EXPORTED = tuple(_ops.__all__)


def get_python_function(func: str):
    return _py_functions[func]


def try_use_C_extension(func: Callable, *depends: str):
    """Reference semantics (fast_2d_gs/_C/__init__.py:18-38): used bare it registers `func` as the Python
    implementation and returns the native one of the same name; used with dependency names it is a decorator that
    returns `func` (the native-backed callable) iff every dependency is exported."""
    if len(depends) == 0:
        _py_functions[func.__name__] = func
        if hasattr(_ops, func.__name__) and func.__name__ in EXPORTED:
            return getattr(_ops, func.__name__)
        warnings.warn(f'No such function in C/CPP/CUDA extension: {func.__name__}')
        return func
    have_all = True
    for name in depends:
        if name not in EXPORTED:
            have_all = False
            warnings.warn(f'No such function in C/CPP/CUDA extension: {name}')
            break

    def wrapper(py_func: Callable) -> Callable:
        _py_functions[py_func.__name__] = py_func
        return func if have_all else py_func

    return wrapper


def get_C_function(func: Union[str, Callable]):
    if isinstance(func, str):
        return getattr(_ops, func, None) if func in EXPORTED else None
    return func


def have_C_functions(*names):
    return all(name in EXPORTED for name in names)


def __getattr__(name):  # `_C.<op>` attribute access, as on the reference's pybind module
    if name in EXPORTED:
        return getattr(_ops, name)
    raise AttributeError(name)


__all__ = ['try_use_C_extension', 'get_C_function', 'get_python_function', 'have_C_functions']
