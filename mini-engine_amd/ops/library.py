"""Loading the compiled HIP library, building it first when it is absent.

There is no other implementation behind these kernels: when the library can be neither found nor
compiled, :func:`lib` raises, and every op fails with it.
"""

from __future__ import annotations

import ctypes
import importlib.util
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
_lock = threading.Lock()
_lib: ctypes.CDLL | None = None
ABI_VERSION = 8


def _build_module():
    spec = importlib.util.spec_from_file_location("mini_engine_amd_csrc_build", os.path.join(_CSRC, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def build(force: bool = True, quiet: bool = False) -> str:
    """Compile the library (always, when ``force``) and return its path."""
    mod = _build_module()
    path = mod.default_lib_path()
    if not force and os.path.exists(path):
        return path
    return mod.build(quiet=quiet)


def _declare(lib: ctypes.CDLL) -> None:
    lib.me_last_error.restype = ctypes.c_char_p
    lib.me_abi_version.restype = ctypes.c_int


def lib() -> ctypes.CDLL:
    """The loaded library; compiled at the first call if no built file is there."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        mod = _build_module()
        path = mod.default_lib_path()
        if not os.path.exists(path):
            alt = os.path.join(__import__("tempfile").gettempdir(), f"mini_engine_hip_{os.getuid()}", mod.LIB_NAME)
            path = alt if os.path.exists(alt) and mod.is_current(alt) else mod.build()
        try:
            loaded = ctypes.CDLL(path)
        except OSError as e:
            raise RuntimeError(f"the HIP kernel library {path} could not be loaded: {e}") from e
        _declare(loaded)
        if loaded.me_abi_version() != ABI_VERSION:
            # a stale build from older sources: compile again and load the new file
            path = mod.build()
            loaded = ctypes.CDLL(path)
            _declare(loaded)
        _lib = loaded
        return _lib


def loaded_path() -> str | None:
    return None if _lib is None else _lib._name


class KernelError(RuntimeError):
    pass


def check(code: int) -> None:
    if code != 0:
        raise KernelError(lib().me_last_error().decode())
