"""Load the compiled kernel libraries through ctypes, compiling on first use.

There is no fallback: if a library is missing and cannot be compiled, or there
is no GPU, every kernel call raises.
"""

from __future__ import annotations

import ctypes
import threading
from pathlib import Path

from . import build

_LOCK = threading.Lock()
_LOADED: dict[str, ctypes.CDLL] = {}


class KernelUnavailable(RuntimeError):
    """The HIP extension is missing and could not be built."""


def _hash_of(library: ctypes.CDLL) -> str | None:
    try:
        fn = library.fe_source_hash
    except AttributeError:
        return None
    fn.restype = ctypes.c_char_p
    fn.argtypes = []
    return fn().decode()


def _try_open(path: Path, expected: str) -> ctypes.CDLL | None:
    # A stale library must not be opened at all: the loader keeps a handle per path name, so a
    # library rebuilt at the same path afterwards would still resolve to the stale code.
    if not path.exists() or expected.encode() not in path.read_bytes():
        return None
    try:
        library = ctypes.CDLL(str(path))
    except OSError:
        return None
    return library if _hash_of(library) == expected else None


def is_built(name: str) -> bool:
    expected = build.source_hash(name)
    for directory in build.library_dirs():
        path = build.library_path(name, directory)
        if path.exists() and expected.encode() in path.read_bytes():
            return True
    return False


def ensure_built(names, announce: bool = True) -> None:
    """Compile, in parallel, those of ``names`` that have no current library."""
    missing = [name for name in names if name not in _LOADED and not is_built(name)]
    if missing:
        try:
            build.compile_many(missing, announce=announce)
        except build.KernelBuildError as error:
            raise KernelUnavailable(str(error)) from error


def load(name: str) -> ctypes.CDLL:
    """Return the library for ``csrc/<name>.hip``."""
    library = _LOADED.get(name)
    if library is not None:
        return library
    with _LOCK:
        library = _LOADED.get(name)
        if library is not None:
            return library
        expected = build.source_hash(name)
        for directory in build.library_dirs():
            library = _try_open(build.library_path(name, directory), expected)
            if library is not None:
                break
        if library is None:
            try:
                path = build.compile_one(name)
            except build.KernelBuildError as error:
                raise KernelUnavailable(
                    f"kernel library '{name}' is not built and could not be compiled: {error}"
                ) from error
            library = _try_open(path, expected)
            if library is None:
                raise KernelUnavailable(f"kernel library {path} was built but does not load")
        _LOADED[name] = library
        return library


def loaded_libraries() -> dict[str, str]:
    return {name: library._name for name, library in _LOADED.items()}
