"""Compile the HIP sources under ``csrc/`` into shared libraries for gfx950.

Each source file becomes one library ``lib/fe_<name>.so`` with ``extern "C"``
entry points, so a model compiles only the kernels it uses.  The hash of the
source (and of the shared header) is baked into the library; a library whose
hash differs from the sources beside it is rebuilt.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor, wait
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent.parent
SOURCE_DIR = PACKAGE_DIR / "csrc"
TARGET_ARCH = "gfx950"
HIPCC_FLAGS = (
    f"--offload-arch={TARGET_ARCH}", "-O3", "-std=c++17", "-shared", "-fPIC",
    # packed float32 instructions are kept off: the compiler must not form them
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


class KernelBuildError(RuntimeError):
    """hipcc is missing or failed."""


def source_names() -> list[str]:
    return sorted(path.stem for path in SOURCE_DIR.glob("*.hip"))


def source_hash(name: str) -> str:
    digest = hashlib.sha256()
    for path in [SOURCE_DIR / f"{name}.hip", *sorted(SOURCE_DIR.glob("*.h"))]:
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    digest.update(" ".join(HIPCC_FLAGS).encode())
    return digest.hexdigest()[:16]


def library_dirs() -> list[Path]:
    """Where libraries are looked for and written: in the tree first, else a
    per-user folder under the temporary directory (for a read-only checkout)."""
    fallback = Path(tempfile.gettempdir()) / f"forge_engine_amd_{os.getuid()}" / "lib"
    return [PACKAGE_DIR / "lib", fallback]


def library_path(name: str, directory: Path) -> Path:
    return directory / f"fe_{name}.so"


def find_hipcc() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    for candidate in ("/opt/rocm/bin/hipcc",):
        if os.access(candidate, os.X_OK):
            return candidate
    raise KernelBuildError("hipcc not found: the HIP kernels cannot be compiled")


def _writable_dir() -> Path:
    for directory in library_dirs():
        try:
            directory.mkdir(parents=True, exist_ok=True)
            probe = directory / f".probe_{os.getpid()}"
            probe.write_bytes(b"")
            probe.unlink()
            return directory
        except OSError:
            continue
    raise KernelBuildError("no writable folder for the kernel libraries")


def compile_one(name: str, directory: Path | None = None) -> Path:
    """Compile ``csrc/<name>.hip``; returns the library path."""
    source = SOURCE_DIR / f"{name}.hip"
    if not source.exists():
        raise KernelBuildError(f"no kernel source {source}")
    directory = _writable_dir() if directory is None else directory
    target = library_path(name, directory)
    partial = target.with_suffix(f".{os.getpid()}.tmp")
    command = [find_hipcc(), *HIPCC_FLAGS, f'-DFE_SOURCE_HASH="{source_hash(name)}"',
               "-include", str(SOURCE_DIR / "hash_symbol.inc"), "-o", str(partial), str(source)]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    result = subprocess.run(command, capture_output=True, text=True, env=env, cwd=str(SOURCE_DIR))
    if result.returncode != 0:
        partial.unlink(missing_ok=True)
        raise KernelBuildError(f"hipcc failed for {source.name}:\n{result.stderr[-4000:]}")
    os.replace(partial, target)
    return target


def compile_many(names: list[str], *, announce: bool = True, jobs: int | None = None) -> dict[str, Path]:
    """Compile several sources in parallel, printing a line now and then."""
    if not names:
        return {}
    directory = _writable_dir()
    jobs = jobs or min(len(names), max(1, min(8, (os.cpu_count() or 2))))
    done: dict[str, Path] = {}
    lock = threading.Lock()
    started = time.time()

    def work(name: str) -> None:
        path = compile_one(name, directory)
        with lock:
            done[name] = path
            if announce:
                print(f"[forge-engine] compiled {name} ({len(done)}/{len(names)}, "
                      f"{time.time() - started:.0f}s)", file=sys.stderr, flush=True)

    if announce:
        print(f"[forge-engine] compiling {len(names)} HIP kernel libraries for {TARGET_ARCH}: "
              f"{', '.join(names)}", file=sys.stderr, flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        pending = {pool.submit(work, name) for name in names}
        while pending:
            finished, pending = wait(pending, timeout=10.0)
            for future in finished:
                future.result()
            if pending and announce:
                print(f"[forge-engine] still compiling ({len(done)}/{len(names)} done, "
                      f"{time.time() - started:.0f}s)", file=sys.stderr, flush=True)
    return done


def build_all(announce: bool = True) -> dict[str, Path]:
    return compile_many(source_names(), announce=announce)
