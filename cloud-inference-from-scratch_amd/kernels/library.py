"""Build and load the HIP kernel library (``csrc/*.hip`` -> one shared object).

The library is plain ``extern "C"`` entry points compiled by ``hipcc`` for
gfx950 and loaded with ``ctypes``; it links neither Python nor torch.  It is
built in-tree under ``csrc/_build`` (or, where the tree is read-only, in a
per-user folder under the temporary directory).  A stamp of the sources' hash
lies beside the built file; a stale or missing library is rebuilt at the first
call, each source printing a line as it finishes.  There is no fallback: if
the library can be neither loaded nor built, :func:`load_library` raises.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import re
import shutil
import stat
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import Any

CSRC = Path(__file__).resolve().parent.parent / "csrc"
LIB_NAME = "libcie_kernels.so"
ARCH = "gfx950"
# Packed float32 instructions are switched off for every kernel of this library.
HIPCC_FLAGS = [
    "-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

# The products with many rows go through the vendor's library (csrc/gemm_library.hip).
LINK_LIBS = ["-lhipblaslt"]

_lock = threading.Lock()
_library: ctypes.CDLL | None = None


class KernelLibraryError(RuntimeError):
    """The HIP kernel library is missing and could not be built."""


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_hash() -> str:
    digest = hashlib.sha256()
    for path in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    digest.update(" ".join(HIPCC_FLAGS + LINK_LIBS).encode())
    return digest.hexdigest()


def _hipcc() -> str | None:
    found = shutil.which("hipcc")
    if found:
        return found
    candidate = Path(os.environ.get("ROCM_PATH", "/opt/rocm")) / "bin" / "hipcc"
    return str(candidate) if candidate.is_file() else None


def _fallback_dir() -> Path:
    return Path(tempfile.gettempdir()) / f"cie_amd_build_{os.getuid()}"


def _private_to_this_user(folder: Path) -> bool:
    """The fallback folder has a name anyone can guess, in a place anyone can write: it is used only if
    it is a real folder of this user's that nobody else can write into.  Otherwise another user could
    have put a library there that this process would load and run."""
    try:
        folder.mkdir(mode=0o700, exist_ok=True)
        info = folder.lstat()
    except OSError:
        return False
    return stat.S_ISDIR(info.st_mode) and info.st_uid == os.getuid() and not info.st_mode & 0o022


def _build_dirs() -> list[Path]:
    """Where a built library may lie: in the tree, else in this user's own folder under the temporary directory."""
    fallback = _fallback_dir()
    return [CSRC / "_build"] + ([fallback] if _private_to_this_user(fallback) else [])


def _log(message: str) -> None:
    print(f"[cie_amd build] {message}", file=sys.stderr, flush=True)


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe_{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def build_library(force: bool = True) -> Path:
    """Compile every ``.hip`` source for gfx950 and link the shared object.

    Works without a GPU (hipcc cross-compiles).  Returns the library's path."""
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelLibraryError("hipcc not found (looked on PATH and under $ROCM_PATH/bin)")
    folder = next((d for d in _build_dirs() if _writable(d)), None)
    if folder is None:
        raise KernelLibraryError(f"no writable build folder among {[str(d) for d in _build_dirs()]}")
    wanted = source_hash()
    target = folder / LIB_NAME
    stamp = folder / "sources.sha256"
    if not force and target.is_file() and stamp.is_file() and stamp.read_text().strip() == wanted:
        return target
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = str(folder)  # hipcc wants a writable home for its temporary files
    files = sources()
    _log(f"compiling {len(files)} HIP sources for {ARCH} into {folder}")
    started = time.time()
    # objects of this build alone: two processes that build at once do not write each other's files
    objects_dir = Path(tempfile.mkdtemp(prefix="objects_", dir=folder))

    def compile_one(path: Path) -> Path:
        obj = objects_dir / (path.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(path), "-o", str(obj)]
        done = subprocess.run(cmd, env=env, capture_output=True, text=True)
        if done.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {path.name}:\n{done.stderr[-4000:]}")
        _log(f"  {path.name} done ({time.time() - started:.0f}s)")
        return obj

    workers = max(1, min(len(files), os.cpu_count() or 4, 8))
    try:
        with ThreadPoolExecutor(max_workers=workers) as pool:
            objects = list(pool.map(compile_one, files))
        scratch = objects_dir / LIB_NAME
        link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(scratch), *map(str, objects), *LINK_LIBS]
        done = subprocess.run(link, env=env, capture_output=True, text=True)
        if done.returncode != 0:
            raise KernelLibraryError(f"linking {LIB_NAME} failed:\n{done.stderr[-4000:]}")
        os.replace(scratch, target)  # (same file system: the finished library appears at once)
    finally:
        shutil.rmtree(objects_dir, ignore_errors=True)
    stamp.write_text(wanted + "\n")
    _log(f"built {target} in {time.time() - started:.0f}s")
    return target


def find_built(check_stamp: bool = True) -> Path | None:
    wanted = source_hash() if check_stamp else None
    for folder in _build_dirs():
        target = folder / LIB_NAME
        stamp = folder / "sources.sha256"
        if target.is_file():
            if not check_stamp or (stamp.is_file() and stamp.read_text().strip() == wanted):
                return target
    return None


_C_TYPES = {"int": ctypes.c_int, "long": ctypes.c_long, "size_t": ctypes.c_size_t, "float": ctypes.c_float}
_ENTRY_POINT = re.compile(r"CIE_API\s+int\s+(\w+)\s*\(([^)]*)\)")


def entry_point_signatures() -> dict[str, list[Any]]:
    """The argument types of every ``CIE_API int name(...)`` in the sources, read from their text (the
    library that is loaded was built from exactly these sources): a pointer of any kind is an address,
    scalars are ``int``, ``long``, ``size_t`` or ``float``.  Anything else is an error, not a guess."""
    found: dict[str, list[Any]] = {}
    for path in sources():
        for name, params in _ENTRY_POINT.findall(path.read_text()):
            types: list[Any] = []
            for param in params.split(","):
                words = param.replace("*", " * ").split()
                if "*" in words:
                    types.append(ctypes.c_void_p)
                    continue
                kind = [w for w in words[:-1] if w not in ("const", "unsigned")]
                if len(kind) != 1 or kind[0] not in _C_TYPES or "unsigned" in words:
                    raise KernelLibraryError(f"{path.name}: cannot read the parameter '{param.strip()}' of {name}")
                types.append(_C_TYPES[kind[0]])
            if name in found:
                raise KernelLibraryError(f"entry point {name} is defined twice")
            found[name] = types
    return found


def load_library() -> ctypes.CDLL:
    """The loaded kernel library; built first if nothing current is there."""
    global _library
    with _lock:
        if _library is not None:
            return _library
        path = find_built(check_stamp=True)
        if path is None:
            # (a library built from other sources is never loaded: its entry points may take other arguments)
            path = build_library(force=False)
        try:
            _library = ctypes.CDLL(str(path))
        except OSError as exc:
            raise KernelLibraryError(f"cannot load {path}: {exc}") from exc
        # declared once: calls then pass plain Python numbers and addresses, which costs a fraction of
        # building a ctypes object per argument
        for name, types in entry_point_signatures().items():
            function = getattr(_library, name)
            function.argtypes = types
            function.restype = ctypes.c_int
        _library.cie_path = str(path)  # type: ignore[attr-defined]
        return _library
