"""Compiles the HIP sources of this folder for gfx950 and loads them through ctypes.

Each library is a group of ``.hip`` files linked into one shared object next to the
sources (or, where that folder cannot be written, under a per-user temporary
folder). ``load(name)`` loads what is built and compiles first only if nothing
usable is there; ``build_all()`` always compiles. There is no fallback: a missing
compiler with a missing library is an error, and so is a library that is older than
its sources and cannot be rebuilt (``KESTREL_AMD_ALLOW_STALE=1`` loads it all the same,
with a warning).
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path
from typing import Dict, List

SOURCE_DIR = Path(__file__).resolve().parent
ARCH = "gfx950"

# library name -> its sources. "core" is all a float32 run needs; "fast" holds the
# bf16 MFMA kernels of serving.
LIBRARIES: Dict[str, List[str]] = {
    "core": ["ka_error.hip", "elementwise.hip", "gemm_generic.hip", "attention_generic.hip", "sampling.hip", "peaks.hip"],
    "fast": ["ka_error.hip", "gemm_bf16.hip", "gemv_bf16.hip", "attention_bf16.hip", "decode_beside.hip", "gemm_library.hip"],
}
HEADERS = ["ka_common.h", "ka_partials.h", "ka_no_alloc.h", "ka_attention_decode.h", "ka_skinny.h"]

# Libraries of the ROCm installation that a library of ours is linked against.
LINK_LIBRARIES: Dict[str, List[str]] = {"fast": ["hipblaslt"]}

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    """The HIP library could not be built or loaded."""


def _say(message: str) -> None:
    print(f"[kestrel_amd build] {message}", file=sys.stderr, flush=True)


def _sources(name: str) -> List[Path]:
    return [SOURCE_DIR / s for s in LIBRARIES[name] if (SOURCE_DIR / s).exists()]


def source_stamp(name: str) -> str:
    """Hash of the sources, headers and flags a library is built from."""
    digest = hashlib.sha256()
    digest.update(" ".join(HIPCC_FLAGS + LINK_LIBRARIES.get(name, [])).encode())
    for path in [SOURCE_DIR / h for h in HEADERS] + _sources(name):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    return digest.hexdigest()[:16]


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def _candidate_dirs() -> List[Path]:
    dirs = []
    override = os.environ.get("KESTREL_AMD_BUILD_DIR")
    if override:
        dirs.append(Path(override))
    dirs.append(SOURCE_DIR)
    dirs.append(Path(tempfile.gettempdir()) / f"kestrel_amd_{os.getuid()}")
    return dirs


def library_path(name: str, folder: Path) -> Path:
    return folder / f"libka_{name}.so"


def _find_built(name: str):
    """(path, fresh) of the first library found; fresh says its stamp matches the sources."""
    stamp = source_stamp(name)
    stale = None
    for folder in _candidate_dirs():
        path = library_path(name, folder)
        if path.exists():
            stamp_file = path.with_suffix(".stamp")
            if stamp_file.exists() and stamp_file.read_text().strip() == stamp:
                return path, True
            stale = stale or path
    return stale, False


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return candidate
    raise KernelBuildError("hipcc not found: the HIP kernels cannot be compiled (no fallback exists)")


def build(name: str, verbose: bool = True) -> Path:
    """Compile one library and return the path of the shared object."""
    sources = _sources(name)
    if len(sources) != len(LIBRARIES[name]):
        missing = [s for s in LIBRARIES[name] if not (SOURCE_DIR / s).exists()]
        raise KernelBuildError(f"library {name!r}: sources missing: {missing}")
    hipcc = _hipcc()
    folder = next((d for d in _candidate_dirs() if _writable(d)), None)
    if folder is None:
        raise KernelBuildError("no writable folder for the compiled HIP library")
    objdir = folder / f"_build_{name}"
    objdir.mkdir(parents=True, exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    started = time.time()
    if verbose:
        _say(f"compiling library '{name}' ({len(sources)} files) for {ARCH} into {folder}")
    procs = []
    for src in sources:
        obj = objdir / (src.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", str(SOURCE_DIR), "-c", str(src), "-o", str(obj)]
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env)))
    objects = []
    pending = list(procs)
    last_note = time.time()
    while pending:
        for item in list(pending):
            src, obj, proc = item
            if proc.poll() is None:
                continue
            pending.remove(item)
            output = proc.stdout.read().decode(errors="replace")
            if proc.returncode != 0:
                for _, _, other in pending:
                    other.kill()
                raise KernelBuildError(f"hipcc failed on {src.name}:\n{output}")
            if verbose:
                _say(f"  compiled {src.name} ({time.time() - started:.0f} s)")
            objects.append(obj)
        if pending:
            time.sleep(0.2)
            if verbose and time.time() - last_note > 15:
                names = ", ".join(s.name for s, _, _ in pending)
                _say(f"  still compiling {names} ({time.time() - started:.0f} s)")
                last_note = time.time()
    target = library_path(name, folder)
    partial = target.with_suffix(f".tmp{os.getpid()}")
    rocm_lib = Path(hipcc).resolve().parent.parent / "lib"
    links = [f"-L{rocm_lib}", f"-Wl,-rpath,{rocm_lib}"] + [f"-l{lib}" for lib in LINK_LIBRARIES.get(name, [])]
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(partial), *map(str, sorted(objects)), *links]
    done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env)
    if done.returncode != 0:
        raise KernelBuildError(f"linking {target.name} failed:\n{done.stdout.decode(errors='replace')}")
    os.replace(partial, target)
    target.with_suffix(".stamp").write_text(source_stamp(name))
    shutil.rmtree(objdir, ignore_errors=True)
    if verbose:
        _say(f"built {target.name} in {time.time() - started:.0f} s")
    return target


def build_all(verbose: bool = True) -> List[Path]:
    return [build(name, verbose) for name in LIBRARIES if _sources(name)]


def load(name: str) -> ctypes.CDLL:
    """The loaded library; built first if none is there or the sources have changed."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        path, fresh = _find_built(name)
        if path is None or not fresh:
            try:
                path = build(name)
            except KernelBuildError as exc:
                if path is None:
                    raise
                if os.environ.get("KESTREL_AMD_ALLOW_STALE") != "1":
                    raise KernelBuildError(
                        f"{path} is older than its sources and could not be rebuilt ({exc}); a stale library would run "
                        f"other code than the sources say. Build it where hipcc is, or set KESTREL_AMD_ALLOW_STALE=1 "
                        f"to load it as it is") from exc
                _say(f"warning: {path.name} is older than its sources and could not be rebuilt; loading it as it is "
                     f"(KESTREL_AMD_ALLOW_STALE=1)")
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as exc:
            raise KernelBuildError(f"cannot load {path}: {exc}") from exc
        _loaded[name] = lib
        return lib
