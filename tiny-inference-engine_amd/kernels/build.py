"""Compiling and loading the HIP kernel libraries.

Each library is one ``.hip`` source of ``csrc/`` (plus the shared header) built
with hipcc for gfx950 into ``csrc/_build/<name>-<hash>.so``; the hash covers the
source, the headers it includes, the defines and the flags, so a stale library is never loaded. A
library is compiled the first time it is asked for and found missing - a fresh
checkout builds what its model needs at its first call, printing a line now
and then while hipcc runs - and ``build_all`` compiles everything up front.
When the package folder cannot be written, a per-user folder under the system's
temporary directory takes the built files.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import pathlib
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, Mapping, Optional, Sequence

from ..errors import KernelUnavailable

CSRC = pathlib.Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
# Packed float32 instructions are switched off for all device code.
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

# Flags of single sources. The attention kernels rescale their output accumulators with ordinary
# multiplications between matrix instructions: these then work on vector registers directly.
SOURCE_FLAGS = {"attention_prefill_bf16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
                "attention_decode_bf16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def _log(message: str) -> None:
    print(f"[tie_amd] {message}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise KernelUnavailable("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                            "the HIP kernels cannot be built")


def _build_dir() -> pathlib.Path:
    preferred = CSRC / "_build"
    try:
        preferred.mkdir(parents=True, exist_ok=True)
        if not os.access(preferred, os.W_OK | os.X_OK):
            raise PermissionError(str(preferred))
        return preferred
    except OSError:
        fallback = pathlib.Path(tempfile.gettempdir()) / f"tie_amd_build_{os.getuid()}"
        fallback.mkdir(parents=True, exist_ok=True)
        return fallback


def _candidates(filename: str):
    yield CSRC / "_build" / filename
    yield pathlib.Path(tempfile.gettempdir()) / f"tie_amd_build_{os.getuid()}" / filename


_INCLUDE = re.compile(r'^\s*#\s*include\s+"([^"]+)"', re.MULTILINE)


def _sources_of(source: str):
    """The source file and the headers of ``csrc/`` it includes, directly or through other headers."""
    seen, todo = [], [source]
    while todo:
        name = todo.pop()
        path = CSRC / name
        if name in seen or not path.exists():
            continue
        seen.append(name)
        todo.extend(_INCLUDE.findall(path.read_text()))
    return [CSRC / n for n in sorted(seen)]


def library_filename(name: str, source: str, defines: Mapping[str, object]) -> str:
    h = hashlib.sha256()
    for path in _sources_of(source):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    h.update(repr(sorted((k, str(v)) for k, v in defines.items())).encode())
    h.update(" ".join(FLAGS + SOURCE_FLAGS.get(source, [])).encode())
    return f"{name}-{h.hexdigest()[:12]}.so"


def compile_library(name: str, source: str, defines: Optional[Mapping[str, object]] = None,
                    force: bool = False) -> pathlib.Path:
    """Builds the library unless an up-to-date file exists (or ``force``); returns its path."""
    defines = dict(defines or {})
    filename = library_filename(name, source, defines)
    if not force:
        for path in _candidates(filename):
            if path.exists():
                return path
    out_dir = _build_dir()
    target = out_dir / filename
    tmp = out_dir / f".{filename}.{os.getpid()}.{threading.get_ident()}.tmp"
    cmd = [_hipcc(), *FLAGS, *SOURCE_FLAGS.get(source, []), *[f"-D{k}={v}" for k, v in sorted(defines.items())],
           "-I", str(CSRC),
           "-o", str(tmp), str(CSRC / source)]
    _log(f"compiling {source} -> {target.name} (hipcc, {ARCH})")
    started = time.time()
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()  # hipcc may want a writable home for its caches
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    output = []
    reader = threading.Thread(target=lambda: output.append(proc.stdout.read()), daemon=True)
    reader.start()
    while True:
        try:
            proc.wait(timeout=15)
            break
        except subprocess.TimeoutExpired:
            _log(f"  still compiling {source} ({int(time.time() - started)} s)")
    reader.join()
    text = "".join(output)
    if proc.returncode != 0:
        try:
            tmp.unlink()
        except OSError:
            pass
        raise KernelUnavailable(f"hipcc failed on {source} (exit {proc.returncode}):\n{text[-4000:]}")
    os.replace(tmp, target)
    _log(f"built {target.name} in {time.time() - started:.1f} s")
    # Older builds of the same library are of no use any more.
    for old in out_dir.glob(f"{name}-*.so"):
        if old != target:
            try:
                old.unlink()
            except OSError:
                pass
    return target


def load_library(name: str, source: str, defines: Optional[Mapping[str, object]] = None) -> ctypes.CDLL:
    """The loaded library, compiled first if no up-to-date build exists."""
    key = f"{name}|{sorted((defines or {}).items())}"
    with _lock:
        lib = _loaded.get(key)
        if lib is None:
            path = compile_library(name, source, defines)
            try:
                lib = ctypes.CDLL(str(path))
            except OSError as e:
                raise KernelUnavailable(f"cannot load {path}: {e}") from None
            _loaded[key] = lib
        return lib


def build_all(libraries: Sequence[tuple], force: bool = True, jobs: int = 8) -> None:
    """Compiles ``(name, source, defines)`` libraries side by side."""
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(libraries)))) as pool:
        futures = [pool.submit(compile_library, n, s, d, force) for n, s, d in libraries]
        for f in futures:
            f.result()
