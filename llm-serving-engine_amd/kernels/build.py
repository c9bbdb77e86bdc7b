"""Compiles the HIP sources under `csrc/` for gfx950 into shared libraries and loads them.

Each source file is one library, optionally specialised by preprocessor constants (a head
size, for instance): what a model needs is compiled at its first use and kept, keyed by a
hash of the source, the shared header, the flags and the constants.  Libraries are kept
in-tree under `csrc/_build/` when that is writable, else under the temporary folder.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"

FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-shared",
    "-fPIC",
    "-std=c++17",
    # hipcc's packed-float32 instructions are switched off: some of their forms are unreliable on this hardware
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]

_loaded: dict[Path, ctypes.CDLL] = {}


class BuildError(RuntimeError):
    pass


def _say(message: str) -> None:
    print(f"[llmserve_amd] {message}", file=sys.stderr, flush=True)


def _build_folders() -> list[Path]:
    folders = [CSRC / "_build"]
    folders.append(Path(tempfile.gettempdir()) / f"llmserve_amd-{os.getuid()}" / "_build")
    return folders


def _key(module: str, defines: dict[str, object]) -> str:
    digest = hashlib.sha256()
    digest.update((CSRC / f"{module}.hip").read_bytes())
    for header in sorted(CSRC.glob("*.h")):
        digest.update(header.read_bytes())
    digest.update(" ".join(FLAGS).encode())
    digest.update(repr(sorted(defines.items())).encode())
    return digest.hexdigest()[:12]


def library_name(module: str, defines: dict[str, object] | None = None) -> str:
    defines = defines or {}
    tag = "".join(f"-{name.lower()}{value}" for name, value in sorted(defines.items()))
    return f"{module}{tag}-{_key(module, defines)}.so"


def find_library(module: str, defines: dict[str, object] | None = None) -> Path | None:
    name = library_name(module, defines)
    for folder in _build_folders():
        if (folder / name).is_file():
            return folder / name
    return None


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).is_file():
            return candidate
    raise BuildError("hipcc was not found: the HIP kernels cannot be compiled")


def build_module(module: str, defines: dict[str, object] | None = None, *, force: bool = False) -> Path:
    """Compiles `csrc/<module>.hip` (if not yet built, or `force`) and returns the library's path."""
    defines = defines or {}
    existing = None if force else find_library(module, defines)
    if existing is not None:
        return existing
    source = CSRC / f"{module}.hip"
    if not source.is_file():
        raise BuildError(f"no kernel source {source}")
    name = library_name(module, defines)
    last_error = None
    for folder in _build_folders():
        try:
            folder.mkdir(parents=True, exist_ok=True)
            if not os.access(folder, os.W_OK | os.X_OK):
                raise PermissionError(f"{folder} is not writable")
            partial = folder / f".{name}.{os.getpid()}.tmp"
            command = [_hipcc(), *FLAGS, f"-I{CSRC}"]
            command += [f"-D{key}={value}" for key, value in sorted(defines.items())]
            command += [str(source), "-o", str(partial)]
            tag = "".join(f" {k}={v}" for k, v in sorted(defines.items()))
            _say(f"compiling {module}.hip{tag} for gfx950 ...")
            started = time.monotonic()
            process = subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            while True:
                try:
                    output, _ = process.communicate(timeout=20)
                    break
                except subprocess.TimeoutExpired:
                    _say(f"  still compiling {module}.hip ({time.monotonic() - started:.0f} s)")
            if process.returncode != 0:
                partial.unlink(missing_ok=True)
                raise BuildError(f"hipcc failed for {module}.hip:\n{output}")
            os.replace(partial, folder / name)
            for stale in folder.glob(f"{name.rsplit('-', 1)[0]}-*.so"):  # older builds of the same source
                if stale.name != name:
                    stale.unlink(missing_ok=True)
            _say(f"  built {name} in {time.monotonic() - started:.1f} s")
            return folder / name
        except OSError as error:  # folder not writable: try the next one
            last_error = error
    raise BuildError(f"no writable folder for built kernels: {last_error}")


def load_module(module: str, defines: dict[str, object] | None = None) -> ctypes.CDLL:
    path = build_module(module, defines)
    if path not in _loaded:
        _loaded[path] = ctypes.CDLL(str(path))
    return _loaded[path]


def build_all(variants: dict[str, list[dict[str, object]]], *, force: bool = True) -> list[Path]:
    """Compiles every (module, constants) pair of `variants`."""
    built = []
    for module, all_defines in variants.items():
        for defines in all_defines:
            built.append(build_module(module, defines, force=force))
    return built
