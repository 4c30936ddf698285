"""Compiles ``csrc/*.hip`` for gfx950 into one shared library with hipcc.

The library is built in-tree, next to its sources; when that folder cannot be
written (an installed, read-only checkout) it is built under the temporary
folder instead.  Compilation prints a line per file so a first call on a fresh
checkout shows progress.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC_DIR = Path(__file__).resolve().parent.parent / "csrc"
LIBRARY_NAME = "libminiserve_hip.so"
OFFLOAD_ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
HIPCC_FLAGS = (
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


def _log(message: str) -> None:
    print(f"[miniserve_amd build] {message}", file=sys.stderr, flush=True)


def find_hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate) and os.access(candidate, os.X_OK):
            return candidate
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc).")


def sources() -> list[Path]:
    found = sorted(CSRC_DIR.glob("*.hip"))
    if not found:
        raise RuntimeError(f"no HIP sources under {CSRC_DIR}")
    return found


def source_digest() -> str:
    digest = hashlib.sha256()
    digest.update(" ".join(HIPCC_FLAGS).encode())
    for path in sorted(CSRC_DIR.glob("*.h*")):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    return digest.hexdigest()


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".write_probe_{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def library_locations() -> list[Path]:
    """Where a built library may lie, in order of preference."""

    fallback = Path(tempfile.gettempdir()) / f"miniserve_amd_{os.getuid()}" / source_digest()[:16]
    return [CSRC_DIR / LIBRARY_NAME, fallback / LIBRARY_NAME]


def find_built_library() -> Path | None:
    for path in library_locations():
        if path.is_file():
            return path
    return None


def is_stale(library: Path) -> bool:
    stamp = library.with_suffix(".digest")
    return not stamp.is_file() or stamp.read_text().strip() != source_digest()


def build(*, force: bool = True, jobs: int | None = None) -> Path:
    """Compile every source and link the library; returns its path."""

    existing = find_built_library()
    if existing is not None and not force and not is_stale(existing):
        return existing
    hipcc = find_hipcc()
    in_tree, fallback = library_locations()
    target = in_tree if _writable(in_tree.parent) else fallback
    if target is fallback and not _writable(fallback.parent):
        raise RuntimeError(f"neither {in_tree.parent} nor {fallback.parent} can be written.")
    object_dir = target.parent / "_build"
    object_dir.mkdir(parents=True, exist_ok=True)
    files = sources()
    jobs = jobs or min(len(files), max(1, min(8, os.cpu_count() or 1)))
    _log(f"compiling {len(files)} HIP sources for {OFFLOAD_ARCH} with {jobs} jobs -> {target}")
    started = time.time()

    def compile_one(source: Path) -> Path:
        obj = object_dir / (source.stem + ".o")
        command = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC_DIR), "-c", str(source), "-o", str(obj)]
        result = subprocess.run(command, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed on {source.name}:\n{result.stderr}")
        _log(f"  compiled {source.name} ({time.time() - started:.0f}s)")
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(compile_one, files))
    partial = target.with_suffix(f".tmp{os.getpid()}")
    command = [hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", "-o", str(partial), *map(str, objects), "-ldl"]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed to link {LIBRARY_NAME}:\n{result.stderr}")
    os.replace(partial, target)
    target.with_suffix(".digest").write_text(source_digest() + "\n")
    _log(f"built {target} in {time.time() - started:.0f}s")
    return target


if __name__ == "__main__":
    build(force=True)
