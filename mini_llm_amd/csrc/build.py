"""Compiles the HIP sources of this folder into one shared library for gfx950 with hipcc.

The library lies in-tree (``mini_llm_amd/_lib``) when that folder can be written, else in a
per-user folder under the temp directory. A digest of the sources lies beside it, so a library
built from other sources is not taken for the current one."""

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

CSRC = Path(__file__).resolve().parent
LIBRARY_NAME = "libmini_llm_hip.so"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    # packed 32-bit float instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


class BuildError(RuntimeError):
    pass


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_digest() -> str:
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for path in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()[:24]


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe-{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def library_dirs() -> list[Path]:
    """Where a built library may lie, in the order in which they are looked at."""
    dirs = []
    if os.environ.get("MINI_LLM_AMD_LIB_DIR"):
        dirs.append(Path(os.environ["MINI_LLM_AMD_LIB_DIR"]))
    dirs.append(CSRC.parent / "_lib")
    dirs.append(Path(tempfile.gettempdir()) / f"mini_llm_amd-{os.getuid()}" / "_lib")
    return dirs


def find_built() -> Path | None:
    """The library that was built from the sources as they are now, if there is one."""
    digest = source_digest()
    for folder in library_dirs():
        lib, stamp = folder / LIBRARY_NAME, folder / (LIBRARY_NAME + ".digest")
        try:
            if lib.is_file() and stamp.read_text().strip() == digest:
                return lib
        except OSError:
            continue
    return None


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).is_file():
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _say(message: str, quiet: bool) -> None:
    if not quiet:
        print(f"[mini_llm_amd] {message}", file=sys.stderr, flush=True)


def build(quiet: bool = False) -> Path:
    """Compiles every source and links the library; returns its path. Always compiles."""
    hipcc = _hipcc()
    folder = next((d for d in library_dirs() if _writable(d)), None)
    if folder is None:
        raise BuildError("no writable folder for the kernel library: " + ", ".join(map(str, library_dirs())))
    objects_dir = folder / "_build"
    objects_dir.mkdir(exist_ok=True)
    digest = source_digest()
    started = time.time()

    def compile_one(src: Path) -> Path:
        obj = objects_dir / (src.stem + ".o")
        _say(f"compiling {src.name} for {ARCH}", quiet)
        done = subprocess.run([hipcc, *FLAGS, "-c", str(src), "-o", str(obj)], capture_output=True, text=True)
        if done.returncode != 0:
            raise BuildError(f"hipcc failed on {src.name}:\n{done.stderr}")
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        objects = list(pool.map(compile_one, sources()))
    partial = folder / f".{LIBRARY_NAME}.{os.getpid()}"
    _say("linking", quiet)
    done = subprocess.run(
        [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(partial), *map(str, objects)],
        capture_output=True, text=True,
    )
    if done.returncode != 0:
        raise BuildError(f"linking failed:\n{done.stderr}")
    os.replace(partial, folder / LIBRARY_NAME)  # atomic: another process never sees half a file
    (folder / (LIBRARY_NAME + ".digest")).write_text(digest + "\n")
    _say(f"built {folder / LIBRARY_NAME} in {time.time() - started:.1f} s", quiet)
    return folder / LIBRARY_NAME


def ensure_built(quiet: bool = False) -> Path:
    """The current library; built now if there is none."""
    found = find_built()
    if found is not None:
        return found
    _say("the kernel library is not built yet; building it (about half a minute)", quiet)
    return build(quiet)


if __name__ == "__main__":
    print(build())
