"""Builds the gfx950 kernel library from ``tokasaurus_amd/csrc`` with hipcc.

The library is one shared object loaded through ctypes (no Python headers, no
torch headers), so a fresh checkout builds it in well under a minute and any
user who can write the build folder can do so.  ``ensure_built`` is what the
loader calls: it compiles only when no library matching the current sources
exists, and prints a line per file meanwhile.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
BUILD_DIR = Path(__file__).resolve().parent / "_build"
LIB_NAME = "libtokasaurus_hip.so"

ARCH = "gfx950"
# packed 32-bit float instructions are kept off for every kernel of this library
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Wno-unused-result",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


class BuildError(RuntimeError):
    pass


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise BuildError("hipcc not found: the kernel library cannot be built on this machine")
    return exe


def _digest() -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for p in sorted(CSRC.glob("*")):
        if p.suffix in (".hip", ".h"):
            h.update(p.name.encode())
            h.update(p.read_bytes())
    return h.hexdigest()


def library_path() -> Path:
    return BUILD_DIR / LIB_NAME


def is_current() -> bool:
    stamp = BUILD_DIR / "stamp"
    return library_path().is_file() and stamp.is_file() and stamp.read_text().strip() == _digest()


def _say(msg: str) -> None:
    print(f"[tokasaurus_amd build] {msg}", file=sys.stderr, flush=True)


def _compile_one(hipcc: str, src: Path, obj: Path) -> tuple[Path, float]:
    t0 = time.time()
    cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
    return src, time.time() - t0


def build(force: bool = True, jobs: int | None = None) -> Path:
    """Compile every source and link the library.  ``force=False`` returns at
    once when a library built from the current sources is already there."""
    if not force and is_current():
        return library_path()
    hipcc = _hipcc()
    BUILD_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise BuildError(f"no kernel sources under {CSRC}")
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16)
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} with {jobs} jobs")
    objs = [BUILD_DIR / (s.stem + ".o") for s in srcs]
    t0 = time.time()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(_compile_one, hipcc, s, o) for s, o in zip(srcs, objs)]
        for fut in futures:
            src, dt = fut.result()
            _say(f"  {src.name} done in {dt:.1f}s")
    tmp = BUILD_DIR / (LIB_NAME + f".tmp{os.getpid()}")
    link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"link failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp, library_path())
    (BUILD_DIR / "stamp").write_text(_digest() + "\n")
    _say(f"built {library_path()} in {time.time() - t0:.1f}s")
    return library_path()


def ensure_built() -> Path:
    """The library for the current sources, compiling it if it is not there."""
    if is_current():
        return library_path()
    if library_path().is_file():
        _say("the built library does not match the sources; building again")
    return build(force=True)


if __name__ == "__main__":
    build(force=True)
