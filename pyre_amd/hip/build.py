"""Compiles the HIP sources under ``pyre_amd/csrc`` into one shared library for gfx950.

``ensure_built()`` returns the path of an up-to-date library, compiling what is
missing or older than its source; ``build(force=True)`` compiles everything. The
objects and the library live in ``pyre_amd/csrc/_build`` (or, when that folder
cannot be written, in a per-user temporary folder). Progress goes to stderr so
that a tool's stdout protocol stays clean.
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

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
LIB_NAME = "libpyre_hip.so"

# -packed-fp32-ops off: hipcc must not form packed fp32 instructions from float code.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[pyre_amd build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers() -> list[Path]:
    return sorted(CSRC.glob("*.h"))


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dir() -> Path:
    """The folder that holds objects and the library."""
    env = os.environ.get("PYRE_AMD_BUILD_DIR")
    if env:
        return Path(env)
    in_tree = CSRC / "_build"
    if (in_tree / LIB_NAME).exists() or _writable(in_tree):
        return in_tree
    tag = hashlib.sha1(str(CSRC).encode()).hexdigest()[:10]
    return Path(tempfile.gettempdir()) / f"pyre_amd_build_{os.getuid()}_{tag}"


def _stale(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _compile_one(hipcc: str, src: Path, obj: Path) -> tuple[Path, float]:
    t0 = time.time()
    cmd = [hipcc, *HIPCC_FLAGS, f"-I{CSRC}", "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
    return src, time.time() - t0


def build(force: bool = False, quiet: bool = False) -> Path:
    """Compile stale (or, with ``force``, all) sources and link the library."""
    out = build_dir()
    out.mkdir(parents=True, exist_ok=True)
    lib = out / LIB_NAME
    hdrs = _headers()
    todo = []
    objs = []
    for src in sources():
        obj = out / (src.stem + ".o")
        objs.append(obj)
        if force or _stale(obj, [src, *hdrs]):
            todo.append((src, obj))
    if not todo and lib.exists() and not _stale(lib, objs):
        return lib
    hipcc = _hipcc()
    if todo:
        if not quiet:
            _log(f"compiling {len(todo)} HIP source(s) for {ARCH} into {out} ...")
        workers = max(1, min(len(todo), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
        t0 = time.time()
        with ThreadPoolExecutor(workers) as pool:
            futures = [pool.submit(_compile_one, hipcc, s, o) for s, o in todo]
            for i, fut in enumerate(futures):
                src, dt = fut.result()
                if not quiet:
                    _log(f"  [{i + 1}/{len(todo)}] {src.name} ({dt:.1f} s, {time.time() - t0:.0f} s elapsed)")
    tmp = out / f".{LIB_NAME}.{os.getpid()}"
    proc = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC",
                           *[str(o) for o in objs], "-o", str(tmp)], capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"link failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp, lib)
    if not quiet:
        _log(f"linked {lib}")
    return lib


def ensure_built() -> Path:
    """Path of the library; compiles only when it is missing or out of date."""
    out = build_dir()
    lib = out / LIB_NAME
    srcs = sources()
    if lib.exists() and (not srcs or not _stale(lib, [*srcs, *_headers()])):
        return lib
    return build(force=False)
