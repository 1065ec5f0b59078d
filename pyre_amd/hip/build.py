"""Compiles the HIP sources under ``pyre_amd/csrc`` into one shared library for gfx950.

``ensure_built()`` returns the path of a library built from the sources as they are now,
compiling what is missing or was compiled from other text; ``build(force=True)`` compiles
everything. Nothing goes by file times: an object carries the digest of its source, the
headers and the flags in a file beside it, and the library has the digest of all sources
compiled in (``pyre_sources_digest()``), which the binding checks when it loads it. The
objects and the library live in ``pyre_amd/csrc/_build`` (or, when that folder cannot be
written, in a per-user temporary folder). Progress goes to stderr so that a tool's stdout
protocol stays clean.
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


def _digest(files: list[Path], extra: str = "") -> str:
    h = hashlib.sha1(extra.encode())
    for f in files:
        h.update(f.name.encode() + b"\0" + f.read_bytes() + b"\0")
    return h.hexdigest()


def sources_digest() -> str:
    """A digest of every source, every header and the compiler's flags: what the library
    answers from ``pyre_sources_digest()`` if it was built from this tree."""
    return _digest([*sources(), *_headers()], " ".join(HIPCC_FLAGS))[:16]


#: the source that has the digest of all of them compiled in
_DIGEST_HOLDER = "runtime.hip"


def _object_digest(src: Path, hdrs: list[Path], tree: str) -> str:
    """What an object was compiled from: its source, the headers, the flags (and, for the
    one source that holds it, the digest of the whole tree)."""
    return _digest([src, *hdrs], " ".join(HIPCC_FLAGS) + (tree if src.name == _DIGEST_HOLDER else ""))


def _stamp(path: Path) -> str:
    try:
        return path.with_name(path.name + ".sha1").read_text().strip()
    except OSError:
        return ""


def _write_stamp(path: Path, digest: str) -> None:
    path.with_name(path.name + ".sha1").write_text(digest + "\n")


def _compile_one(hipcc: str, src: Path, obj: Path, digest: str, tree: str) -> tuple[Path, float]:
    t0 = time.time()
    define = [f'-DPYRE_SOURCES_DIGEST="{tree}"'] if src.name == _DIGEST_HOLDER else []
    cmd = [hipcc, *HIPCC_FLAGS, *define, f"-I{CSRC}", "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
    _write_stamp(obj, digest)
    return src, time.time() - t0


def build(force: bool = False, quiet: bool = False) -> Path:
    """Compile stale (or, with ``force``, all) sources and link the library."""
    out = build_dir()
    out.mkdir(parents=True, exist_ok=True)
    lib = out / LIB_NAME
    hdrs = _headers()
    tree = sources_digest()
    todo = []
    objs = []
    for src in sources():
        obj = out / (src.stem + ".o")
        objs.append(obj)
        digest = _object_digest(src, hdrs, tree)
        if force or not obj.exists() or _stamp(obj) != digest:
            todo.append((src, obj, digest))
    if not todo and lib.exists() and _stamp(lib) == tree:
        return lib
    hipcc = _hipcc()
    if todo:
        if not quiet:
            _log(f"compiling {len(todo)} HIP source(s) for {ARCH} into {out} ...")
        workers = max(1, min(len(todo), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
        t0 = time.time()
        with ThreadPoolExecutor(workers) as pool:
            futures = [pool.submit(_compile_one, hipcc, s, o, d, tree) for s, o, d in todo]
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
    _write_stamp(lib, tree)
    if not quiet:
        _log(f"linked {lib}")
    return lib


def ensure_built() -> Path:
    """Path of the library; compiles only when it is missing or was built from other sources."""
    lib = build_dir() / LIB_NAME
    if lib.exists() and (not sources() or _stamp(lib) == sources_digest()):
        return lib
    return build(force=False)
