"""Compile the HIP sources in this folder into one shared library for gfx950.

``hipcc`` is called directly (no torch headers, no ninja): each ``.hip`` file becomes an
object file, in parallel, and the objects are linked into
``flambeau_amd/_build/libflambeau_hip-<hash>.so``.  The hash covers the text of every
source and header and the compiler flags, so a library built from other sources is never
loaded.  When the package folder is not writable the library goes to
``$FLAMBEAU_BUILD_DIR`` or a per-user folder under the system's temporary folder.
"""
from __future__ import annotations

import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    # packed 32-bit float instructions are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-attributes",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers() -> list[Path]:
    return sorted(CSRC.glob("*.h"))


def source_hash() -> str:
    h = hashlib.sha256()
    for p in sources() + _headers():
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("flambeau_amd: hipcc not found (looked at $HIPCC, PATH, /opt/rocm/bin)")


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe-{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dir() -> Path:
    env = os.environ.get("FLAMBEAU_BUILD_DIR")
    if env:
        d = Path(env)
        d.mkdir(parents=True, exist_ok=True)
        return d
    d = CSRC.parent / "_build"
    if _writable(d):
        return d
    d = Path(tempfile.gettempdir()) / f"flambeau_amd-build-{os.getuid()}"
    d.mkdir(parents=True, exist_ok=True)
    return d


def library_path() -> Path:
    return build_dir() / f"libflambeau_hip-{source_hash()}.so"


def _log(msg: str) -> None:
    print(f"[flambeau_amd] {msg}", file=sys.stderr, flush=True)


def _run(cmd: list[str], what: str) -> None:
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"flambeau_amd: {what} failed\n$ {' '.join(cmd)}\n{r.stdout}\n{r.stderr}")


def build(force: bool = False, verbose: bool = True) -> Path:
    """Compile (always when ``force``; otherwise only if the library is missing)."""
    target = library_path()
    if target.exists() and not force:
        return target
    bdir = target.parent
    hipcc = _hipcc()
    with open(bdir / ".lock", "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if target.exists() and not force:
            return target
        t0 = time.time()
        srcs = sources()
        if verbose:
            _log(f"compiling {len(srcs)} HIP sources for {ARCH} into {target}")
        objdir = bdir / f"obj-{source_hash()}"
        objdir.mkdir(parents=True, exist_ok=True)
        done = threading.Event()

        def heartbeat():
            while not done.wait(20.0):
                _log(f"still compiling ({time.time() - t0:.0f} s)")

        hb = threading.Thread(target=heartbeat, daemon=True)
        if verbose:
            hb.start()

        def one(src: Path) -> Path:
            obj = objdir / (src.stem + ".o")
            _run([hipcc, *FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)], f"compiling {src.name}")
            if verbose:
                _log(f"compiled {src.name} ({time.time() - t0:.0f} s)")
            return obj

        try:
            with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
                objs = list(pool.map(one, srcs))
            tmp = target.with_suffix(f".tmp{os.getpid()}.so")
            _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)],
                 "linking")
            os.replace(tmp, target)
        finally:
            done.set()
        shutil.rmtree(objdir, ignore_errors=True)
        for old in bdir.glob("libflambeau_hip-*.so"):
            if old != target:
                try:
                    old.unlink()
                except OSError:
                    pass
        if verbose:
            _log(f"built {target.name} in {time.time() - t0:.0f} s")
    return target


def build_own_library(name: str, srcs: list, out_dir, force: bool = False) -> Path:
    """Compile HIP sources of the caller's own (a part that brings kernels which this library does not
    have) into ``out_dir/lib<name>-<hash>.so``, with this library's flags and with this folder on the
    include path (``api.h`` for ``FlArg``, ``recordable.h`` for the trampoline a step program replays a
    launch function through).  Compiles only if that file is missing, or when ``force``."""
    srcs = [Path(s) for s in srcs]
    h = hashlib.sha256()
    for s in srcs + _headers():
        h.update(s.name.encode())
        h.update(s.read_bytes())
    h.update(" ".join(FLAGS).encode())
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    target = out_dir / f"lib{name}-{h.hexdigest()[:16]}.so"
    if target.exists() and not force:
        return target
    tmp = target.with_suffix(f".tmp{os.getpid()}.so")
    _run([_hipcc(), *FLAGS, "-I", str(CSRC), "-shared", "-o", str(tmp), *map(str, srcs)], f"compiling {name}")
    os.replace(tmp, target)
    for old in out_dir.glob(f"lib{name}-*.so"):
        if old != target:
            try:
                old.unlink()
            except OSError:
                pass
    return target


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
