"""Building and loading of the HIP kernel library (`csrc/*.hip` -> one shared object for gfx950).

`load()` gives the library through ctypes; if no built library fits the sources it compiles one
first, each file with hipcc in a process of its own, and prints a line for each file so that a
first call in a fresh checkout shows that it is alive.  The library lies beside the sources when
that folder can be written, else in a per-user folder under the system's temporary directory.
There is no other implementation of the kernels: if the library cannot be built or loaded the
error is raised.
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
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
LIB_NAME = "libgeneinfer_gfx950.so"
ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


class KernelBuildError(RuntimeError):
    pass


def _sources():
    return sorted(CSRC.glob("*.hip"))


def source_digest() -> str:
    h = hashlib.sha256()
    for p in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe-{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def _fallback_dir() -> Path:
    return Path(tempfile.gettempdir()) / f"geneinfer-amd-{os.getuid()}" / source_digest()


def _candidates():
    return [CSRC, _fallback_dir()]


def _is_current(folder: Path) -> bool:
    stamp = folder / (LIB_NAME + ".digest")
    return (folder / LIB_NAME).exists() and stamp.exists() and stamp.read_text().strip() == source_digest()


def find_built():
    for folder in _candidates():
        if _is_current(folder):
            return folder / LIB_NAME
    return None


def build(verbose: bool = True) -> Path:
    """Compiles every source for gfx950 and links the library; returns its path."""
    hipcc = _hipcc()
    out_dir = CSRC if _writable(CSRC) else _fallback_dir()
    if not _writable(out_dir):
        raise KernelBuildError(f"neither {CSRC} nor {out_dir} can be written")
    obj_dir = out_dir / "_build"
    obj_dir.mkdir(exist_ok=True)
    sources = _sources()
    if not sources:
        raise KernelBuildError(f"no .hip sources in {CSRC}")
    say = (lambda m: print(f"[geneinfer_amd] {m}", file=sys.stderr, flush=True)) if verbose else (lambda m: None)
    say(f"compiling {len(sources)} HIP sources for {ARCH} into {out_dir}")
    env = dict(os.environ)
    env.setdefault("HOME", str(out_dir))           # hipcc wants a home for its caches

    def compile_one(src: Path):
        t0 = time.time()
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise KernelBuildError(f"hipcc failed on {src.name}:\n{r.stderr[-4000:]}")
        say(f"  compiled {src.name} in {time.time() - t0:.1f} s")
        return obj

    workers = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(compile_one, sources))
    lib = out_dir / LIB_NAME
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(tmp), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise KernelBuildError(f"linking {LIB_NAME} failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib)
    (out_dir / (LIB_NAME + ".digest")).write_text(source_digest() + "\n")
    say(f"built {lib}")
    return lib


_LIB = None


def load() -> ctypes.CDLL:
    """The kernel library, built first if no current build exists."""
    global _LIB
    if _LIB is None:
        path = find_built() or build()
        try:
            _LIB = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from None
        _LIB.gi_last_error.restype = ctypes.c_char_p
    return _LIB
