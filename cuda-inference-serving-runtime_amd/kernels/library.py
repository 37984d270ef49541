"""Builds and loads the HIP kernel library (gfx950 only).

The sources under ``csrc/`` are compiled with ``hipcc`` into one shared object
whose file name carries a digest of the sources and flags, so a stale build is
never loaded.  Loading looks for that file first and compiles only if it is
missing; compilation prints a line per file so a first call is visibly alive.
There is no fallback: if the library cannot be built or loaded, or no GPU is
present when a kernel is called, an error is raised.
"""
import ctypes
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

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    # packed-float instructions are kept out of the device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

_lock = threading.Lock()
_lib = None


class KernelLibraryError(RuntimeError):
    pass


def _log(msg):
    print(f"[runtime.kernels] {msg}", file=sys.stderr, flush=True)


def sources():
    return sorted(CSRC.glob("*.hip"))


def _digest():
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for path in sorted(p for p in CSRC.iterdir() if p.suffix in (".hip", ".h", ".inc")):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()[:16]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise KernelLibraryError("hipcc not found: the HIP kernel library cannot be built")


def _build_dirs():
    """In-tree first (it travels with the checkout); a per-user temporary
    folder when the tree is read-only."""
    yield CSRC / "_build"
    yield Path(tempfile.gettempdir()) / f"cisr_amd_build_{os.getuid()}"


def library_path(create=False):
    name = f"libcisr_kernels_{_digest()}.so"
    for d in _build_dirs():
        if (d / name).exists():
            return d / name
    if not create:
        return None
    for d in _build_dirs():
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".w{os.getpid()}"
            probe.write_text("")
            probe.unlink()
            return d / name
        except OSError:
            continue
    raise KernelLibraryError("no writable folder for the kernel build")


def _compile_one(hipcc, src, obj):
    t0 = time.time()
    _log(f"compiling {src.name} for {ARCH} ...")
    proc = subprocess.run([hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise KernelLibraryError(f"hipcc failed on {src.name}:\n{proc.stdout}\n{proc.stderr}")
    _log(f"compiled {src.name} in {time.time() - t0:.1f} s")
    return obj


def build(force=False):
    """Compile every kernel source and link the shared library.  Returns its path."""
    target = library_path(create=True)
    if target.exists() and not force:
        return target
    hipcc = _hipcc()
    work = Path(tempfile.mkdtemp(prefix="obj_", dir=str(target.parent)))
    try:
        srcs = sources()
        with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
            objs = list(pool.map(lambda s: _compile_one(hipcc, s, work / (s.stem + ".o")), srcs))
        tmp = work / target.name
        _log("linking " + target.name)
        proc = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)],
                              capture_output=True, text=True)
        if proc.returncode != 0:
            raise KernelLibraryError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
        os.replace(tmp, target)  # atomic: a concurrent loader sees the whole file or none
        for old in target.parent.glob("libcisr_kernels_*.so"):   # builds of other source states
            if old != target:
                try:
                    old.unlink()
                except OSError:
                    pass
    finally:
        shutil.rmtree(work, ignore_errors=True)
    return target


def load():
    """The loaded library (built at the first call if no current build exists)."""
    global _lib
    with _lock:
        if _lib is None:
            path = library_path() or build()
            try:
                _lib = ctypes.CDLL(str(path))
            except OSError as exc:
                raise KernelLibraryError(f"cannot load {path}: {exc}") from exc
            _lib._cisr_path = str(path)
        return _lib


def loaded_path():
    return None if _lib is None else _lib._cisr_path
