"""Builds and loads the HIP kernel library (gfx950 only).

The sources under ``csrc/`` are compiled with ``hipcc`` into shared objects (the
core, and one per head size of the matrix-core attention, so that a first call
compiles only what its model needs) whose file names carry a digest of the
sources and flags, so a stale build is never loaded.  Loading looks for that
file first and compiles only if it is missing; compilation prints a line per
file so a first call is visibly alive.
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
_libs = {}

CORE = "kernels"                                   # everything but the matrix-core attention and the measurement kernels
MEASURE = "measure"                                # kernels that only measure the machine; the engine never loads them
ATTENTION_PADS = (32, 64, 96, 128, 160, 192, 224, 256)


class KernelLibraryError(RuntimeError):
    pass


def _log(msg):
    print(f"[runtime.kernels] {msg}", file=sys.stderr, flush=True)


def attention_unit(dpad):
    return f"attn_d{dpad}"


def units():
    """The shared objects the kernels are built into: the core, and one per padded head size of the
    matrix-core attention (a model needs only its own, so a first call compiles only that one)."""
    return [CORE, MEASURE] + [attention_unit(d) for d in ATTENTION_PADS]


def sources(unit=CORE):
    if unit == CORE:
        return sorted(p for p in CSRC.glob("*.hip") if not p.name.startswith("attention_mfma_d") and p.stem != MEASURE)
    if unit == MEASURE:
        return [CSRC / "measure.hip"]
    path = CSRC / f"attention_mfma_{unit[len('attn_'):]}.hip"
    if not path.exists():
        raise KernelLibraryError(f"no source for kernel unit {unit}")
    return [path]


def _digest(unit):
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    included = sorted(p for p in CSRC.iterdir() if p.suffix in (".h", ".inc"))
    for path in sources(unit) + included:
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


def library_path(unit=CORE, create=False):
    name = f"libcisr_{unit}_{_digest(unit)}.so"
    for d in _build_dirs():
        if (d / name).exists():
            return d / name
    if not create:
        return None
    for d in _build_dirs():
        try:
            d.mkdir(parents=True, exist_ok=True)
            fd, probe = tempfile.mkstemp(prefix=".w", dir=str(d))   # (a name of its own: units are built side by side)
            os.close(fd)
            os.unlink(probe)
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


def build_unit(unit, force=False):
    """Compile one unit's sources and link its shared object.  Returns its path."""
    target = library_path(unit, create=True)
    if target.exists() and not force:
        return target
    hipcc = _hipcc()
    work = Path(tempfile.mkdtemp(prefix="obj_", dir=str(target.parent)))
    try:
        srcs = sources(unit)
        with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
            objs = list(pool.map(lambda s: _compile_one(hipcc, s, work / (s.stem + ".o")), srcs))
        tmp = work / target.name
        _log("linking " + target.name)
        proc = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-o", str(tmp)],
                              capture_output=True, text=True)
        if proc.returncode != 0:
            raise KernelLibraryError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
        os.replace(tmp, target)  # atomic: a concurrent loader sees the whole file or none
        for old in target.parent.glob(f"libcisr_{unit}_*.so"):   # builds of other source states
            if old != target:
                try:
                    old.unlink()
                except OSError:
                    pass
    finally:
        shutil.rmtree(work, ignore_errors=True)
    return target


def build(force=False):
    """Compile every unit (the core and every attention head size).  Returns the core's path."""
    with ThreadPoolExecutor(max_workers=4) as pool:
        paths = list(pool.map(lambda u: build_unit(u, force), units()))
    return paths[0]


def ensure(wanted):
    """Build the units of `wanted` that have no current build, side by side."""
    missing = [u for u in dict.fromkeys(wanted) if library_path(u) is None]
    if missing:
        with ThreadPoolExecutor(max_workers=len(missing)) as pool:
            list(pool.map(build_unit, missing))


def load(unit=CORE):
    """The loaded shared object of a unit (built at the first call if no current build exists)."""
    with _lock:
        handle = _libs.get(unit)
        if handle is None:
            path = library_path(unit) or build_unit(unit)
            try:
                handle = ctypes.CDLL(str(path))
            except OSError as exc:
                raise KernelLibraryError(f"cannot load {path}: {exc}") from exc
            handle._cisr_path = str(path)
            _libs[unit] = handle
        return handle


def load_attention(dpad):
    if dpad not in ATTENTION_PADS:
        raise KernelLibraryError(f"no matrix-core attention for a padded head size of {dpad}")
    return load(attention_unit(dpad))


def loaded_path(unit=CORE):
    handle = _libs.get(unit)
    return None if handle is None else handle._cisr_path
