"""Compiles the HIP sources under ``csrc/`` for gfx950 and loads the resulting library.

The library's file name carries a hash of every source, header and compiler flag, so a library that
was built from other sources is never loaded by mistake: when no file with the current hash exists
the sources are compiled at that first call (each ``.hip`` file by its own ``hipcc`` process, a few
at a time), with a progress line on standard error now and then. Objects and libraries go to
``csrc/_build`` when that folder can be written, else to a per-user folder under the system's
temporary directory. There is no fallback: without the library every kernel call raises.
"""

from __future__ import annotations

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
# -packed-fp32-ops is switched off: the compiler must not form packed 32-bit float instructions.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core accumulators stay in ordinary vector registers: no moves to and from the
    # accumulation registers around the online softmax's rescaling
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
]
LIB_STEM = "libdli_hip"

_lock = threading.Lock()
_library: ctypes.CDLL | None = None


class KernelBuildError(RuntimeError):
    """The HIP library could not be compiled or loaded."""


def _say(msg: str) -> None:
    print(f"[dli_amd] {msg}", file=sys.stderr, flush=True)


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers() -> list[Path]:
    return sorted(CSRC.glob("*.h"))


def _digest(paths: list[Path], extra: str = "") -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(extra.encode())
    for p in paths:
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()[:16]


def library_hash() -> str:
    return _digest(sources() + _headers())


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe-{os.getpid()}-{threading.get_ident()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dirs() -> list[Path]:
    """Folders that may hold a built library, in order of preference."""
    dirs = [CSRC / "_build"]
    env = os.environ.get("DLI_AMD_BUILD_DIR")
    if env:
        dirs.insert(0, Path(env))
    dirs.append(Path(tempfile.gettempdir()) / f"dli_amd_build_{os.getuid()}")
    return dirs


def find_library() -> Path | None:
    name = f"{LIB_STEM}-{library_hash()}.so"
    for d in build_dirs():
        if (d / name).is_file():
            return d / name
    return None


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).is_file():
            return cand
    raise KernelBuildError(
        "hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be "
        "compiled, and the engine has no other implementation to fall back on"
    )


def _run(cmd: list[str], what: str) -> None:
    start = time.monotonic()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    done = threading.Event()

    def ticker() -> None:
        while not done.wait(15.0):
            _say(f"still compiling {what} ({time.monotonic() - start:.0f} s)")

    t = threading.Thread(target=ticker, daemon=True)
    t.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise KernelBuildError(f"hipcc failed on {what}:\n{' '.join(cmd)}\n{out}")


def build(force: bool = False, verbose: bool = True) -> Path:
    """Compile what is missing (everything with ``force``) and return the library's path."""
    hipcc = _hipcc()
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise KernelBuildError(f"no writable build folder among {[str(d) for d in build_dirs()]}")
    lib = out_dir / f"{LIB_STEM}-{library_hash()}.so"
    if lib.is_file() and not force:
        return lib
    srcs, hdrs = sources(), _headers()
    if not srcs:
        raise KernelBuildError(f"no .hip sources under {CSRC}")
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    jobs: list[tuple[Path, Path]] = []
    objects: list[Path] = []
    for src in srcs:
        obj = out_dir / f"{src.stem}-{_digest([src] + hdrs)}.o"
        objects.append(obj)
        if force or not obj.is_file():
            jobs.append((src, obj))

    def compile_one(job: tuple[Path, Path]) -> None:
        src, obj = job
        tmp = obj.with_suffix(f".tmp{os.getpid()}.o")
        _run([hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(tmp)], src.name)
        os.replace(tmp, obj)
        if verbose:
            _say(f"compiled {src.name}")

    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "8")), 16))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(compile_one, jobs))
    tmp_lib = lib.with_suffix(f".tmp{os.getpid()}.so")
    # the vendor's matrix-product library (gemm_lt.hip calls it) lies beside the compiler
    rocm_lib = Path(os.path.realpath(hipcc)).parent.parent / "lib"
    link = [f"-L{rocm_lib}", f"-Wl,-rpath,{rocm_lib}"] if rocm_lib.is_dir() else []
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp_lib), *map(str, objects), *link,
          "-lhipblaslt"], lib.name)
    os.replace(tmp_lib, lib)
    keep = {lib.name, *(o.name for o in objects)}
    for stale in list(out_dir.glob(f"{LIB_STEM}-*.so")) + list(out_dir.glob("*.o")):
        if stale.name not in keep and ".tmp" not in stale.name:
            try:
                stale.unlink()  # built from sources that have changed since
            except OSError:
                pass
    if verbose:
        _say(f"built {lib.name}")
    return lib


def load() -> ctypes.CDLL:
    """The loaded library; compiled first when no library of the current sources exists."""
    global _library
    with _lock:
        if _library is None:
            path = find_library()
            if path is None:
                path = build()
            try:
                _library = ctypes.CDLL(str(path))
            except OSError as exc:
                raise KernelBuildError(f"cannot load {path}: {exc}") from exc
            _library._dli_path = str(path)  # type: ignore[attr-defined]
        return _library


def loaded_path() -> str | None:
    return getattr(_library, "_dli_path", None) if _library is not None else None
