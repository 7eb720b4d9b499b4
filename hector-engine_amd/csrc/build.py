"""Builds the gfx950 kernel library with hipcc: one object per ``.hip`` file,
compiled in parallel, linked into ``libhector_kernels.so`` next to the sources.

The library is found by :func:`library_path`; :func:`ensure_built` compiles only
when no library matching the current sources exists (a stamp holds the hash of
sources and flags). When the source folder cannot be written (a read-only
checkout) the build goes to a per-user folder under the temporary directory.
"""
from __future__ import annotations

import concurrent.futures
import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

CSRC = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libhector_kernels.so"
ARCH = "gfx950"

# Packed fp32 instructions are switched off for all device code of this library.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the kernel library cannot be built "
                       "(set HIPCC or put /opt/rocm/bin on PATH)")


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def source_hash() -> str:
    h = hashlib.sha256()
    for path in sources() + sorted(glob.glob(os.path.join(CSRC, "*.h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def private_folder() -> str:
    """The per-user folder under the temporary directory (fallback build, tuning file).
    Created with mode 0700; a folder of that name that belongs to someone else, or that
    others may write, is refused: a library found there would be loaded as code."""
    folder = os.path.join(tempfile.gettempdir(), f"hector-engine_amd-{os.getuid()}")
    os.makedirs(folder, mode=0o700, exist_ok=True)
    st = os.lstat(folder)
    import stat
    if not stat.S_ISDIR(st.st_mode) or st.st_uid != os.getuid() or st.st_mode & 0o022:
        raise RuntimeError(f"{folder} is not a private folder of this user (owner {st.st_uid}, "
                           f"mode {stat.S_IMODE(st.st_mode):o}): remove it or set TMPDIR")
    return folder


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _candidate_dirs() -> list[str]:
    """The source folder, then the private fallback (left out when it cannot be trusted)."""
    try:
        return [CSRC, private_folder()]
    except (OSError, RuntimeError):
        return [CSRC]


def _stamp_path(folder: str) -> str:
    return os.path.join(folder, "_build", "stamp")


def _is_current(folder: str, digest: str) -> bool:
    lib = os.path.join(folder, LIB_NAME)
    try:
        with open(_stamp_path(folder)) as f:
            return os.path.exists(lib) and f.read().strip() == digest
    except OSError:
        return False


def library_path() -> str | None:
    """Path of a built library that matches the current sources, or None."""
    digest = source_hash()
    for folder in _candidate_dirs():
        if _is_current(folder, digest):
            return os.path.join(folder, LIB_NAME)
    return None


def _log(msg: str) -> None:
    print(f"[hector-engine_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = True, jobs: int | None = None) -> str:
    """Compiles every kernel source and links the library; returns its path."""
    digest = source_hash()
    if not force:
        found = library_path()
        if found:
            return found
    hipcc = _hipcc()
    folder = next((d for d in _candidate_dirs() if _writable(d)), None)
    if folder is None:
        raise RuntimeError("no writable folder for the kernel library build")
    # objects of this process only: two processes that build at once do not share files
    obj_dir = os.path.join(folder, "_build", f"obj{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    # the product kernels have the most instantiations and take longest: they start first
    srcs = sorted(sources(), key=lambda s: (not os.path.basename(s).startswith("gemm_"), s))
    jobs = jobs or max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    _log(f"compiling {len(srcs)} sources for {ARCH} with {jobs} jobs into {folder}")
    t0 = time.time()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {os.path.basename(src)}:\n{proc.stderr[-6000:]}")
        _log(f"  {os.path.basename(src)} done ({time.time() - t0:.0f} s)")
        return obj

    with concurrent.futures.ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib = os.path.join(folder, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr[-6000:]}")
    os.replace(tmp, lib)
    stamp_tmp = _stamp_path(folder) + f".tmp{os.getpid()}"
    with open(stamp_tmp, "w") as f:
        f.write(digest)
    os.replace(stamp_tmp, _stamp_path(folder))
    shutil.rmtree(obj_dir, ignore_errors=True)
    _log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def ensure_built() -> str:
    return build(force=False)


if __name__ == "__main__":
    print(build(force=True))
