"""Builds libshrike_hip.so from the .hip sources with hipcc for gfx950.

`ensure_built()` is what the package calls when it needs the library: it loads
what is there when the sources have not changed since it was built, and builds
otherwise.  `build(force=True)` always compiles.  The library is placed beside
the sources when that folder can be written, else in a per-user cache folder,
so a fresh checkout compiles what it needs at its first call.
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

CSRC = Path(__file__).resolve().parent
LIB_NAME = "libshrike_hip.so"
ARCH = "gfx950"

# -packed-fp32-ops is switched off: the compiler must not form packed float32
# arithmetic from scalar float code.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    f"--offload-arch={ARCH}",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + os.environ.get("SHRIKE_HIPCC_EXTRA", "").split()


# Flags for single sources.  The attention kernels scale their MFMA accumulators
# between the matrix instructions; in accumulation registers every such step
# would cost a copy out and a copy back.
FILE_FLAGS = {
    "attention_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for path in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()[:16]


def find_hipcc() -> str | None:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        with tempfile.NamedTemporaryFile(dir=folder):
            pass
        return True
    except OSError:
        return False


def _candidate_dirs() -> list[Path]:
    dirs = [CSRC]
    cache = os.environ.get("XDG_CACHE_HOME")
    if cache:
        dirs.append(Path(cache) / "shrike_amd")
    dirs.append(Path(tempfile.gettempdir()) / f"shrike_amd_{os.getuid()}")
    return dirs


def built_library() -> Path | None:
    """Path of a library built from the present sources, if there is one."""
    want = source_hash()
    for folder in _candidate_dirs():
        lib, stamp = folder / LIB_NAME, folder / (LIB_NAME + ".hash")
        if lib.is_file() and stamp.is_file() and stamp.read_text().strip() == want:
            return lib
    return None


def _say(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[shrike_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = True, verbose: bool = True) -> Path:
    """Compile every .hip source and link the shared library; returns its path."""
    if not force:
        lib = built_library()
        if lib is not None:
            return lib
    hipcc = find_hipcc()
    if hipcc is None:
        raise RuntimeError(
            "libshrike_hip.so is not built and hipcc was not found (looked at $HIPCC, PATH and "
            "/opt/rocm/bin/hipcc); the HIP kernels are required, there is no fallback"
        )
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the built library")
    obj_dir = out_dir / "_build"
    obj_dir.mkdir(exist_ok=True)
    srcs = sources()
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}", verbose)
    t0 = time.time()

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *FILE_FLAGS.get(src.name, []), "-I", str(CSRC), "-c", str(src),
               "-o", str(obj)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
        _say(f"  {src.name} done ({time.time() - t0:.0f}s)", verbose)
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed to link {LIB_NAME}:\n{proc.stderr[-4000:]}")
    os.replace(tmp, out_dir / LIB_NAME)
    (out_dir / (LIB_NAME + ".hash")).write_text(source_hash() + "\n")
    _say(f"built {out_dir / LIB_NAME} in {time.time() - t0:.0f}s", verbose)
    return out_dir / LIB_NAME


def ensure_built(verbose: bool = True) -> Path:
    return build(force=False, verbose=verbose)


if __name__ == "__main__":
    print(build(force="--if-needed" not in sys.argv))
