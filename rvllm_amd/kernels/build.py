"""Builds the HIP kernels into one shared library with hipcc, for gfx950.

The library's file name carries a hash of the sources and flags, so a library
built from other sources is never loaded by mistake.  ``ensure_built`` compiles
only when no library with the current hash exists; ``build(force=True)``
compiles always.  Objects are compiled in parallel, one hipcc call per source
file, and a line is printed as each one finishes so that a first call in a
fresh checkout shows progress.

The library goes to ``rvllm_amd/_lib`` when that can be written, else to a
folder under the system's temporary directory (a read-only checkout, an
empty HOME).
"""

from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
# Packed 32-bit float instructions stay off for every kernel.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # A wave finds its kernel's first arguments in registers when it starts instead of fetching them: a decode
    # step is some 370 short kernels one after the other, and each starts that much sooner (about 3 % of a step).
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",  # the copies into LDS name the register m0, which the compiler calls reserved
]
# The products of many rows go to hipBLASLt (csrc/library_gemm.hip).
LINK_FLAGS = ["-lhipblaslt"]
LIB_STEM = "librvllm_amd"


def _sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers() -> list[Path]:
    return sorted(list(CSRC.glob("*.h")) + list(CSRC.glob("*.inc")))


def source_hash() -> str:
    h = hashlib.sha256()
    for path in _sources() + _headers():
        h.update(path.name.encode())
        h.update(path.read_bytes())
    h.update(" ".join(HIPCC_FLAGS + LINK_FLAGS).encode())
    return h.hexdigest()[:12]


def _candidate_dirs() -> list[Path]:
    dirs = [Path(__file__).resolve().parent.parent / "_lib"]
    env = os.environ.get("RVLLM_AMD_BUILD_DIR")
    if env:
        dirs.insert(0, Path(env))
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(Path(tempfile.gettempdir()) / f"rvllm_amd_build_{uid}")
    return dirs


def _writable_dir() -> Path:
    for d in _candidate_dirs():
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".probe_{os.getpid()}"
            probe.write_bytes(b"")
            probe.unlink()
            return d
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel library: tried " + ", ".join(map(str, _candidate_dirs())))


def library_name() -> str:
    return f"{LIB_STEM}_{source_hash()}.so"


def find_library() -> Path | None:
    name = library_name()
    for d in _candidate_dirs():
        p = d / name
        if p.is_file():
            return p
    return None


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _say(msg: str) -> None:
    print(f"[rvllm_amd build] {msg}", file=sys.stderr, flush=True)


def _compile_one(hipcc: str, src: Path, obj: Path) -> tuple[Path, float, str]:
    t0 = time.time()
    cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
    return src, time.time() - t0, proc.stderr


def build(force: bool = True, jobs: int | None = None) -> Path:
    """Compile every source and link the library; returns its path."""
    existing = find_library()
    if existing is not None and not force:
        return existing
    hipcc = _hipcc()
    out_dir = _writable_dir()
    name = library_name()
    srcs = _sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    jobs = jobs or min(len(srcs), max(1, min(16, (os.cpu_count() or 4))))
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir / name} ({jobs} at a time)")
    t0 = time.time()
    with tempfile.TemporaryDirectory(dir=out_dir, prefix="obj_") as tmp:
        objs = []
        with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
            futures = []
            for src in srcs:
                obj = Path(tmp) / (src.stem + ".o")
                objs.append(obj)
                futures.append(pool.submit(_compile_one, hipcc, src, obj))
            done = 0
            for fut in concurrent.futures.as_completed(futures):
                src, secs, _ = fut.result()
                done += 1
                _say(f"  [{done}/{len(srcs)}] {src.name} ({secs:.1f} s)")
        tmp_lib = Path(tmp) / name
        link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp_lib), *map(str, objs), *LINK_FLAGS]
        proc = subprocess.run(link, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr[-4000:]}")
        os.replace(tmp_lib, out_dir / name)  # atomic: a concurrent reader sees all or nothing
    for old in out_dir.glob(f"{LIB_STEM}_*.so"):
        if old.name != name:
            try:
                old.unlink()
            except OSError:
                pass
    _say(f"done in {time.time() - t0:.1f} s")
    return out_dir / name


def ensure_built() -> Path:
    return build(force=False)


if __name__ == "__main__":
    print(build(force=True))
