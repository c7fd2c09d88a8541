"""Compile the HIP sources of this folder into one shared library for gfx950.

    python -m tokenmill_amd.csrc.build            # build (or rebuild) in place

The library is built with hipcc alone (no torch headers), so a first build in a fresh checkout
takes well under a minute. Objects are compiled in parallel and a line is printed for each.
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
LIB_NAME = "libtokenmill_hip.so"
ARCH = "gfx950"
# -packed-fp32-ops off: hipcc's packed 32-bit float instructions are kept out of every kernel.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


# the library matrix products (gemm_library.hip) call hipBLASLt
LINK_LIBS = ["-lhipblaslt"]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_digest() -> str:
    h = hashlib.sha256()
    for p in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(HIPCC_FLAGS + LINK_LIBS).encode())
    return h.hexdigest()[:16]


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe{os.getpid()}"
        probe.write_text("x")
        probe.unlink()
        return True
    except OSError:
        return False


def lib_dirs() -> list[Path]:
    """Where a built library may live: in the tree first, else a per-user folder under the temp dir."""
    return [CSRC.parent / "_lib", Path(tempfile.gettempdir()) / f"tokenmill_amd-{os.getuid()}" / "_lib"]


def find_library() -> Path | None:
    """A built library that matches the current sources, if there is one."""
    digest = source_digest()
    for d in lib_dirs():
        lib, stamp = d / LIB_NAME, d / (LIB_NAME + ".digest")
        if lib.exists() and stamp.exists() and stamp.read_text().strip() == digest:
            return lib
    return None


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the HIP kernels of tokenmill_amd cannot be built")
    return exe


def build(verbose: bool = True) -> Path:
    """Compile every .hip file and link the library; returns its path."""
    out_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable folder for the kernel library among {lib_dirs()}")
    obj_dir = out_dir / "obj"
    obj_dir.mkdir(exist_ok=True)
    cc = hipcc()
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()          # the compiler wants a writable home for its caches

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        if verbose:
            print(f"[tokenmill_amd] hipcc {src.name} ({ARCH})", flush=True)
        t0 = time.monotonic()
        r = subprocess.run([cc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)],
                           capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src.name}:\n{r.stdout}\n{r.stderr}")
        if verbose:
            print(f"[tokenmill_amd] {src.name} compiled in {time.monotonic() - t0:.0f} s", flush=True)
        return obj

    # the largest sources first: they take the longest, and the build is over when the last of them is
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 4)) as pool:
        objs = list(pool.map(compile_one, sorted(sources(), key=lambda p: -p.stat().st_size)))
    lib = out_dir / LIB_NAME
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    r = subprocess.run([cc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(tmp), *map(str, objs), *LINK_LIBS],
                       capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, lib)
    (out_dir / (LIB_NAME + ".digest")).write_text(source_digest())
    if verbose:
        print(f"[tokenmill_amd] built {lib}", flush=True)
    return lib


if __name__ == "__main__":
    build()
    sys.exit(0)
