"""Builds the HIP kernel library for gfx950 with hipcc and finds the built file.

The library is keyed by a hash of its sources and flags, so a stale build is never
loaded.  It is built into `csrc/_build/` inside the package when that is writable, else
into a per-user folder under the temporary directory; a fresh checkout compiles at its
first use and prints a line per file meanwhile.
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
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # matrix-core results in ordinary vector registers: no copies to and from the
         # accumulation registers around the float32 work between two products
         "-mllvm", "-amdgpu-mfma-vgpr-form",
         "-Wno-unused-command-line-argument", "-Wno-inline-asm"]


# the vendor library of matrix products, for the plain products with many rows
LINK = ["-L" + os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib"), "-lhipblaslt",
        "-Wl,-rpath," + os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")]


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels cannot be built "
                     "(set HIPCC or install ROCm under /opt/rocm)")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_hash(defines: tuple[str, ...] = ()) -> str:
    h = hashlib.sha256()
    for f in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    h.update(" ".join(FLAGS + LINK + list(defines)).encode())
    return h.hexdigest()[:16]


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dirs() -> list[Path]:
    """Where a built library may live, in order of preference."""
    user = f"tokensprint_amd_{os.getuid()}"
    return [CSRC / "_build", Path(tempfile.gettempdir()) / user]


def library_name() -> str:
    return f"libtokensprint_hip.{source_hash()}.so"


def find_library() -> Path | None:
    name = library_name()
    for d in build_dirs():
        if (d / name).is_file():
            return d / name
    return None


def _say(msg: str) -> None:
    print(f"[tokensprint_amd] {msg}", file=sys.stderr, flush=True)


def _run(cmd: list[str], what: str) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"{what} failed:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")


def build(force: bool = False, verbose: bool = True, jobs: int | None = None) -> Path:
    """Compile every kernel source and link the library; returns its path."""
    found = None if force else find_library()
    if found is not None:
        return found
    hipcc = _hipcc()
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError(f"no writable folder for the kernel library among {build_dirs()}")
    tag = source_hash()
    obj_dir = out_dir / f"obj.{tag}.{os.getpid()}"
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if verbose:
        _say(f"building HIP kernels for {ARCH} ({len(srcs)} files) into {out_dir}")
    t0 = time.time()

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        t = time.time()
        _run([hipcc, *FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)],
             f"compiling {src.name}")
        if verbose:
            _say(f"  compiled {src.name} ({time.time() - t:.1f}s)")
        return obj

    jobs = jobs or min(8, os.cpu_count() or 1, len(srcs))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib = out_dir / library_name()
    tmp = out_dir / f".{lib.name}.{os.getpid()}"
    _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", str(tmp)]
         + [str(o) for o in objs] + LINK, "linking the kernel library")
    os.replace(tmp, lib)
    shutil.rmtree(obj_dir, ignore_errors=True)
    for old in out_dir.glob("libtokensprint_hip.*.so"):
        if old != lib:
            old.unlink(missing_ok=True)
    if verbose:
        _say(f"built {lib.name} in {time.time() - t0:.1f}s")
    return lib
