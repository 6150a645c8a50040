"""Builds the HIP kernels of ``csrc/`` into one shared library for gfx950.

``library_path()`` returns the built library, compiling it first when there is
none or when a source has changed since it was built.  The library is kept inside
the package (``lib/``) when that folder can be written, else under the system's
temporary folder, so that a read-only checkout and an empty HOME both work.
"""
from __future__ import annotations

import hashlib
import json
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor, as_completed
from pathlib import Path
from typing import List, Optional

PACKAGE_DIR = Path(__file__).resolve().parent.parent
CSRC_DIR = PACKAGE_DIR / "csrc"
LIB_NAME = "libqwen_engine_hip.so"
ARCH = "gfx950"

# -packed-fp32-ops: the compiler must not form packed 32-bit float instructions.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    exe = shutil.which("hipcc")
    if exe:
        return exe
    for cand in ("/opt/rocm/bin/hipcc",):
        if os.path.isfile(cand):
            return cand
    raise BuildError("hipcc was not found; the HIP kernels cannot be built")


def sources() -> List[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for p in sorted(list(CSRC_DIR.glob("*.hip")) + list(CSRC_DIR.glob("*.h"))):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe_{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def _lib_dirs() -> List[Path]:
    tmp = Path(tempfile.gettempdir()) / f"qwen_engine_amd_{os.getuid()}"
    return [PACKAGE_DIR / "lib", tmp]


def _stamp_ok(lib_dir: Path, want: str) -> bool:
    lib, stamp = lib_dir / LIB_NAME, lib_dir / "build_stamp.json"
    if not (lib.is_file() and stamp.is_file()):
        return False
    try:
        return json.loads(stamp.read_text()).get("hash") == want
    except (OSError, ValueError):
        return False


def _filter(text: str) -> str:
    keep = [ln for ln in text.splitlines()
            if "packed-fp32-ops" not in ln and ln.strip()]
    return "\n".join(keep)


def _log(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[qwen-engine build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True, jobs: Optional[int] = None) -> Path:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    want = source_hash()
    lib_dir = next((d for d in _lib_dirs() if _writable(d)), None)
    if lib_dir is None:
        raise BuildError("no writable folder for the kernel library")
    obj_dir = lib_dir / "_build"
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise BuildError(f"no HIP sources under {CSRC_DIR}")
    jobs = jobs or max(1, min(8, os.cpu_count() or 1, len(srcs)))
    _log(f"compiling {len(srcs)} HIP sources for {ARCH} with {jobs} jobs into {lib_dir}", verbose)
    t0 = time.time()

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC_DIR), "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise BuildError(f"hipcc failed on {src.name}:\n{_filter(r.stdout + r.stderr)}")
        return obj

    objs = []
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = {pool.submit(compile_one, s): s for s in srcs}
        for n, fut in enumerate(as_completed(futures), 1):
            objs.append(fut.result())
            _log(f"  [{n}/{len(srcs)}] {futures[fut].name} ({time.time() - t0:.0f} s)", verbose)
    tmp_lib = lib_dir / f".{LIB_NAME}.{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp_lib)] + [str(o) for o in sorted(objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise BuildError(f"linking the kernel library failed:\n{_filter(r.stdout + r.stderr)}")
    os.replace(tmp_lib, lib_dir / LIB_NAME)
    (lib_dir / "build_stamp.json").write_text(json.dumps({"hash": want, "arch": ARCH}))
    _log(f"built {lib_dir / LIB_NAME} in {time.time() - t0:.0f} s", verbose)
    return lib_dir / LIB_NAME


def library_path(verbose: bool = True) -> Path:
    """The built library that matches the sources; builds it when there is none."""
    want = source_hash()
    for d in _lib_dirs():
        if _stamp_ok(d, want):
            return d / LIB_NAME
    return build(verbose=verbose)
