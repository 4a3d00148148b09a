"""Compiles csrc/*.hip for gfx950 into one shared library with hipcc.

`ensure_built()` is what the kernel loader calls: it compiles when no library
matching the sources' hash is there, into `_lib/` beside the package or, if that
place cannot be written, into a per-user folder under the temp directory.
`build(force=True)` always compiles.  A progress line goes to stderr for every
file so that a first call shows that it is alive.
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
from typing import List, Optional

PKG_DIR = os.path.dirname(os.path.realpath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "liblqkernels.so"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


class BuildError(RuntimeError):
    pass


def _sources() -> List[str]:
    return sorted(os.path.join(SRC_DIR, f) for f in os.listdir(SRC_DIR) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(os.path.join(SRC_DIR, f) for f in os.listdir(SRC_DIR) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for path in _sources() + _headers():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dirs() -> List[str]:
    """Where a built library may lie, in order of preference."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [
        os.path.join(PKG_DIR, "_lib"),
        os.path.join(tempfile.gettempdir(), f"lqkernels-{uid}"),
    ]


def find_built() -> Optional[str]:
    want = source_hash()
    for d in lib_dirs():
        lib = os.path.join(d, LIB_NAME)
        stamp = os.path.join(d, LIB_NAME + ".hash")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
    return None


def _log(msg: str) -> None:
    print(f"[longbow-quarrel_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = False, jobs: Optional[int] = None) -> str:
    if not force:
        got = find_built()
        if got:
            return got
    hipcc = _hipcc()
    out_dir = next((d for d in lib_dirs() if _writable_dir(d)), None)
    if out_dir is None:
        raise BuildError(f"no writable place for the kernel library among {lib_dirs()}")
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    env = dict(os.environ)
    # an empty or unwritable HOME must not stop the compiler's own caches
    env.setdefault("TMPDIR", tempfile.gettempdir())
    srcs = _sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16)
    t0 = time.time()
    _log(f"compiling {len(srcs)} files for {ARCH} with {hipcc} into {out_dir}")

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *FLAGS, "-c", src, "-o", obj]
        t = time.time()
        proc = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if proc.returncode != 0:
            raise BuildError(f"hipcc failed on {src}:\n{proc.stderr[-4000:]}")
        _log(f"  {os.path.basename(src)} done in {time.time() - t:.1f}s")
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib_tmp = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", lib_tmp]
    proc = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        raise BuildError(f"link failed:\n{proc.stderr[-4000:]}")
    lib = os.path.join(out_dir, LIB_NAME)
    os.replace(lib_tmp, lib)
    with open(os.path.join(out_dir, LIB_NAME + ".hash"), "w") as f:
        f.write(source_hash())
    _log(f"built {lib} in {time.time() - t0:.1f}s")
    return lib


def ensure_built() -> str:
    return build(force=False)


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
