"""Compiles the HIP sources under csrc/ for gfx950 into one shared library.

The library is built in-tree (csrc/_build/) when the tree is writable, else in
a per-user temporary folder. `ensure_built()` loads nothing and compiles only
when no library matches the current sources (a hash of the sources and flags
is kept beside it); `build(force=True)` always compiles.
"""
from __future__ import annotations

import concurrent.futures
import fcntl
import glob
import hashlib
import os
import subprocess
import sys
import tempfile
import time
from typing import List, Optional

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_NAME = "libninfer_hip.so"
ENGINE_LIB_NAME = "libninfer_engine.so"   # the engine's C interface (csrc/engine_api)
ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
         # packed 32-bit float instructions are kept out of all device code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    return "hipcc"


def sources() -> List[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def engine_api_sources() -> List[str]:
    return sorted(glob.glob(os.path.join(CSRC, "engine_api", "*.cpp")))


def _fingerprint() -> str:
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for path in sources() + sorted(glob.glob(os.path.join(CSRC, "*.h"))) + engine_api_sources() \
            + sorted(glob.glob(os.path.join(CSRC, "engine_api", "*.h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _build_dirs() -> List[str]:
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(CSRC, "_build"),
            os.path.join(tempfile.gettempdir(), f"ninfer_hip_build_{uid}")]


def _trusted(d: str) -> bool:
    """The in-tree folder is trusted as the sources beside it are. The fallback folder lies
    in a place anyone can write to: it counts only if it is this user's own and nobody else
    can write into it, so that no other user's library is ever loaded."""
    if d == os.path.join(CSRC, "_build"):
        return True
    try:
        st = os.lstat(d)
    except OSError:
        return False
    import stat
    return (stat.S_ISDIR(st.st_mode) and st.st_uid == os.getuid()
            and not st.st_mode & (stat.S_IWGRP | stat.S_IWOTH))


def _matching_library() -> Optional[str]:
    want = _fingerprint()
    for d in _build_dirs():
        if not _trusted(d):
            continue
        lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, "fingerprint")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
    return None


def _say(msg: str) -> None:
    print(f"[ninfer build] {msg}", file=sys.stderr, flush=True)


def _run(cmd: List[str]) -> None:
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in p.stdout.splitlines() if noise not in l)
    if p.returncode != 0:
        raise RuntimeError(f"command failed ({p.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        _say(out)


def build(force: bool = True, jobs: int = 8) -> str:
    """Compile every source and link the library; returns its path."""
    if not force:
        lib = _matching_library()
        if lib:
            return lib
    out_dir = None
    for d in _build_dirs():
        try:
            os.makedirs(d, mode=0o700, exist_ok=True)
            if not _trusted(d):
                continue
            with open(os.path.join(d, ".probe"), "w"):
                pass
            os.remove(os.path.join(d, ".probe"))
            out_dir = d
            break
        except OSError:
            continue
    if out_dir is None:
        raise RuntimeError("no writable folder to build the HIP library in")
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    # one build at a time per folder: a second process waits, then finds the library made
    with open(os.path.join(out_dir, ".lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if not force:
            lib = _matching_library()
            if lib:
                return lib
        return _compile_and_link(srcs, out_dir, jobs)


def _compile_and_link(srcs: List[str], out_dir: str, jobs: int) -> str:
    hipcc = _hipcc()
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    t0 = time.time()
    objs = [os.path.join(out_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        _run([hipcc, *FLAGS, "-I", CSRC, "-c", src, "-o", obj])
        _say(f"  {os.path.basename(src)} done ({time.time() - t0:.0f} s)")

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(one, zip(srcs, objs)))
    lib = os.path.join(out_dir, LIB_NAME)
    # -z defs: a kernel whose host-side stub the compiler dropped (it does so without a word
    # for some constructs it cannot instantiate on the host) fails here, not at the first load
    _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-Wl,-z,defs", "-o", lib + ".tmp",
          *objs])
    os.replace(lib + ".tmp", lib)
    try:
        _link_engine_api(out_dir)
    except (RuntimeError, OSError) as e:
        # the engine runs without it (it serves host programs in C): say so and go on
        _say(f"the engine's C interface was not built: {e}")
        for stale in (ENGINE_LIB_NAME, ENGINE_LIB_NAME + ".tmp"):
            if os.path.exists(os.path.join(out_dir, stale)):
                os.remove(os.path.join(out_dir, stale))
    with open(os.path.join(out_dir, "fingerprint"), "w") as f:
        f.write(_fingerprint())
    _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def _link_engine_api(out_dir: str) -> None:
    """The engine's C interface: host code only, over the interpreter this build runs in (its
    headers and library); the folder of the package's parent goes in as the place to import
    the engine from."""
    import sysconfig
    cfg = sysconfig.get_config_var
    lib = os.path.join(out_dir, ENGINE_LIB_NAME)
    root = os.path.dirname(os.path.dirname(CSRC))
    libdir, version = cfg("LIBDIR"), cfg("LDVERSION") or cfg("VERSION")
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
          "-I", sysconfig.get_paths()["include"], f'-DNINFER_AMD_ROOT="{root}"',
          *engine_api_sources(), "-o", lib + ".tmp", f"-L{libdir}", f"-Wl,-rpath,{libdir}",
          f"-lpython{version}", "-ldl"])
    os.replace(lib + ".tmp", lib)
    _say(f"built {lib}")


def engine_library() -> str:
    """Path of the engine's C interface beside a kernel library that matches the sources."""
    path = os.path.join(os.path.dirname(ensure_built()), ENGINE_LIB_NAME)
    if not os.path.isfile(path):
        raise RuntimeError(f"{path} is missing: the host compiler or the interpreter's headers "
                           "were not there when the kernel library was built")
    return path


def ensure_built() -> str:
    """Path of a library that matches the sources; compiles if there is none."""
    return build(force=False)
