"""Builds the HIP kernel library for gfx950 with hipcc.

The library is a plain shared object with a C interface (no PyTorch headers), so a
build takes seconds.  It lives next to the sources, in ``atom_amd/csrc/_build``;
where that folder cannot be written (a read-only checkout) a per-user folder under
the system's temporary directory is used instead.  A library is rebuilt when a
source is newer than it, and on the first use in a fresh checkout.
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

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc")
CSRC = os.path.normpath(CSRC)
LIB_NAME = "libatom_hip.so"
ARCH = "gfx950"
# packed float32 instructions are switched off for every kernel of this library
HIPCC_FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-option-ignored",
]


class BuildError(RuntimeError):
    pass


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                     "the kernels of this engine cannot be built")


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dirs() -> list[str]:
    """Where a built library may live: in-tree first, then a per-user temporary folder."""
    tag = hashlib.sha1(CSRC.encode()).hexdigest()[:10]
    return [os.path.join(CSRC, "_build"),
            os.path.join(tempfile.gettempdir(), f"atom_amd_build_{os.getuid()}_{tag}")]


def _stale(lib: str) -> bool:
    if not os.path.isfile(lib):
        return True
    built = os.path.getmtime(lib)
    return any(os.path.getmtime(p) > built for p in sources() + _headers())


def find_library() -> str | None:
    """The path of an up-to-date built library, or None."""
    for folder in build_dirs():
        lib = os.path.join(folder, LIB_NAME)
        if not _stale(lib):
            return lib
    return None


def _say(msg: str) -> None:
    print(f"[atom_amd build] {msg}", file=sys.stderr, flush=True)


def _compile(hipcc: str, src: str, obj: str) -> None:
    cmd = [hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj, f"-I{CSRC}"]
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    start = time.time()
    while True:
        try:
            out, _ = proc.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            _say(f"still compiling {os.path.basename(src)} ({time.time() - start:.0f} s)")
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {src}:\n{out}")
    # the host pass does not know the device feature flag; that warning is harmless
    noise = "is not a recognized feature for this target"
    for line in out.splitlines():
        if line.strip() and noise not in line and "warning generated" not in line and "warnings generated" not in line:
            _say(line)


def build(force: bool = False) -> str:
    """Compiles every kernel source and links the library; returns its path."""
    if not force:
        lib = find_library()
        if lib:
            return lib
    hipcc = _hipcc()
    folder = next((d for d in build_dirs() if _writable(d)), None)
    if folder is None:
        raise BuildError(f"no writable build folder among {build_dirs()}")
    srcs = sources()
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {folder}")
    objs = [os.path.join(folder, os.path.basename(s)[:-4] + ".o") for s in srcs]
    start = time.time()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        list(pool.map(lambda so: _compile(hipcc, *so), zip(srcs, objs)))
    lib = os.path.join(folder, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise BuildError(f"linking {lib} failed:\n{res.stdout}")
    os.replace(tmp, lib)
    _say(f"built {lib} in {time.time() - start:.0f} s")
    return lib


def build_sources(srcs: list[str], lib_name: str, out_dir: str | None = None) -> str:
    """Compiles HIP sources that are not part of this library (a part that brings kernels of its own) with the
    library's flags and links them into ``lib_name``; returns its path.  The library lands in ``out_dir``
    (default: a ``_build`` folder beside the first source, or a per-user temporary folder where that cannot be
    written) and is rebuilt only when a source is newer.  The sources may include ``common.h`` of this library."""
    srcs = [os.path.abspath(s) for s in srcs]
    tag = hashlib.sha1("|".join(srcs).encode()).hexdigest()[:10]
    candidates = [out_dir] if out_dir else [os.path.join(os.path.dirname(srcs[0]), "_build"),
                                            os.path.join(tempfile.gettempdir(), f"atom_amd_ext_{os.getuid()}_{tag}")]
    for folder in candidates:
        lib = os.path.join(folder, lib_name)
        if os.path.isfile(lib) and all(os.path.getmtime(s) <= os.path.getmtime(lib) for s in srcs):
            return lib
    folder = next((d for d in candidates if _writable(d)), None)
    if folder is None:
        raise BuildError(f"no writable build folder among {candidates}")
    hipcc = _hipcc()
    _say(f"compiling {len(srcs)} HIP source(s) into {os.path.join(folder, lib_name)}")
    objs = [os.path.join(folder, os.path.basename(s).rsplit(".", 1)[0] + ".o") for s in srcs]
    for src, obj in zip(srcs, objs):
        _compile(hipcc, src, obj)
    lib = os.path.join(folder, lib_name)
    tmp = lib + f".tmp{os.getpid()}"
    res = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise BuildError(f"linking {lib} failed:\n{res.stdout}")
    os.replace(tmp, lib)
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
