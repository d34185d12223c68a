"""Compiles the HIP sources of this folder into one shared library for gfx950.

``hipcc`` is driven directly (no torch headers are involved, so a file takes
seconds). The library is written next to the package when that place is
writable, else under a per-user folder of the temporary directory. A stamp
file holds a hash of the sources and flags; ``ensure_built`` compiles when no
library with the current stamp is found.
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
LIB_NAME = "libtransformer_amd_kernels.so"
ARCH = "gfx950"
# packed float32 instructions are switched off for all device code
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-result"]


class BuildError(RuntimeError):
    pass


def sources():
    return sorted(CSRC.glob("*.hip"))


def source_stamp() -> str:
    h = hashlib.sha256()
    for p in sorted(list(CSRC.glob("*.hip")) + [x for x in CSRC.glob("*.h") if not x.name.startswith("ref_")]):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def candidate_dirs():
    """Places a built library may live, in order of preference."""
    dirs = [CSRC.parent / "lib"]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(Path(tempfile.gettempdir()) / f"transformer_amd-{uid}")
    return dirs


def find_built(require_current=False):
    """Path of a built library, or None. Without ``require_current`` any built
    library is taken (a box without the compiler runs what was shipped)."""
    stamp = source_stamp()
    for d in candidate_dirs():
        lib, st = d / LIB_NAME, d / (LIB_NAME + ".stamp")
        if lib.exists():
            current = st.exists() and st.read_text().strip() == stamp
            if current or not require_current:
                return lib
    return None


def _writable_dir():
    for d in candidate_dirs():
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".probe-{os.getpid()}"
            probe.write_text("")
            probe.unlink()
            return d
        except OSError:
            continue
    raise BuildError("no writable place for the kernel library: tried "
                     + ", ".join(str(d) for d in candidate_dirs()))


def build(verbose=True, jobs=None) -> Path:
    """Compile every source and link the library; always compiles."""
    hipcc = _hipcc()
    out_dir = _writable_dir()
    obj_dir = out_dir / "_build"
    obj_dir.mkdir(exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16)
    t0 = time.time()

    def say(msg):
        if verbose:
            print(f"[transformer_amd build] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} HIP files for {ARCH} with {jobs} jobs into {out_dir}")

    def one(src):
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *FLAGS, "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise BuildError(f"hipcc failed on {src.name}:\n{r.stderr[-4000:]}")
        say(f"  {src.name} done ({time.time() - t0:.0f}s)")
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(one, srcs))
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise BuildError(f"linking the kernel library failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, out_dir / LIB_NAME)
    (out_dir / (LIB_NAME + ".stamp")).write_text(source_stamp())
    say(f"built {out_dir / LIB_NAME} in {time.time() - t0:.0f}s")
    return out_dir / LIB_NAME


def ensure_built(verbose=True) -> Path:
    """The library to load: a current one if there is one; else compile when a
    compiler is at hand; else whatever was shipped; else fail loudly."""
    lib = find_built(require_current=True)
    if lib is not None:
        return lib
    try:
        _hipcc()
    except BuildError:
        lib = find_built(require_current=False)
        if lib is not None:
            return lib
        raise BuildError(f"{LIB_NAME} is not built and hipcc is not available; "
                         f"run `python -m transformer_amd.csrc.build` where ROCm is installed")
    return build(verbose=verbose)


# ------------------------------------------------------------------ the plain C++ twins
# *_ref.cpp beside the kernels: host code only, compiled with the host compiler into a library
# of its own that the tests load (nothing on the product path does).
REF_LIB_NAME = "libtransformer_amd_ref.so"
REF_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared"]


def ref_sources():
    return sorted(CSRC.glob("*_ref.cpp"))


def ref_stamp() -> str:
    h = hashlib.sha256()
    for p in ref_sources() + [CSRC / "ref_common.h"]:
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(REF_FLAGS).encode())
    return h.hexdigest()[:16]


def _host_compiler() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/llvm/bin/clang++"):
        if cand and (Path(cand).exists() or shutil.which(cand)):
            return cand
    raise BuildError("no C++ compiler found for the plain twins (looked at $CXX, g++, c++, clang++)")


def build_ref(verbose=True) -> Path:
    """Compile the plain twins into their library; always compiles."""
    out_dir = _writable_dir()
    tmp = out_dir / (REF_LIB_NAME + f".tmp{os.getpid()}")
    cmd = [_host_compiler(), *REF_FLAGS, *map(str, ref_sources()), "-o", str(tmp)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise BuildError(f"compiling the plain twins failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, out_dir / REF_LIB_NAME)
    (out_dir / (REF_LIB_NAME + ".stamp")).write_text(ref_stamp())
    if verbose:
        print(f"[transformer_amd build] built {out_dir / REF_LIB_NAME}", file=sys.stderr, flush=True)
    return out_dir / REF_LIB_NAME


def ensure_ref_built(verbose=False) -> Path:
    stamp = ref_stamp()
    for d in candidate_dirs():
        lib, st = d / REF_LIB_NAME, d / (REF_LIB_NAME + ".stamp")
        if lib.exists() and st.exists() and st.read_text().strip() == stamp:
            return lib
    return build_ref(verbose=verbose)


if __name__ == "__main__":
    print(build())
    print(build_ref())
