"""Builds the gfx950 kernel library from ``rustinfer_amd/csrc`` with hipcc and loads it.

The library is built in-tree (``rustinfer_amd/_lib/librustinfer_hip.so``) the first time it
is needed, or when a source is newer than it; objects are compiled in parallel and a line
is printed for each file, so a first call on a fresh checkout shows that it is alive.
If the tree is not writable the build goes to a folder under the system temp directory.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "librustinfer_hip.so"
ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-result", "-Wno-unknown-warning-option"]

# Per-file additions.  The prefill attention kernel rescales its accumulators on the vector unit
# now and then; with the accumulators in AGPRs every step would copy them there and back, so its
# MFMAs are compiled in the form that writes VGPRs.
# the vendor's GEMM library, for bfloat16 products of many rows (csrc/gemm_library.cpp)
LINK_LIBS = ["-lhipblaslt"]

EXTRA_FLAGS = {
    # matrix-instruction results in ordinary registers (no moves to and from the accumulation
    # file); no IEEE mode and no NaNs, so that fmaxf is a bare v_max3_f32 (the kernel's scores are
    # finite or -inf by construction)
    "attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form", "-fno-honor-nans", "-mno-amdgpu-ieee"],
}

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH); "
                           "the HIP kernels cannot be built and there is no other path")


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC)
                  if f.endswith(".hip") or f.endswith(".cpp"))


def _headers() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def _lib_dirs() -> List[str]:
    dirs = [os.path.join(PKG_DIR, "_lib")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"rustinfer_amd_lib_{uid}"))
    return dirs


def lib_path() -> Optional[str]:
    """Path of an up-to-date built library, or None."""
    newest = max(os.path.getmtime(p) for p in sources() + _headers())
    for d in _lib_dirs():
        p = os.path.join(d, LIB_NAME)
        if os.path.isfile(p) and os.path.getmtime(p) >= newest:
            return p
    return None


def _say(msg: str) -> None:
    print(f"[rustinfer_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = False, verbose: bool = True) -> str:
    """Compile every source for gfx950 and link the library; returns its path."""
    if not force:
        p = lib_path()
        if p:
            return p
    hipcc = _hipcc()
    out_dir = None
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".w{os.getpid()}")
            open(probe, "w").close()
            os.remove(probe)
            out_dir = d
            break
        except OSError:
            continue
    if out_dir is None:
        raise KernelBuildError("no writable folder for the kernel library")
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    env.setdefault("HOME", tempfile.gettempdir())
    t0 = time.time()
    if verbose:
        _say(f"compiling {len(srcs)} files for {ARCH} with {hipcc} into {out_dir}")

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        cmd = [hipcc] + HIPCC_FLAGS + EXTRA_FLAGS.get(os.path.basename(src), []) \
            + ["-x", "hip", "-c", src, "-o", obj, "-I", CSRC]
        t = time.time()
        r = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise KernelBuildError(f"hipcc failed on {src}:\n{r.stdout}")
        if verbose:
            _say(f"  {os.path.basename(src)} done in {time.time() - t:.1f}s")
        return obj

    jobs = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
    with ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp] + objs + LINK_LIBS
    r = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise KernelBuildError(f"link failed:\n{r.stdout}")
    final = os.path.join(out_dir, LIB_NAME)
    os.replace(tmp, final)
    if verbose:
        _say(f"built {final} in {time.time() - t0:.1f}s")
    return final


def load() -> ctypes.CDLL:
    """The kernel library, built first if it is not there.  There is no fallback: without it
    nothing in the engine runs."""
    global _lib
    with _lock:
        if _lib is None:
            path = lib_path() or build()
            try:
                _lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelBuildError(f"cannot load {path}: {e}") from None
            _lib.ri_last_error.restype = ctypes.c_char_p
        return _lib
