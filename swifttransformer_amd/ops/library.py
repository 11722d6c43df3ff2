"""Building and loading the HIP kernel library.

The kernels are plain HIP sources under ``csrc/`` compiled by ``hipcc`` for
gfx950 into one shared library that is loaded with ``ctypes`` (C entry points,
raw device pointers).  ``load()`` uses a built library whose recorded source
hash matches the sources; otherwise it compiles, printing a line per file.
There is no fallback: without the library nothing in the engine runs.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")
LIB_NAME = "libst_kernels.so"
ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    # the first kernel arguments arrive in scalar registers with the dispatch instead of by a
    # load from memory that every address computation would wait for
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]
# per-file additions: the prompt attention kernels keep their matrix-core accumulators in ordinary
# vector registers, where the softmax rescales them without moves to and from the
# accumulation registers
FILE_FLAGS = {"attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
              "attention_prefill_dma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
              "attention_prefill_f32.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}
# the vendor's matrix-product library backs the large bfloat16 products (csrc/gemm_library.hip)
LINK_LIBS = ["-lhipblaslt"]

_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None


class KernelLibraryError(RuntimeError):
    pass


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for p in sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC)
                    if f.endswith((".hip", ".h"))):
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS + LINK_LIBS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()[:16]


def _candidate_dirs() -> List[str]:
    """Places for the built library, in order: in-tree, a cache directory."""
    dirs = [os.path.join(_PKG, "_lib")]
    env = os.environ.get("ST_AMD_BUILD_DIR")
    if env:
        dirs.insert(0, env)
    cache = os.environ.get("XDG_CACHE_HOME") or (
        os.path.join(os.environ["HOME"], ".cache") if os.environ.get("HOME") else None)
    if cache:
        dirs.append(os.path.join(cache, "swifttransformer_amd"))
    dirs.append(os.path.join(tempfile.gettempdir(), f"swifttransformer_amd_{os.getuid()}"))
    return dirs


def _is_current(d: str, want: str) -> bool:
    lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, "source.hash")
    if not (os.path.isfile(lib) and os.path.isfile(stamp)):
        return False
    with open(stamp, "r") as f:
        return f.read().strip() == want


def find_built() -> Optional[str]:
    want = source_hash()
    for d in _candidate_dirs():
        if _is_current(d, want):
            return os.path.join(d, LIB_NAME)
    return None


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.isfile(c):
            return c
    raise KernelLibraryError(
        "the HIP kernel library is not built and hipcc was not found; "
        "run `python __graft_entry__.py` (or swifttransformer_amd.ops.library.build()) "
        "on a machine with ROCm")


def _writable_dir() -> str:
    for d in _candidate_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe{os.getpid()}")
            with open(probe, "w") as f:
                f.write("x")
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelLibraryError("no writable directory for the kernel library")


def build(verbose: bool = True, out_dir: Optional[str] = None) -> str:
    """Compile every source for gfx950 and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = out_dir or _writable_dir()
    os.makedirs(out_dir, exist_ok=True)
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    t0 = time.time()

    def say(msg: str) -> None:
        if verbose:
            print(f"[swifttransformer_amd] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *FILE_FLAGS.get(os.path.basename(src), []), "-I", CSRC, "-c", src, "-o", obj]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src}:\n{r.stdout}")
        say(f"  compiled {os.path.basename(src)} ({time.time() - t0:.0f} s)")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), os.cpu_count() or 1))
    with ThreadPoolExecutor(workers) as ex:
        objs = list(ex.map(compile_one, srcs))
    tmp_lib = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, *LINK_LIBS, "-o", tmp_lib]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise KernelLibraryError(f"linking the kernel library failed:\n{r.stdout}")
    os.replace(tmp_lib, os.path.join(out_dir, LIB_NAME))
    with open(os.path.join(out_dir, "source.hash"), "w") as f:
        f.write(source_hash() + "\n")
    shutil.rmtree(obj_dir, ignore_errors=True)
    say(f"built {LIB_NAME} in {time.time() - t0:.0f} s")
    return os.path.join(out_dir, LIB_NAME)


def load() -> ctypes.CDLL:
    """The loaded kernel library (built first if no current build is found)."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = find_built()
        if path is None:
            path = build()
        try:
            _lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from e
        _lib._st_path = path
        return _lib


def loaded_path() -> Optional[str]:
    return getattr(_lib, "_st_path", None) if _lib is not None else None
