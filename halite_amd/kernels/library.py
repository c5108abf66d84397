"""Builds the HIP sources under ``halite_amd/csrc`` for gfx950 and loads them.

A library is one shared object made with ``hipcc`` from a list of sources and a set
of ``-D`` definitions.  Its file name carries a hash of the sources' text and the
flags, so a stale build is never loaded: if the named file is missing it is compiled
at the first call (objects in parallel, a progress line now and then) and stored
beside the sources, or in the temporary folder if that place cannot be written.
Nothing here needs a home directory or the network.
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

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wno-unused-value",
    # no packed float32 instructions from the code generator
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]

CORE_SOURCES = [
    "runtime.hip",
    "elementwise.hip",
    "attention_simple.hip",
    "gemm_f32.hip",
    "gemm_bf16.hip",
    "sampling.hip",
]
ATTENTION_SOURCES = ["runtime.hip", "attention_mfma.hip"]

_loaded: dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelLibraryError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelLibraryError(
        "hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels "
        "cannot be built and there is no other implementation to fall back to"
    )


def _headers() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))


def _digest(sources: list[str], defines: dict[str, int]) -> str:
    h = hashlib.sha256()
    for name in list(sources) + _headers():
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(repr(sorted(defines.items())).encode())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _build_dirs() -> list[str]:
    dirs = [os.path.join(CSRC, "_build")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"halite_amd_build_{uid}"))
    return dirs


def library_path(name: str, sources: list[str], defines: dict[str, int]) -> tuple[str, str]:
    """(file name, path of an existing build or '')."""
    fname = f"libhalite_{name}_{_digest(sources, defines)}.so"
    for d in _build_dirs():
        p = os.path.join(d, fname)
        if os.path.isfile(p):
            return fname, p
    return fname, ""


def _say(msg: str):
    print(f"[halite_amd] {msg}", file=sys.stderr, flush=True)


def build_library(name: str, sources: list[str], defines: dict[str, int], force=False) -> str:
    """Compile (if needed) and return the path of the shared object."""
    fname, existing = library_path(name, sources, defines)
    if existing and not force:
        return existing
    hipcc = _hipcc()
    out_dir = None
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            fd, probe = tempfile.mkstemp(prefix=".w", dir=d)  # a name of its own: builds run side by side
            os.close(fd)
            os.remove(probe)
            out_dir = d
            break
        except OSError:
            continue
    if out_dir is None:
        raise KernelLibraryError(f"no writable place for the build among {_build_dirs()}")

    work = tempfile.mkdtemp(prefix=f"{name}_", dir=out_dir)
    dflags = [f"-D{k}={v}" for k, v in sorted(defines.items())]
    _say(f"compiling {name} for {ARCH}: {len(sources)} sources {' '.join(dflags)}")
    t0 = time.time()

    def compile_one(src: str) -> str:
        obj = os.path.join(work, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *dflags, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src}:\n{_filter(r.stderr)}")
        return obj

    try:
        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            futures = [pool.submit(compile_one, s) for s in sources]
            while True:
                pending = [f for f in futures if not f.done()]
                if not pending:
                    break
                time.sleep(0.2)
                if time.time() - t0 > 10 and int(time.time() - t0) % 10 == 0:
                    _say(f"  ... still compiling {name} ({int(time.time() - t0)} s)")
                    time.sleep(1.0)
            objs = [f.result() for f in futures]
        tmp_so = os.path.join(work, fname)
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp_so]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed to link {name}:\n{_filter(r.stderr)}")
        final = os.path.join(out_dir, fname)
        os.replace(tmp_so, final)
    finally:
        shutil.rmtree(work, ignore_errors=True)
    _say(f"built {fname} in {time.time() - t0:.1f} s")
    return final


def _filter(stderr: str) -> str:
    return "\n".join(
        line for line in stderr.splitlines() if "is not a recognized feature" not in line
    )


def _check_device() -> None:
    """The kernels use instructions and LDS sizes of gfx950 alone; another GPU is refused
    here rather than met by a code object that does not load."""
    import torch

    if torch.cuda.is_available():
        name = torch.cuda.get_device_properties(torch.cuda.current_device()).gcnArchName
        if not name.startswith(ARCH):
            raise KernelLibraryError(f"the HIP kernels are written for {ARCH} (MI355X); this GPU is {name}")


def load_library(name: str, sources: list[str], defines: dict[str, int] | None = None) -> ctypes.CDLL:
    defines = defines or {}
    key = name + repr(sorted(defines.items()))
    with _lock:
        if key in _loaded:
            return _loaded[key]
        _check_device()
        path = build_library(name, sources, defines)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from e
        lib.hal_last_error.restype = ctypes.c_char_p
        _loaded[key] = lib
        return lib


def core_library() -> ctypes.CDLL:
    return load_library("core", CORE_SOURCES)


def attention_library(head_dim: int) -> ctypes.CDLL:
    return load_library(f"attn_d{head_dim}", ATTENTION_SOURCES, {"HAL_HEAD_DIM": head_dim})


def build_all(head_dims=(16, 32, 64, 128), force=True, prune=True) -> list[str]:
    """Compile every library for the given head sizes (the build check); with
    ``prune`` builds of older sources are removed from the in-tree build folder."""
    jobs = [("core", CORE_SOURCES, {})]
    jobs += [(f"attn_d{d}", ATTENTION_SOURCES, {"HAL_HEAD_DIM": d}) for d in head_dims]
    with ThreadPoolExecutor(max_workers=4) as pool:  # each job compiles its sources in parallel too
        paths = list(pool.map(lambda j: build_library(*j, force=force), jobs))
    if prune:
        folder = _build_dirs()[0]
        keep = {os.path.basename(p) for p in paths}
        for name in os.listdir(folder) if os.path.isdir(folder) else []:
            if name.startswith("libhalite_") and name.endswith(".so") and name not in keep:
                os.remove(os.path.join(folder, name))
    return paths
