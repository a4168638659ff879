"""Building and loading the native libraries.

Two kinds of library exist, each a plain shared object with a C interface that is called through ``ctypes``:

* HIP modules for gfx950, compiled with ``hipcc`` from ``csrc/kernels/*.hip``.  A module is a list of sources
  plus ``-D`` definitions; the attention kernels, for example, are compiled once per head size, and only the
  head size a model has is compiled when that model is first used.
* the host library (page tables, free lists), compiled with ``g++`` from ``csrc/host/*.cpp``.

A built library lies next to the sources, in ``csrc/lib/``, with a stamp holding the hash of its sources and flags.
``load`` uses it when the stamp matches, compiles otherwise (printing a line per file, so a long first call shows
life), and raises ``KernelBuildError`` when it can do neither: there is no fallback to other code.  If the
source tree is not writable, libraries go to a per-user folder under the temporary directory.
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
from typing import Dict, List, Optional, Sequence, Tuple

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
_KERNELS = os.path.join(_CSRC, "kernels")
_HOST = os.path.join(_CSRC, "host")

GPU_ARCH = "gfx950"
# (kernarg preload: the first 14 words of a kernel's arguments are in scalar registers when a wave starts, where the
# others are fetched from memory; the kernels order their arguments for it)
HIP_FLAGS = ["--offload-arch=" + GPU_ARCH, "-O3", "-std=c++17", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
             "-mllvm", "-amdgpu-kernarg-preload-count=14"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall"]


class KernelBuildError(RuntimeError):
    pass


# name -> (sources relative to csrc/kernels, fixed definitions)
HIP_MODULES: Dict[str, Tuple[Sequence[str], Sequence[str]]] = {
    "core": (("elementwise.hip", "attention_generic.hip", "gemm_generic.hip", "sampling.hip"), ()),
    "gemm_bf16": (("gemm_bf16.hip",), ()),
    "microbench": (("microbench.hip",), ()),
}

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()
_module_locks: Dict[str, threading.Lock] = {}

# head sizes whose attention module the build check compiles ahead of time: every one the kernel takes (a few
# seconds each); a model compiles only its own when it is first used and no built module is there
STANDARD_HEAD_SIZES = tuple(range(16, 257, 16))
# (head size, tokens a page) beyond pages of 16 tokens that the build check compiles too: the head sizes of the Llamas
# with pages of 32 and 64 tokens, and what the tests run; any other pair is compiled when a cache first has it
LARGER_PAGE_MODULES = tuple((hd, page) for hd in (32, 48, 64, 128) for page in (32, 64)) + ((64, 48), (80, 48))


def _lock_for(name: str) -> threading.Lock:
    with _lock:
        return _module_locks.setdefault(name, threading.Lock())


def _say(msg: str) -> None:
    print(f"[atoma_infer_amd build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _lib_dirs() -> List[str]:
    dirs = [os.path.join(_CSRC, "lib")]
    try:
        uid = os.getuid()
    except AttributeError:  # pragma: no cover
        uid = 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"atoma_infer_amd_lib_{uid}"))
    return dirs


def _writable_lib_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            fd, probe = tempfile.mkstemp(prefix=".probe_", dir=d)
            os.close(fd)
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelBuildError(f"no writable folder for built libraries among {_lib_dirs()}")


def _hash(paths: Sequence[str], flags: Sequence[str]) -> str:
    h = hashlib.sha256()
    h.update("\0".join(flags).encode())
    headers = sorted(os.path.join(os.path.dirname(paths[0]), f) for f in os.listdir(os.path.dirname(paths[0]))
                     if f.endswith(".h"))
    for p in list(paths) + headers:
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _find_built(name: str, digest: str) -> Optional[str]:
    for d in _lib_dirs():
        so, stamp = os.path.join(d, f"libatoma_{name}.so"), os.path.join(d, f"libatoma_{name}.stamp")
        try:
            with open(stamp, "r") as f:
                if f.read().strip() == digest and os.path.isfile(so):
                    return so
        except OSError:
            continue
    return None


def _run(cmd: List[str], what: str) -> None:
    t0 = time.time()
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if r.returncode != 0:
        raise KernelBuildError(f"{what} failed ({' '.join(cmd)}):\n{r.stdout}\n{r.stderr}")
    _say(f"{what}: {time.time() - t0:.1f} s")


def _compile(name: str, compiler: str, sources: Sequence[str], flags: Sequence[str], digest: str,
             link_flags: Sequence[str] = ()) -> str:
    out_dir = _writable_lib_dir()
    work = tempfile.mkdtemp(prefix=f"build_{name}_", dir=out_dir)
    try:
        objs = [os.path.join(work, os.path.splitext(os.path.basename(s))[0] + ".o") for s in sources]
        _say(f"compiling module '{name}' ({len(sources)} file(s)) with {os.path.basename(compiler)}")
        jobs = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
        with ThreadPoolExecutor(jobs) as pool:
            futs = [pool.submit(_run, [compiler, *flags, "-c", s, "-o", o], f"{name}: {os.path.basename(s)}")
                    for s, o in zip(sources, objs)]
            for f in futs:
                f.result()
        so_tmp = os.path.join(work, "lib.so")
        _run([compiler, "-shared", "-fPIC", *[f for f in flags if f.startswith("--offload-arch")], *objs,
              *link_flags, "-o", so_tmp], f"{name}: link")
        so, stamp = os.path.join(out_dir, f"libatoma_{name}.so"), os.path.join(out_dir, f"libatoma_{name}.stamp")
        os.replace(so_tmp, so)
        with open(stamp + ".tmp", "w") as f:
            f.write(digest)
        os.replace(stamp + ".tmp", stamp)
        return so
    finally:
        shutil.rmtree(work, ignore_errors=True)


def _module_plan(name: str, sources: Sequence[str], defines: Sequence[str]):
    paths = [os.path.join(_KERNELS, s) for s in sources]
    flags = HIP_FLAGS + [f"-D{d}" for d in defines]
    # the include path is left out of the hash: it differs between checkouts of the same sources
    return paths, flags + ["-I" + _KERNELS], _hash(paths, flags)


def load_hip_module(name: str, sources: Optional[Sequence[str]] = None, defines: Sequence[str] = (),
                    *, force_build: bool = False) -> ctypes.CDLL:
    """Load HIP module ``name``, compiling it first if no built library matches its sources."""
    with _lock_for(name):
        if name in _loaded and not force_build:
            return _loaded[name]
        if sources is None:
            sources, defines = HIP_MODULES[name]
        paths, flags, digest = _module_plan(name, sources, defines)
        so = None if force_build else _find_built(name, digest)
        if so is None:
            cc = _hipcc()
            if cc is None:
                raise KernelBuildError(f"HIP module '{name}' is not built and hipcc was not found; "
                                       f"this framework has no other code path")
            so = _compile(name, cc, paths, flags, digest)
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise KernelBuildError(f"cannot load {so}: {e}") from None
        _loaded[name] = lib
        return lib


def load_host_library(*, force_build: bool = False) -> ctypes.CDLL:
    """The host library (cache manager); needs no GPU and no ROCm."""
    name = "host"
    with _lock_for(name):
        if name in _loaded and not force_build:
            return _loaded[name]
        paths = sorted(os.path.join(_HOST, f) for f in os.listdir(_HOST) if f.endswith(".cpp"))
        digest = _hash(paths, HOST_FLAGS)
        so = None if force_build else _find_built(name, digest)
        if so is None:
            cc = shutil.which("g++") or shutil.which("c++") or _hipcc()
            if cc is None:
                raise KernelBuildError("the host library is not built and no C++ compiler was found")
            so = _compile(name, cc, paths, HOST_FLAGS, digest)
        lib = ctypes.CDLL(so)
        _loaded[name] = lib
        return lib


def build_all(head_sizes: Sequence[int] = STANDARD_HEAD_SIZES) -> List[str]:
    """Compile every module from scratch (the build check); returns the names built."""
    from . import attention_bf16
    built = []
    load_host_library(force_build=True)
    built.append("host")
    jobs = [(name, None, ()) for name in HIP_MODULES]
    jobs += [(attention_bf16.module_name(hd), ("attention_mfma.hip",), attention_bf16.module_defines(hd))
             for hd in head_sizes]
    jobs += [(attention_bf16.module_name(hd, page), ("attention_mfma.hip",), attention_bf16.module_defines(hd, page))
             for hd, page in LARGER_PAGE_MODULES]
    with ThreadPoolExecutor(min(8, len(jobs))) as pool:
        futs = [pool.submit(load_hip_module, n, src, d, force_build=True) for n, src, d in jobs]
        for (n, _, _), f in zip(jobs, futs):
            f.result()
            built.append(n)
    return built
