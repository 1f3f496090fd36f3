"""Building and loading the HIP kernel libraries.

Each source ``csrc/<name>.hip`` becomes ``csrc/_build/libptl_<name>.so`` (gfx950
only) and is loaded with ctypes; its functions are plain ``extern "C"`` entry
points that take device pointers and a stream. A library is compiled when it is
missing or older than its sources, which is how a fresh checkout builds what a
model needs at its first call. There is no other backend: when a library cannot
be built or loaded the op raises.
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
from typing import Dict, Iterable, List

CSRC_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
BUILD_DIR = os.path.join(CSRC_DIR, "_build")
ARCH = "gfx950"
# packed float32 instructions are switched off for every kernel of this package
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-shared", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

KERNEL_LIBRARIES = ("embedding", "norm", "rope", "attention", "attention_prefill", "activation",
                    "gemm", "gemm_rows", "blaslt", "sampling", "probe")
# options of single sources. attention_prefill: no value there is a NaN unless an input is, and
# without the promise every maximum of scores is preceded by instructions that quiet its inputs
EXTRA_FLAGS = {"attention_prefill": ["-fno-honor-nans"]}
# libraries a source is linked with (after the source on the command line)
LINK_FLAGS = {"blaslt": ["-lhipblaslt"]}

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelLibraryError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelLibraryError("hipcc not found: the HIP kernels of this package cannot be built")


def source_path(name: str) -> str:
    return os.path.join(CSRC_DIR, name + ".hip")


_build_dir_cache = None


def build_dir() -> str:
    """csrc/_build inside the package; when the checkout is read-only for this
    user, a folder of their own under the temporary directory."""
    global _build_dir_cache
    if _build_dir_cache is None:
        d = BUILD_DIR
        try:
            os.makedirs(d, exist_ok=True)
            ok = os.access(d, os.W_OK)
        except OSError:
            ok = False
        if not ok:
            import tempfile
            d = os.path.join(tempfile.gettempdir(), f"pytriton_llama_amd_build_{os.getuid()}")
            os.makedirs(d, exist_ok=True)
        _build_dir_cache = d
    return _build_dir_cache


def library_path(name: str) -> str:
    for d in (BUILD_DIR, build_dir()):
        p = os.path.join(d, f"libptl_{name}.so")
        if os.path.isfile(p):
            return p
    return os.path.join(build_dir(), f"libptl_{name}.so")


def _headers() -> List[str]:
    return [os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".h")]


def is_stale(name: str) -> bool:
    lib = library_path(name)
    if not os.path.isfile(lib):
        return True
    t = os.path.getmtime(lib)
    return any(os.path.getmtime(p) > t for p in [source_path(name)] + _headers())


def compile_command(name: str, out: str) -> List[str]:
    return ([_hipcc()] + HIPCC_FLAGS + EXTRA_FLAGS.get(name, []) +
            ["-I", CSRC_DIR, "-o", out, source_path(name)] + LINK_FLAGS.get(name, []))


def build(names: Iterable[str] = KERNEL_LIBRARIES, force: bool = False, verbose: bool = True) -> None:
    """Compile the named libraries (all of them by default), in parallel
    processes, printing a line when one starts, every few seconds while any is
    still running, and when one is done."""
    todo = [n for n in names if force or is_stale(n)]
    if not todo:
        return
    procs = {}
    t0 = time.time()
    for n in todo:
        if not os.path.isfile(source_path(n)):
            raise KernelLibraryError(f"no kernel source {source_path(n)}")
        final = os.path.join(build_dir(), f"libptl_{n}.so")
        tmp = final + f".tmp{os.getpid()}"
        if verbose:
            print(f"[pytriton_llama_amd] compiling {n}.hip for {ARCH} ...", file=sys.stderr, flush=True)
        # the compiler's messages go to a file, not a pipe: nobody reads a pipe while the
        # compiler runs, and one with many warnings would fill it and wait for ever
        log = tempfile.TemporaryFile(mode="w+", encoding="utf-8", errors="replace")
        procs[n] = (subprocess.Popen(compile_command(n, tmp), stdout=log, stderr=subprocess.STDOUT,
                                     stdin=subprocess.DEVNULL), tmp, final, log)
    last = time.time()
    pending = dict(procs)
    errors = []
    while pending:
        for n, (p, tmp, final, log) in list(pending.items()):
            if p.poll() is None:
                continue
            log.seek(0)
            out = log.read()
            log.close()
            del pending[n]
            if p.returncode != 0:
                errors.append(f"{n}.hip failed to compile:\n{out}")
                if os.path.exists(tmp):
                    os.remove(tmp)
            else:
                os.replace(tmp, final)
                if verbose:
                    print(f"[pytriton_llama_amd] built {n} ({time.time() - t0:.1f}s)",
                          file=sys.stderr, flush=True)
        if pending:
            time.sleep(0.1)
            if verbose and time.time() - last > 5:
                last = time.time()
                print(f"[pytriton_llama_amd] still compiling {sorted(pending)} "
                      f"({last - t0:.0f}s)", file=sys.stderr, flush=True)
    if errors:
        raise KernelLibraryError("\n".join(errors))


def load(name: str) -> ctypes.CDLL:
    """The loaded library ``name``; built first when missing or stale."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        if is_stale(name):
            build([name])
        try:
            lib = ctypes.CDLL(library_path(name))
        except OSError as e:
            raise KernelLibraryError(
                f"cannot load HIP kernel library {library_path(name)}: {e}") from e
        _loaded[name] = lib
        return lib


def require(names: Iterable[str]) -> None:
    """Build (if needed) and load several libraries at once, so that what a
    model needs is compiled side by side rather than one after the other."""
    names = [n for n in dict.fromkeys(names) if n not in _loaded]
    stale = [n for n in names if is_stale(n)]
    if stale:
        with _lock:
            build(stale)
    for n in names:
        load(n)
