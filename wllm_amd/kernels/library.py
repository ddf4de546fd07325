"""Building and loading the kernel library.

The kernels under `wllm_amd/csrc` are compiled with hipcc for gfx950 into one
shared library, `wllm_amd/libwllm_kernels.so`, whose `extern "C"` entry points
are called through ctypes with raw device pointers and a stream.  Nothing of
torch is compiled against, so a build takes about a minute from nothing.

`load()` loads the library if it is built from the present sources and builds it
first if not (a line is printed per compiled file, so that a first call in a
fresh checkout shows what it is doing).  If the package folder cannot be
written to, the build goes to a folder under the system's temporary directory.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE_DIR = os.path.join(PACKAGE_DIR, "csrc")
LIBRARY_NAME = "libwllm_kernels.so"
ARCH = "gfx950"
# packed float32 instructions are switched off for all device code
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-fvisibility=hidden", "-Wno-unused-command-line-argument"]


class KernelLibraryMissing(RuntimeError):
    """The kernel library is not built and cannot be built here."""


def sources(source_dir: str = SOURCE_DIR) -> list:
    return sorted(f for f in os.listdir(source_dir) if f.endswith(".hip"))


def _fingerprint(source_dir: str = SOURCE_DIR) -> str:
    """Of the flags and of every source and header of the folder (and, for a folder of kernels that
    is not the framework's own, of the framework's headers it may include)."""
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    folders = [source_dir] if os.path.samefile(source_dir, SOURCE_DIR) else [source_dir, SOURCE_DIR]
    for folder in folders:
        for name in sorted(os.listdir(folder)):
            if name.endswith(".h") or (folder == source_dir and name.endswith(".hip")):
                h.update(name.encode())
                with open(os.path.join(folder, name), "rb") as f:
                    h.update(f.read())
    return h.hexdigest()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise KernelLibraryMissing("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                               "the kernel library cannot be built")


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _locations(fingerprint: str, source_dir: str = SOURCE_DIR, library_name: str = LIBRARY_NAME) -> list:
    """(library path, object folder) candidates, beside the sources first (the framework's own
    library lies in the package folder, one level above its sources)."""
    fallback = os.path.join(tempfile.gettempdir(), f"wllm_amd_build_{os.getuid()}_{fingerprint[:16]}")
    beside = PACKAGE_DIR if os.path.samefile(source_dir, SOURCE_DIR) else source_dir
    return [(os.path.join(beside, library_name), os.path.join(source_dir, "_build")),
            (os.path.join(fallback, library_name), os.path.join(fallback, "obj"))]


def _is_current(lib_path: str, fingerprint: str) -> bool:
    stamp = lib_path + ".stamp"
    if not (os.path.isfile(lib_path) and os.path.isfile(stamp)):
        return False
    with open(stamp, "r", encoding="utf-8") as f:
        return f.read().strip() == fingerprint


def build(verbose: bool = True, force: bool = True, source_dir: str = SOURCE_DIR, library_name: str = LIBRARY_NAME) -> str:
    """Compiles every source of the folder for gfx950 and links the library; returns its path.
    The framework's headers are on the include path of any folder."""
    fingerprint = _fingerprint(source_dir)
    hipcc = _hipcc()
    lib_path = obj_dir = None
    for cand_lib, cand_obj in _locations(fingerprint, source_dir, library_name):
        if _writable(os.path.dirname(cand_lib)) and _writable(cand_obj):
            lib_path, obj_dir = cand_lib, cand_obj
            break
    if lib_path is None:
        raise KernelLibraryMissing("no writable place for the kernel library (beside its sources and the temporary folder)")
    if not force and _is_current(lib_path, fingerprint):
        return lib_path
    names = sources(source_dir)
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    t0 = time.time()

    def say(msg: str) -> None:
        if verbose:
            print(f"[wllm_amd build] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(names)} kernel files of {source_dir} for {ARCH} with {hipcc}")

    def compile_one(name: str):
        obj = os.path.join(obj_dir, name[:-4] + ".o")
        cmd = [hipcc] + FLAGS + ["-I", source_dir, "-I", SOURCE_DIR, "-c", os.path.join(source_dir, name), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        return name, obj, r

    objects = []
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(names)))) as pool:
        for name, obj, r in pool.map(compile_one, names):
            if r.returncode != 0:
                raise KernelLibraryMissing(f"hipcc failed on {name}:\n{r.stderr[-4000:]}")
            say(f"compiled {name} ({time.time() - t0:.0f} s)")
            objects.append(obj)
    tmp = lib_path + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp] + objects,
                       capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise KernelLibraryMissing(f"linking the kernel library failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib_path)
    with open(lib_path + ".stamp", "w", encoding="utf-8") as f:
        f.write(fingerprint)
    say(f"built {lib_path} in {time.time() - t0:.0f} s")
    return lib_path


_loaded: dict = {}


def load(verbose: bool = True, source_dir: str = SOURCE_DIR, library_name: str = LIBRARY_NAME) -> ctypes.CDLL:
    """The loaded library of a folder of kernels (the framework's own by default); built first when
    no build of the present sources exists.  A part that brings kernels of its own keeps them in a
    folder of `.hip` files and loads them with `load(source_dir=..., library_name=...)`: the same
    compiler flags, the framework's headers on the include path, the library beside the sources."""
    key = (os.path.realpath(source_dir), library_name)
    if key in _loaded:
        return _loaded[key]
    fingerprint = _fingerprint(source_dir)
    path = None
    for cand_lib, _ in _locations(fingerprint, source_dir, library_name):
        if _is_current(cand_lib, fingerprint):
            path = cand_lib
            break
    if path is None:
        path = build(verbose=verbose, source_dir=source_dir, library_name=library_name)
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryMissing(f"{path} cannot be loaded: {e}") from e
    lib.wllm_path = path
    _loaded[key] = lib
    return lib
