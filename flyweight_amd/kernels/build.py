"""Builds the gfx950 kernel library from ``csrc/*.hip`` with hipcc, and the host library
(cache bookkeeping and scheduler, ``csrc/host/*.cpp``) with the host compiler.

The library is built in-tree (``csrc/_build/libflyweight_hip.so``) so that it travels
with the source tree; when the tree is not writable it is built under the temporary
folder instead. ``ensure_built()`` builds only when no current library is found, and
prints a line per file meanwhile, since a first build takes a minute or two.
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

CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))
LIB_NAME = "libflyweight_hip.so"
ARCH = "gfx950"
# packed float32 instructions are switched off: the compiler otherwise forms them from
# ordinary float code
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _say(text: str) -> None:
    print(f"[flyweight_amd] {text}", file=sys.stderr, flush=True)


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _fingerprint() -> str:
    digest = hashlib.sha256()
    for path in sources() + sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")):
        digest.update(os.path.basename(path).encode())
        with open(path, "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(FLAGS).encode())
    return digest.hexdigest()


def _hipcc() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    for candidate in ("/opt/rocm/bin/hipcc",):
        if os.path.isfile(candidate):
            return candidate
    raise RuntimeError("hipcc not found: the gfx950 kernels cannot be built")


def build_dirs() -> List[str]:
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(CSRC, "_build"),
            os.path.join(tempfile.gettempdir(), f"flyweight_amd_build_{uid}")]


def find_library(require_current: bool = True) -> Optional[str]:
    wanted = _fingerprint() if require_current else None
    for folder in build_dirs():
        lib = os.path.join(folder, LIB_NAME)
        stamp = os.path.join(folder, "build.stamp")
        if not os.path.isfile(lib):
            continue
        if wanted is None:
            return lib
        if os.path.isfile(stamp):
            with open(stamp, "r", encoding="utf-8") as handle:
                if handle.read().strip() == wanted:
                    return lib
    return None


def _writable_dir() -> str:
    for folder in build_dirs():
        try:
            os.makedirs(folder, exist_ok=True)
            probe = os.path.join(folder, f".probe_{os.getpid()}")
            with open(probe, "w") as handle:
                handle.write("x")
            os.remove(probe)
            return folder
        except OSError:
            continue
    raise RuntimeError("no writable folder to build the kernel library in")


def build(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    folder = _writable_dir()
    files = sources()
    started = time.time()
    if verbose:
        _say(f"building {LIB_NAME} for {ARCH} from {len(files)} sources in {folder}")
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())

    def compile_one(path: str) -> str:
        obj = os.path.join(folder, os.path.basename(path)[:-4] + ".o")
        begun = time.time()
        result = subprocess.run([hipcc, *FLAGS, "-c", path, "-o", obj], capture_output=True, text=True, env=env)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed on {path}:\n{result.stderr}")
        if verbose:
            _say(f"  compiled {os.path.basename(path)} in {time.time() - begun:.0f} s")
        return obj

    workers = max(1, min(8, len(files), (os.cpu_count() or 2)))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objects = list(pool.map(compile_one, files))
    lib = os.path.join(folder, LIB_NAME)
    partial = lib + f".{os.getpid()}.tmp"
    result = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", partial, *objects],
                            capture_output=True, text=True, env=env)
    if result.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{result.stderr}")
    os.replace(partial, lib)
    with open(os.path.join(folder, "build.stamp"), "w", encoding="utf-8") as handle:
        handle.write(_fingerprint())
    if verbose:
        _say(f"built {lib} in {time.time() - started:.0f} s")
    return lib


def ensure_built() -> str:
    lib = find_library(require_current=True)
    if lib is not None:
        return lib
    try:
        return build()
    except RuntimeError:
        stale = find_library(require_current=False)
        if stale is not None:
            _say(f"warning: could not rebuild; loading {stale}, which is older than the sources")
            return stale
        raise


# ----- the host library: no GPU code, built with the host compiler alone -------------------------
HOST_DIR = os.path.join(CSRC, "host")
HOST_LIB_NAME = "libflyweight_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]
HOST_SELFTEST = "selftest.cpp"      # a program of its own (see build_host_selftest), not part of the library
# address and undefined-behaviour sanitizers, their runtimes linked into the program itself
SANITIZE_FLAGS = ["-O1", "-g", "-std=c++17", "-Wall", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
                  "-fno-sanitize-recover=undefined", "-static-libasan", "-static-libubsan"]


def _host_fingerprint() -> str:
    digest = hashlib.sha256()
    for name in sorted(os.listdir(HOST_DIR)):
        if name.endswith((".cpp", ".hpp", ".h")):
            digest.update(name.encode())
            with open(os.path.join(HOST_DIR, name), "rb") as handle:
                digest.update(handle.read())
    digest.update(" ".join(HOST_FLAGS).encode())
    return digest.hexdigest()


def _host_compiler() -> str:
    for name in ("g++", "c++", "clang++"):
        found = shutil.which(name)
        if found:
            return found
    return _hipcc()


def find_host_library(require_current: bool = True) -> Optional[str]:
    wanted = _host_fingerprint() if require_current else None
    for folder in build_dirs():
        lib = os.path.join(folder, HOST_LIB_NAME)
        stamp = os.path.join(folder, "host.stamp")
        if not os.path.isfile(lib):
            continue
        if wanted is None:
            return lib
        if os.path.isfile(stamp):
            with open(stamp, "r", encoding="utf-8") as handle:
                if handle.read().strip() == wanted:
                    return lib
    return None


def build_host(verbose: bool = True) -> str:
    folder = _writable_dir()
    started = time.time()
    units = sorted(os.path.join(HOST_DIR, f) for f in os.listdir(HOST_DIR) if f.endswith(".cpp") and f != HOST_SELFTEST)
    lib = os.path.join(folder, HOST_LIB_NAME)
    partial = lib + f".{os.getpid()}.tmp"
    result = subprocess.run([_host_compiler(), *HOST_FLAGS, "-o", partial, *units], capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"building {HOST_LIB_NAME} failed:\n{result.stderr}")
    os.replace(partial, lib)
    with open(os.path.join(folder, "host.stamp"), "w", encoding="utf-8") as handle:
        handle.write(_host_fingerprint())
    if verbose:
        _say(f"built {lib} in {time.time() - started:.0f} s")
    return lib


def build_host_selftest(folder: Optional[str] = None) -> str:
    """Builds the host library's sources together with ``selftest.cpp`` into one program under
    the address and undefined-behaviour sanitizers and returns its path. The program drives the
    C entry points through random request lifetimes and scheduler runs and exits with 0 when
    every check held and the sanitizers found nothing."""
    folder = folder or _writable_dir()
    program = os.path.join(folder, "host_selftest_sanitized")
    units = sorted(os.path.join(HOST_DIR, f) for f in os.listdir(HOST_DIR) if f.endswith(".cpp"))
    result = subprocess.run([_host_compiler(), *SANITIZE_FLAGS, "-o", program, *units], capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"building the sanitized host self-test failed:\n{result.stderr}")
    return program


def ensure_host_built() -> str:
    lib = find_host_library(require_current=True)
    if lib is not None:
        return lib
    try:
        return build_host()
    except RuntimeError:
        stale = find_host_library(require_current=False)
        if stale is not None:
            _say(f"warning: could not rebuild; loading {stale}, which is older than the sources")
            return stale
        raise


# ----- the plain C++ references of the kernels: host code, for tests ------------------------------
REFERENCE_DIR = os.path.join(CSRC, "reference")
REFERENCE_LIB_NAME = "libflyweight_reference.so"


def _reference_fingerprint() -> str:
    digest = hashlib.sha256()
    for name in sorted(os.listdir(REFERENCE_DIR)):
        if name.endswith((".cpp", ".h")):
            digest.update(name.encode())
            with open(os.path.join(REFERENCE_DIR, name), "rb") as handle:
                digest.update(handle.read())
    digest.update(" ".join(HOST_FLAGS).encode())
    return digest.hexdigest()


def build_reference(verbose: bool = True) -> str:
    folder = _writable_dir()
    started = time.time()
    units = sorted(os.path.join(REFERENCE_DIR, f) for f in os.listdir(REFERENCE_DIR) if f.endswith(".cpp"))
    lib = os.path.join(folder, REFERENCE_LIB_NAME)
    partial = lib + f".{os.getpid()}.tmp"
    result = subprocess.run([_host_compiler(), *HOST_FLAGS, "-o", partial, *units], capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"building {REFERENCE_LIB_NAME} failed:\n{result.stderr}")
    os.replace(partial, lib)
    with open(os.path.join(folder, "reference.stamp"), "w", encoding="utf-8") as handle:
        handle.write(_reference_fingerprint())
    if verbose:
        _say(f"built {lib} in {time.time() - started:.0f} s")
    return lib


def ensure_reference_built() -> str:
    wanted = _reference_fingerprint()
    for folder in build_dirs():
        lib, stamp = os.path.join(folder, REFERENCE_LIB_NAME), os.path.join(folder, "reference.stamp")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp, "r", encoding="utf-8") as handle:
                if handle.read().strip() == wanted:
                    return lib
    return build_reference()


if __name__ == "__main__":
    build()
    build_host()
    build_reference()
