"""Compile the sources under `csrc/` into two shared libraries.

The HIP kernels (`csrc/*.hip`): `hipcc` turns each file into an object for gfx950 (in parallel), then links
them.  The host core (`csrc/host/*.cpp`: page allocator, cache manager, batch packing, host sampler): one
call of the C++ compiler, no GPU code and no dependency on HIP.  A library lands beside this package when
that folder can be written, else in a per-user folder under the temporary directory.
"""
from __future__ import annotations

import concurrent.futures
import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE_DIR = os.path.join(PACKAGE_DIR, "csrc")
LIB_NAME = "libtokenizer_amd_kernels.so"
HOST_LIB_NAME = "libtokenizer_amd_host.so"
HOST_SOURCE_DIR = os.path.join(SOURCE_DIR, "host")
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra"]
ARCH = "gfx950"
# Packed float32 instructions are switched off for all device code.
HIPCC_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               # Matrix-core accumulators stay in ordinary registers: the softmax and the epilogues work on
               # them with vector instructions, which cannot read the accumulation registers directly.
               "-mllvm", "-amdgpu-mfma-vgpr-form=1",
               # The first sixteen words of a kernel's arguments are in scalar registers when a wave starts,
               # instead of being fetched by its first instructions (a trip to memory at the head of every kernel;
               # kernels begin with code that fetches them all the same where the firmware does not do this).
               "-mllvm", "-amdgpu-kernarg-preload-count=16",
               "-Wno-unused-command-line-argument"]


# The vendor's matrix library, for the plain products that go to it (library_gemm.hip).
ROCM_LIB_DIR = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")
LINK_FLAGS = [f"-L{ROCM_LIB_DIR}", "-lhipblaslt", f"-Wl,-rpath,{ROCM_LIB_DIR}"]


def _say(message: str) -> None:
    print(f"[tokenizer_amd build] {message}", file=sys.stderr, flush=True)


def hipcc_path() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                       "the HIP kernels cannot be built")


def library_candidates(name: str = LIB_NAME) -> list[str]:
    fallback = os.path.join(tempfile.gettempdir(), f"tokenizer_amd_{os.getuid()}")
    return [os.path.join(PACKAGE_DIR, name), os.path.join(fallback, name)]


def _first_built(name: str) -> str | None:
    for path in library_candidates(name):
        if os.path.exists(path):
            return path
    return None


def kernel_sources() -> list[str]:
    """Everything the kernel library is compiled from: the HIP files and the headers beside them."""
    return sorted(glob.glob(os.path.join(SOURCE_DIR, "*.hip")) + glob.glob(os.path.join(SOURCE_DIR, "*.h")))


def _digest(sources: list[str], flags: list[str]) -> str:
    """A digest of what a library is built from: the text of its sources and the compiler's flags."""
    digest = hashlib.sha256(" ".join(flags).encode())
    for source in sources:
        digest.update(os.path.basename(source).encode() + b"\0")
        with open(source, "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()


def _stamp_of(path: str) -> str | None:
    try:
        with open(path + ".stamp") as handle:
            return handle.read().strip()
    except OSError:
        return None


def _write_stamp(path: str, digest: str) -> None:
    with open(path + ".stamp", "w") as handle:
        handle.write(digest + "\n")


def find_library(name: str = LIB_NAME) -> str | None:
    """A built kernel library that was built from the sources as they are now (an edited kernel beside an old
    library would otherwise run the old code without a word): the build leaves a digest of its sources beside
    the library, which is compared with theirs.  None if there is no such library, and the caller builds it."""
    path = _first_built(name)
    if path is None or name != LIB_NAME:
        return path
    if _stamp_of(path) != _digest(kernel_sources(), HIPCC_FLAGS):
        _say(f"{path} was not built from the sources under {SOURCE_DIR} as they are now: it is not used")
        return None
    return path


def _writable_target(name: str = LIB_NAME) -> str:
    for path in library_candidates(name):
        folder = os.path.dirname(path)
        try:
            os.makedirs(folder, exist_ok=True)
            probe = os.path.join(folder, f".write_probe_{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return path
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel library")


def _compile_one(hipcc: str, source: str, obj: str) -> tuple[str, float]:
    started = time.time()
    proc = subprocess.run([hipcc, *HIPCC_FLAGS, "-I", SOURCE_DIR, "-c", source, "-o", obj],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {os.path.basename(source)}:\n{proc.stderr[-4000:]}")
    return os.path.basename(source), time.time() - started


def build_library(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = hipcc_path()
    sources = sorted(glob.glob(os.path.join(SOURCE_DIR, "*.hip")))
    if not sources:
        raise RuntimeError(f"no HIP sources under {SOURCE_DIR}")
    target = _writable_target()
    env_home = os.environ.get("HOME")
    if not env_home or not os.access(env_home, os.W_OK):
        os.environ["HOME"] = tempfile.gettempdir()  # the compiler wants a place for its caches
    started = time.time()
    with tempfile.TemporaryDirectory(prefix="tokenizer_amd_obj_") as obj_dir:
        if verbose:
            _say(f"compiling {len(sources)} HIP sources for {ARCH} with {hipcc}")
        objects = []
        workers = max(1, min(len(sources), (os.cpu_count() or 2), 16))
        with concurrent.futures.ThreadPoolExecutor(workers) as pool:
            futures = []
            for source in sources:
                obj = os.path.join(obj_dir, os.path.basename(source) + ".o")
                objects.append(obj)
                futures.append(pool.submit(_compile_one, hipcc, source, obj))
            for future in concurrent.futures.as_completed(futures):
                name, seconds = future.result()
                if verbose:
                    _say(f"  {name} done in {seconds:.1f} s ({time.time() - started:.0f} s elapsed)")
        partial = target + f".{os.getpid()}.tmp"
        proc = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objects, *LINK_FLAGS, "-o", partial],
                              capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"linking the kernel library failed:\n{proc.stderr[-4000:]}")
        os.replace(partial, target)
        _write_stamp(target, _digest(kernel_sources(), HIPCC_FLAGS))
    if verbose:
        _say(f"built {target} in {time.time() - started:.1f} s")
    return target


def host_compiler() -> str:
    for candidate in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                      "/opt/rocm/lib/llvm/bin/clang++"):
        if candidate and (os.path.exists(candidate) or shutil.which(candidate)):
            return candidate
    raise RuntimeError("no C++ compiler was found (looked at $CXX, g++, c++, clang++); the host library cannot be built")


def host_sources() -> list[str]:
    return sorted(glob.glob(os.path.join(HOST_SOURCE_DIR, "*.cpp")))


def find_host_library() -> str | None:
    """A built host library that was built from its sources as they are now."""
    path = _first_built(HOST_LIB_NAME)
    if path is None:
        return None
    return path if _stamp_of(path) == _digest(_host_inputs(), HOST_FLAGS) else None


def _host_inputs() -> list[str]:
    return sorted(glob.glob(os.path.join(HOST_SOURCE_DIR, "*.cpp")) + glob.glob(os.path.join(HOST_SOURCE_DIR, "*.h")))


def build_host_library(verbose: bool = True) -> str:
    """Compile the host core; returns the library's path."""
    sources = host_sources()
    if not sources:
        raise RuntimeError(f"no C++ sources under {HOST_SOURCE_DIR}")
    compiler, target = host_compiler(), _writable_target(HOST_LIB_NAME)
    started = time.time()
    partial = target + f".{os.getpid()}.tmp"
    proc = subprocess.run([compiler, *HOST_FLAGS, "-I", HOST_SOURCE_DIR, *sources, "-o", partial],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"compiling the host library failed:\n{proc.stderr[-4000:]}")
    os.replace(partial, target)
    _write_stamp(target, _digest(_host_inputs(), HOST_FLAGS))
    if verbose:
        _say(f"built {target} in {time.time() - started:.1f} s")
    return target


if __name__ == "__main__":
    build_host_library()
    build_library()
