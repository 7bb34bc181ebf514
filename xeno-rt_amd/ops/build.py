"""Compile the HIP sources under csrc/ for gfx950 into one shared library, in the tree.

Each source file is compiled by its own hipcc process (in parallel), then the objects
are linked. While it works it prints a line now and then, because a first build takes
a minute. The library and a record of the sources' hash lie next to this file; if that
folder cannot be written, a folder under the temporary directory is used instead.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor, as_completed

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
LIBRARY_NAME = "libxrt_hip.so"
ARCH = "gfx950"
# packed float32 arithmetic is switched off for all device code of this library
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


class BuildError(RuntimeError):
    pass


def sources():
    return sorted(os.path.join(CSRC, name) for name in os.listdir(CSRC) if name.endswith(".hip"))


def source_hash() -> str:
    digest = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            digest.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as handle:
                digest.update(handle.read())
    digest.update(" ".join(FLAGS).encode())
    return digest.hexdigest()[:16]


def _hipcc() -> str:
    for candidate in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise BuildError("hipcc not found: the HIP kernels cannot be compiled")


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


def library_folders():
    """Where the library may lie: in the tree first, else under the temporary directory."""
    return [HERE, os.path.join(tempfile.gettempdir(), f"xrt_hip_{os.getuid()}")]


def find_library(require_fresh: bool = True):
    """Path of a built library (whose sources' hash matches, if require_fresh), or None."""
    wanted = source_hash()
    for folder in library_folders():
        path = os.path.join(folder, LIBRARY_NAME)
        stamp = path + ".hash"
        if os.path.isfile(path):
            if not require_fresh:
                return path
            if os.path.isfile(stamp) and open(stamp).read().strip() == wanted:
                return path
    return None


def build(verbose: bool = True) -> str:
    """Compile everything and return the library's path."""
    hipcc = _hipcc()
    folder = next((f for f in library_folders() if _writable(f)), None)
    if folder is None:
        raise BuildError("no writable folder for the kernel library")
    objects_folder = os.path.join(folder, "_build")
    os.makedirs(objects_folder, exist_ok=True)
    files = sources()
    started = time.time()

    def say(text):
        if verbose:
            print(f"[xrt build] {text}", file=sys.stderr, flush=True)

    say(f"compiling {len(files)} HIP files for {ARCH} into {folder}")

    def compile_one(path):
        obj = os.path.join(objects_folder, os.path.basename(path)[:-4] + ".o")
        done = subprocess.run([hipcc, *FLAGS, "-I", CSRC, "-c", path, "-o", obj],
                              capture_output=True, text=True)
        return path, obj, done

    objects = []
    workers = max(1, min(8, os.cpu_count() or 1, len(files)))
    with ThreadPoolExecutor(workers) as pool:
        futures = [pool.submit(compile_one, path) for path in files]
        for count, future in enumerate(as_completed(futures), 1):
            path, obj, done = future.result()
            if done.returncode != 0:
                raise BuildError(f"hipcc failed on {path}:\n{done.stderr}")
            objects.append(obj)
            say(f"{count}/{len(files)} {os.path.basename(path)} ({time.time() - started:.0f} s)")
    library = os.path.join(folder, LIBRARY_NAME)
    partial = library + f".{os.getpid()}.tmp"
    done = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", partial, *sorted(objects)],
                          capture_output=True, text=True)
    if done.returncode != 0:
        raise BuildError(f"linking {library} failed:\n{done.stderr}")
    os.replace(partial, library)
    with open(library + ".hash", "w") as handle:
        handle.write(source_hash() + "\n")
    say(f"built {library} in {time.time() - started:.0f} s")
    return library


# ---- the plain C++ references of the kernels (csrc/reference/): host code, built with the host compiler ----------

REFERENCE = os.path.join(CSRC, "reference")
REFERENCE_LIBRARY = "libxrt_ref.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-Wall", "-Wextra"]
SANITIZE_FLAGS = ["-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan"]


def _host_compiler() -> str:
    for name in ("g++", "c++", "clang++"):
        found = shutil.which(name)
        if found:
            return found
    raise BuildError("no host C++ compiler found: the plain C++ references cannot be compiled")


def reference_hash() -> str:
    digest = hashlib.sha256()
    for name in sorted(os.listdir(REFERENCE)):
        with open(os.path.join(REFERENCE, name), "rb") as handle:
            digest.update(name.encode())
            digest.update(handle.read())
    return digest.hexdigest()[:16]


def find_reference_library():
    wanted = reference_hash()
    for folder in library_folders():
        path = os.path.join(folder, REFERENCE_LIBRARY)
        stamp = path + ".hash"
        if os.path.isfile(path) and os.path.isfile(stamp) and open(stamp).read().strip() == wanted:
            return path
    return None


def build_reference(verbose: bool = True) -> str:
    """Compile csrc/reference/reference.cpp for the CPU into a shared library of its own; returns its path."""
    folder = next((f for f in library_folders() if _writable(f)), None)
    if folder is None:
        raise BuildError("no writable folder for the reference library")
    library = os.path.join(folder, REFERENCE_LIBRARY)
    partial = library + f".{os.getpid()}.tmp"
    done = subprocess.run([_host_compiler(), *HOST_FLAGS, "-fPIC", "-shared", "-o", partial,
                           os.path.join(REFERENCE, "reference.cpp")], capture_output=True, text=True)
    if done.returncode != 0:
        raise BuildError(f"compiling the C++ references failed:\n{done.stderr}")
    os.replace(partial, library)
    with open(library + ".hash", "w") as handle:
        handle.write(reference_hash() + "\n")
    if verbose:
        print(f"[xrt build] built {library}", file=sys.stderr, flush=True)
    return library


# ---- the host library (csrc/host/): the runtime's bookkeeping on the CPU, built with the host compiler ----------

HOST = os.path.join(CSRC, "host")
HOST_LIBRARY = "libxrt_host.so"


def host_hash() -> str:
    digest = hashlib.sha256()
    for name in sorted(os.listdir(HOST)):
        with open(os.path.join(HOST, name), "rb") as handle:
            digest.update(name.encode())
            digest.update(handle.read())
    return digest.hexdigest()[:16]


def find_host_library():
    wanted = host_hash()
    for folder in library_folders():
        path = os.path.join(folder, HOST_LIBRARY)
        stamp = path + ".hash"
        if os.path.isfile(path) and os.path.isfile(stamp) and open(stamp).read().strip() == wanted:
            return path
    return None


def build_host(verbose: bool = True) -> str:
    """Compile csrc/host/xrt_host.cpp for the CPU into a shared library; returns its path."""
    folder = next((f for f in library_folders() if _writable(f)), None)
    if folder is None:
        raise BuildError("no writable folder for the host library")
    library = os.path.join(folder, HOST_LIBRARY)
    partial = library + f".{os.getpid()}.tmp"
    done = subprocess.run([_host_compiler(), *HOST_FLAGS, "-fPIC", "-shared", "-o", partial,
                           os.path.join(HOST, "xrt_host.cpp")], capture_output=True, text=True)
    if done.returncode != 0:
        raise BuildError(f"compiling the host library failed:\n{done.stderr}")
    os.replace(partial, library)
    with open(library + ".hash", "w") as handle:
        handle.write(host_hash() + "\n")
    if verbose:
        print(f"[xrt build] built {library}", file=sys.stderr, flush=True)
    return library


def build_host_selftest(sanitize: bool = True) -> str:
    """Compile the host library with its self-test (csrc/host/selftest.cpp) into a program, under the host's address
    and undefined-behaviour sanitizers unless told otherwise; returns its path."""
    folder = os.path.join(next((f for f in library_folders() if _writable(f)), tempfile.gettempdir()), "_build")
    os.makedirs(folder, exist_ok=True)
    program = os.path.join(folder, "host_selftest" + ("_sanitized" if sanitize else ""))
    flags = SANITIZE_FLAGS if sanitize else HOST_FLAGS
    done = subprocess.run([_host_compiler(), *flags, "-o", program, os.path.join(HOST, "selftest.cpp"),
                           os.path.join(HOST, "xrt_host.cpp")], capture_output=True, text=True)
    if done.returncode != 0:
        raise BuildError(f"compiling the host library's self-test failed:\n{done.stderr}")
    return program


def build_reference_selftest(sanitize: bool = True) -> str:
    """Compile the references with their self-test (csrc/reference/selftest.cpp) into a program, under the host's
    address and undefined-behaviour sanitizers unless told otherwise; returns its path."""
    folder = os.path.join(next((f for f in library_folders() if _writable(f)), tempfile.gettempdir()), "_build")
    os.makedirs(folder, exist_ok=True)
    program = os.path.join(folder, "reference_selftest" + ("_sanitized" if sanitize else ""))
    flags = SANITIZE_FLAGS if sanitize else HOST_FLAGS
    done = subprocess.run([_host_compiler(), *flags, "-o", program, os.path.join(REFERENCE, "selftest.cpp"),
                           os.path.join(REFERENCE, "reference.cpp")], capture_output=True, text=True)
    if done.returncode != 0:
        raise BuildError(f"compiling the references' self-test failed:\n{done.stderr}")
    return program


if __name__ == "__main__":
    print(build())
    print(build_reference())
    print(build_host())
