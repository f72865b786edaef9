"""Builds the two native libraries from the sources in this folder.

``libleone_hip.so`` holds the gfx950 kernels (the ``.hip`` files here); ``hipcc``
cross-compiles them without a GPU.  ``libleone_host.so`` holds the host runtime
(cache manager, scheduler, step layout; plain C++ under ``host/``) and needs only
a C++ compiler.  Objects and libraries go to ``_build/`` beside the sources; if
that folder cannot be written (a read-only checkout) a per-user folder under the
system's temporary directory is used.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libleone_hip.so"
ARCH = "gfx950"
# Packed single-precision instructions are kept off for every device function.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wno-unused-result"] + DEVICE_FLAGS


def sources() -> list[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".h"))


def source_digest() -> str:
    digest = hashlib.sha256()
    for name in sources() + _headers():
        digest.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(FLAGS).encode())
    return digest.hexdigest()[:16]


HOST_DIR = os.path.join(HERE, "host")
HOST_LIB_NAME = "libleone_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall"]


def host_sources() -> list[str]:
    return sorted(f for f in os.listdir(HOST_DIR) if f.endswith(".cpp"))


def host_digest() -> str:
    digest = hashlib.sha256()
    for name in sorted(os.listdir(HOST_DIR)):
        if name.endswith((".cpp", ".h")):
            digest.update(name.encode())
            with open(os.path.join(HOST_DIR, name), "rb") as handle:
                digest.update(handle.read())
    digest.update(" ".join(HOST_FLAGS).encode())
    return digest.hexdigest()[:16]


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dir() -> str:
    in_tree = os.path.join(HERE, "_build")
    if _writable(in_tree):
        return in_tree
    fallback = os.path.join(tempfile.gettempdir(), f"leone_amd_build_{os.getuid()}")
    os.makedirs(fallback, exist_ok=True)
    return fallback


def _built(lib_name: str, stamp_name: str, digest: str) -> str | None:
    for folder in (os.path.join(HERE, "_build"),
                   os.path.join(tempfile.gettempdir(), f"leone_amd_build_{os.getuid()}")):
        lib = os.path.join(folder, lib_name)
        stamp = os.path.join(folder, stamp_name)
        if os.path.exists(lib) and os.path.exists(stamp):
            with open(stamp) as handle:
                if handle.read().strip() == digest:
                    return lib
    return None


def library_path() -> str | None:
    """The built kernel library that matches the present sources, if there is one."""
    return _built(LIB_NAME, "digest.txt", source_digest())


def host_library_path() -> str | None:
    """The built host library that matches the present sources, if there is one."""
    return _built(HOST_LIB_NAME, "digest_host.txt", host_digest())


def host_compiler() -> str:
    for name in ("g++", "c++", "clang++"):
        found = shutil.which(name)
        if found:
            return found
    return hipcc()      # its clang compiles plain C++ as well


def build_host(verbose: bool = True, force: bool = True) -> str:
    """Compiles the host runtime; returns the library's path."""
    if not force:
        ready = host_library_path()
        if ready:
            return ready
    out_dir = build_dir()
    started = time.time()
    lib = os.path.join(out_dir, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = ([host_compiler()] + HOST_FLAGS + ["-shared", "-I", HOST_DIR, "-o", tmp]
           + [os.path.join(HOST_DIR, name) for name in host_sources()])
    if verbose:
        print(f"[leone_amd] building {HOST_LIB_NAME} from {len(host_sources())} sources into {out_dir}",
              file=sys.stderr, flush=True)
    result = subprocess.run(cmd, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"the C++ compiler failed on the host library:\n{result.stderr}")
    os.replace(tmp, lib)
    with open(os.path.join(out_dir, "digest_host.txt"), "w") as handle:
        handle.write(host_digest() + "\n")
    if verbose:
        print(f"[leone_amd] built {lib} in {time.time() - started:.0f}s", file=sys.stderr, flush=True)
    return lib


def hipcc() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    candidate = "/opt/rocm/bin/hipcc"
    if os.path.exists(candidate):
        return candidate
    raise RuntimeError("hipcc not found: the kernel library cannot be built")


def build(verbose: bool = True, force: bool = True) -> str:
    """Compiles every source and links the library; returns its path."""
    if not force:
        ready = library_path()
        if ready:
            return ready
    out_dir = build_dir()
    compiler = hipcc()
    names = sources()
    started = time.time()
    done = threading.Event()

    def heartbeat():
        while not done.wait(10.0):
            if verbose:
                print(f"[leone_amd] compiling kernels for {ARCH} ... {time.time() - started:.0f}s",
                      file=sys.stderr, flush=True)

    def compile_one(name: str) -> str:
        obj = os.path.join(out_dir, name[:-4] + ".o")
        cmd = [compiler] + FLAGS + ["-I", HERE, "-c", os.path.join(HERE, name), "-o", obj]
        result = subprocess.run(cmd, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{result.stderr}")
        return obj

    if verbose:
        print(f"[leone_amd] building {LIB_NAME} from {len(names)} sources into {out_dir}",
              file=sys.stderr, flush=True)
    ticker = threading.Thread(target=heartbeat, daemon=True)
    ticker.start()
    try:
        workers = max(1, min(len(names), int(os.environ.get("MAX_JOBS", "8")), 16))
        with ThreadPoolExecutor(max_workers=workers) as pool:
            objects = list(pool.map(compile_one, names))
        lib = os.path.join(out_dir, LIB_NAME)
        tmp = lib + f".tmp{os.getpid()}"
        link = [compiler, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp] + objects
        result = subprocess.run(link, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed to link {LIB_NAME}:\n{result.stderr}")
        os.replace(tmp, lib)
        with open(os.path.join(out_dir, "digest.txt"), "w") as handle:
            handle.write(source_digest() + "\n")
    finally:
        done.set()
    if verbose:
        print(f"[leone_amd] built {lib} in {time.time() - started:.0f}s", file=sys.stderr, flush=True)
    return lib


def _tool_version(tool: str) -> str | None:
    try:
        out = subprocess.run([tool, "--version"], capture_output=True, text=True, timeout=30)
    except (OSError, subprocess.TimeoutExpired):
        return None
    lines = [line.strip() for line in (out.stdout or out.stderr).splitlines() if line.strip()]
    return lines[0] if lines else None


def build_info() -> dict:
    """Where the two native libraries come from: sources and flags (as digests), compilers, and whether the
    built files match the present sources.  The reference prints the same kind of record for its
    executable (crates/leone-cli/src/build_info.rs:37-75)."""
    from .. import __version__

    def one(name, names, flags, digest, path, compiler):
        return {"library": name, "sources": names, "flags": flags, "source_digest": digest,
                "built": path, "built_matches_sources": path is not None,
                "compiler": compiler, "compiler_version": _tool_version(compiler) if compiler else None}

    try:
        device_compiler = hipcc()
    except RuntimeError:
        device_compiler = None
    try:
        cxx = host_compiler()
    except RuntimeError:
        cxx = None
    return {"schema_version": "leone_amd.build-info.v1", "version": __version__, "target": ARCH,
            "python": sys.version.split()[0],
            "kernels": one(LIB_NAME, sources(), FLAGS, source_digest(), library_path(), device_compiler),
            "host": one(HOST_LIB_NAME, host_sources(), HOST_FLAGS, host_digest(), host_library_path(), cxx)}


if __name__ == "__main__":
    print(build_host())
    print(build())
