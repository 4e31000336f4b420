"""Compiles the native code in-tree: the gfx950 kernels (hipcc) and the host
runtime (g++), each into one shared library next to the sources.

The libraries are loaded with ctypes; nothing here needs torch's extension
builder, a writable HOME or a network.  ``build_*`` always compiles;
``ensure_*`` compiles when the library is missing or was built from other
sources than those that lie beside it now (a digest of the sources is kept next
to each library).
"""

from __future__ import annotations

import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.dirname(os.path.abspath(__file__))
HIP_DIR = os.path.join(CSRC, "hip")
HOST_DIR = os.path.join(CSRC, "host")
KERNEL_LIB = os.path.join(CSRC, "libmgpt_kernels.so")
HOST_LIB = os.path.join(CSRC, "libmgpt_host.so")

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep hipcc from forming packed 32-bit float instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results in ordinary registers: left to itself the compiler puts them into the
    # accumulation registers and copies each one out again for the arithmetic that follows
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
]


HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-D_GLIBCXX_ASSERTIONS"]


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[mini_gpt_inference_amd build] {msg}", file=sys.stderr, flush=True)


def _find(tool: str, extra_dirs: tuple[str, ...] = ()) -> str:
    found = shutil.which(tool)
    if found:
        return found
    for d in extra_dirs:
        cand = os.path.join(d, tool)
        if os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError(f"{tool} not found; it is needed to compile the native code")


def _run(cmd: list[str], what: str) -> None:
    """Runs one compiler command, printing a line now and then while it works."""
    done = threading.Event()

    def ticker() -> None:
        start = time.time()
        while not done.wait(10.0):
            _say(f"still compiling {what} ({time.time() - start:.0f} s)")

    t = threading.Thread(target=ticker, daemon=True)
    t.start()
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    finally:
        done.set()
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{' '.join(cmd)}\n{proc.stdout}")


def _writable_target(path: str) -> str:
    """The in-tree path if its folder can be written, else a per-user folder under the temp dir."""
    folder = os.path.dirname(path)
    if os.access(folder, os.W_OK):
        return path
    alt = os.path.join(tempfile.gettempdir(), f"mgpt_build_{os.getuid()}")
    os.makedirs(alt, exist_ok=True)
    return os.path.join(alt, os.path.basename(path))


def kernel_sources() -> list[str]:
    return sorted(glob.glob(os.path.join(HIP_DIR, "*.hip")) + glob.glob(os.path.join(HIP_DIR, "*.h")))


def host_sources() -> list[str]:
    return sorted(glob.glob(os.path.join(HOST_DIR, "*.cpp")) + glob.glob(os.path.join(HOST_DIR, "*.h")))


def sources_digest(files: list[str], flags: list[str]) -> str:
    """A digest of the sources' names and contents and of the compiler's flags."""
    h = hashlib.sha256(" ".join(flags).encode())
    for path in files:
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _stamp(lib: str) -> str:
    return lib + ".digest"


def _write_stamp(lib: str, digest: str) -> None:
    with open(_stamp(lib), "w", encoding="ascii") as fh:
        fh.write(digest)


def is_current(lib: str, digest: str) -> bool:
    """Whether the library exists and was built from sources with this digest."""
    try:
        with open(_stamp(lib), encoding="ascii") as fh:
            return os.path.isfile(lib) and fh.read().strip() == digest
    except OSError:
        return False


def kernel_lib_path() -> str:
    return KERNEL_LIB if os.path.isfile(KERNEL_LIB) else _writable_target(KERNEL_LIB)


def host_lib_path() -> str:
    return HOST_LIB if os.path.isfile(HOST_LIB) else _writable_target(HOST_LIB)


def build_kernels() -> str:
    hipcc = _find("hipcc", ("/opt/rocm/bin",))
    sources = sorted(glob.glob(os.path.join(HIP_DIR, "*.hip")))
    if not sources:
        raise BuildError(f"no kernel sources under {HIP_DIR}")
    target = _writable_target(KERNEL_LIB)
    objdir = tempfile.mkdtemp(prefix="mgpt_obj_")
    try:
        _say(f"compiling {len(sources)} gfx950 kernel files with hipcc")
        errors: list[BaseException] = []
        objects = []

        def compile_one(src: str, obj: str) -> None:
            try:
                _run([hipcc, *HIP_FLAGS, "-I", HIP_DIR, "-c", src, "-o", obj], os.path.basename(src))
            except BaseException as exc:  # collected and raised by the caller
                errors.append(exc)

        threads = []
        for src in sources:
            obj = os.path.join(objdir, os.path.basename(src) + ".o")
            objects.append(obj)
            th = threading.Thread(target=compile_one, args=(src, obj))
            th.start()
            threads.append(th)
        for th in threads:
            th.join()
        if errors:
            raise errors[0]
        tmp = target + f".tmp{os.getpid()}"
        digest = sources_digest(kernel_sources(), HIP_FLAGS)
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", tmp], "kernel library")
        os.replace(tmp, target)
        _write_stamp(target, digest)
    finally:
        shutil.rmtree(objdir, ignore_errors=True)
    _say(f"built {target}")
    return target


def build_host() -> str:
    cxx = _find("g++")
    sources = sorted(glob.glob(os.path.join(HOST_DIR, "*.cpp")))
    if not sources:
        raise BuildError(f"no host sources under {HOST_DIR}")
    target = _writable_target(HOST_LIB)
    tmp = target + f".tmp{os.getpid()}"
    _say("compiling the host runtime with g++")
    # _GLIBCXX_ASSERTIONS: an index past the end of a vector stops the process with a message instead
    # of reading whatever lies there (the scheduler's and the cache manager's work is small: the
    # checks cost nothing that a step would notice)
    digest = sources_digest(host_sources(), HOST_FLAGS)
    _run([cxx, *HOST_FLAGS, "-I", HOST_DIR, *sources, "-o", tmp], "host runtime")
    os.replace(tmp, target)
    _write_stamp(target, digest)
    _say(f"built {target}")
    return target


def ensure_kernels() -> str:
    """The kernel library's path; compiles it first if there is none or if a source has changed
    since it was built."""
    path = kernel_lib_path()
    if not is_current(path, sources_digest(kernel_sources(), HIP_FLAGS)):
        if os.path.isfile(path):
            _say("the kernel sources have changed since the library was built")
        path = build_kernels()
    return path


def ensure_host() -> str:
    path = host_lib_path()
    if not is_current(path, sources_digest(host_sources(), HOST_FLAGS)):
        if os.path.isfile(path):
            _say("the host sources have changed since the library was built")
        path = build_host()
    return path


def build_all() -> None:
    build_host()
    build_kernels()


if __name__ == "__main__":
    build_all()
