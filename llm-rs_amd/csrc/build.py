"""Builds and loads the native libraries.

`libllmrs_host.so`   g++     cache manager, batch builder, scheduler (csrc/host)
`libllmrs_hip.so`    hipcc   the gfx950 kernels and their launchers (csrc/hip)
`libllmrs_plain.so`  g++     plain C++ twins of the kernels (csrc/plain): the tests' second oracle, which
                             nothing in the package loads

They are built into `csrc/_build/` inside the package (or, when that folder
cannot be written, into a per-user folder under the temporary directory) the
first time they are needed, and again when a source has changed since.  There is
no other implementation to fall back to: if the HIP library cannot be built or
loaded, the call that needs it raises.
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
from typing import List, Optional

CSRC = os.path.dirname(os.path.abspath(__file__))
GPU_ARCH = "gfx950"
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={GPU_ARCH}",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-pthread", "-ffp-contract=off"]
# LLMRS_SANITIZE=1 in the environment: the two g++ libraries (raw-pointer C interfaces fed through ctypes) are built
# with the address and undefined-behaviour sanitizers, under names of their own beside the ordinary ones.  A Python
# that loads them needs the address sanitizer's runtime loaded first: `sanitizer_env()` gives the variables to start
# it with.  The kernel library is never built this way (there is no sanitizer for the device on these machines).
SANITIZE = os.environ.get("LLMRS_SANITIZE", "") not in ("", "0")
SANITIZE_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-g", "-O1"]
if SANITIZE:
    HOST_FLAGS = HOST_FLAGS + SANITIZE_FLAGS
_SUFFIX = "_san" if SANITIZE else ""


class BuildError(RuntimeError):
    pass


def _sources(sub: str, exts) -> List[str]:
    d = os.path.join(CSRC, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(tuple(exts)))


def _digest(sub: str) -> str:
    h = hashlib.sha256()
    for path in _sources(sub, (".h", ".cpp", ".hip")) + _sources("shared", (".h",)):   # both libraries include csrc/shared
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIP_FLAGS if sub == "hip" else HOST_FLAGS).encode())
    return h.hexdigest()


def _build_dir() -> str:
    d = os.path.join(CSRC, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        open(probe, "w").close()
        os.unlink(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"llmrs_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _say(msg: str) -> None:
    print(f"[llm-rs_amd build] {msg}", file=sys.stderr, flush=True)


def _run(cmd: List[str], what: str) -> None:
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        lines = [l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l]
        raise BuildError(f"{what} failed ({' '.join(cmd[:3])} ...):\n" + "\n".join(lines[-60:]))


def _is_current(lib: str, sub: str) -> bool:
    stamp = lib + ".stamp"
    if not (os.path.exists(lib) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == _digest(sub)


def _finish(lib: str, tmp: str, sub: str) -> None:
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(_digest(sub))


def build_host(force: bool = False) -> str:
    d = _build_dir()
    lib = os.path.join(d, f"libllmrs_host{_SUFFIX}.so")
    if not force and _is_current(lib, "host"):
        return lib
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if cxx is None:
        raise BuildError("no C++ compiler (g++) to build the host library with")
    _say("compiling the host library (cache manager, scheduler) ...")
    tmp = f"{lib}.{os.getpid()}.tmp"
    _run([cxx, *HOST_FLAGS, "-shared", "-o", tmp, *_sources("host", (".cpp",))], "host library build")
    _finish(lib, tmp, "host")
    return lib


def build_plain(force: bool = False) -> str:
    """The kernels' plain C++ twins (test equipment: the package has no CPU path and never loads them)."""
    d = _build_dir()
    lib = os.path.join(d, f"libllmrs_plain{_SUFFIX}.so")
    if not force and _is_current(lib, "plain"):
        return lib
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if cxx is None:
        raise BuildError("no C++ compiler (g++) to build the plain twins with")
    _say("compiling the kernels' plain C++ twins ...")
    tmp = f"{lib}.{os.getpid()}.tmp"
    _run([cxx, *HOST_FLAGS, "-shared", "-o", tmp, *_sources("plain", (".cpp",))], "plain twins build")
    _finish(lib, tmp, "plain")
    return lib


def sanitizer_env(env=None) -> dict:
    """The environment to start a Python in that is to load the sanitized host libraries: LLMRS_SANITIZE set, the
    address sanitizer's runtime first among the preloaded libraries (whatever was there stays behind it), and no
    leak report at exit (the interpreter itself never frees much of what it allocates)."""
    env = dict(os.environ if env is None else env)
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise BuildError("no g++ to ask for the sanitizer's runtime")
    runtime = subprocess.run([cxx, "-print-file-name=libasan.so"], capture_output=True, text=True).stdout.strip()
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        raise BuildError("this compiler has no address sanitizer runtime (libasan.so)")
    # (the C++ runtime too: the sanitizer looks up the real `__cxa_throw` when it starts, and an interpreter that is
    # not itself linked against libstdc++ has none to show then, so the first exception inside a library would abort)
    cxxlib = subprocess.run([cxx, "-print-file-name=libstdc++.so.6"], capture_output=True, text=True).stdout.strip()
    env["LLMRS_SANITIZE"] = "1"
    env["LD_PRELOAD"] = ":".join(x for x in (os.path.realpath(runtime), os.path.realpath(cxxlib) if os.path.isabs(cxxlib) else "",
                                             env.get("LD_PRELOAD", "")) if x)
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1:" + env.get("ASAN_OPTIONS", "")
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1:" + env.get("UBSAN_OPTIONS", "")
    return env


def _hipcc() -> Optional[str]:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


def build_hip(force: bool = False) -> str:
    d = _build_dir()
    lib = os.path.join(d, "libllmrs_hip.so")
    if not force and _is_current(lib, "hip"):
        return lib
    hipcc = _hipcc()
    if hipcc is None:
        raise BuildError("hipcc not found: the gfx950 kernel library cannot be built")
    srcs = _sources("hip", (".hip",))
    objdir = os.path.join(d, f"obj{os.getpid()}")
    os.makedirs(objdir, exist_ok=True)
    _say(f"compiling {len(srcs)} kernel files for {GPU_ARCH} (first call only) ...")
    start = time.time()

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        _run([hipcc, *HIP_FLAGS, "-c", src, "-o", obj], f"compiling {os.path.basename(src)}")
        _say(f"  {os.path.basename(src)} done ({time.time() - start:.0f}s)")
        return obj

    try:
        with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
            objs = list(ex.map(compile_one, srcs))
        tmp = f"{lib}.{os.getpid()}.tmp"
        _run([hipcc, "-shared", "-fPIC", f"--offload-arch={GPU_ARCH}", "-Wl,--no-undefined", "-o", tmp, *objs],
             "linking the kernel library")
        _finish(lib, tmp, "hip")
    finally:
        shutil.rmtree(objdir, ignore_errors=True)
    _say(f"kernel library ready ({time.time() - start:.0f}s)")
    return lib


_host_lib = None
_hip_lib = None


def load_host() -> ctypes.CDLL:
    global _host_lib
    if _host_lib is None:
        _host_lib = ctypes.CDLL(build_host())
    return _host_lib


def load_hip() -> ctypes.CDLL:
    """The kernel library; raises when it cannot be built or loaded."""
    global _hip_lib
    if _hip_lib is None:
        path = build_hip()
        try:
            _hip_lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"cannot load the kernel library {path}: {e}") from None
    return _hip_lib


def build_all(force: bool = True) -> None:
    build_host(force)
    build_plain(force)
    build_hip(force)
