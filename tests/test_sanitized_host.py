"""The host libraries under the address and undefined-behaviour sanitizers.  `libllmrs_host.so` (page pool, cache
manager, batch flattening, scheduler) and `libllmrs_plain.so` (the kernels' plain twins) are C interfaces that take
raw pointers from ctypes: an index one past a block table or a freed request read again would go unnoticed in an
ordinary run.  Here their own CPU tests run once more in a Python started with LLMRS_SANITIZE=1 (csrc/build.py
builds both libraries with -fsanitize=address,undefined under names of their own) and the sanitizer's runtime
loaded first; any report ends that run with an error."""
import os
import subprocess
import sys

import pytest

from llm_rs_amd.csrc import build as native

HERE = os.path.dirname(os.path.abspath(__file__))
SUITES = ["test_cache_manager.py", "test_scheduler.py", "test_engine_cpu.py", "test_plain_twins.py"]


def test_host_libraries_under_sanitizers():
    try:
        env = native.sanitizer_env()
    except native.BuildError as e:
        pytest.skip(str(e))
    env["PYTHONFAULTHANDLER"] = "1"
    p = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider", *SUITES],
                       cwd=HERE, env=env, capture_output=True, text=True, timeout=1500)
    tail = (p.stdout + p.stderr)[-4000:]
    assert p.returncode == 0, tail
    assert "passed" in p.stdout and "ERROR: AddressSanitizer" not in tail and "runtime error:" not in tail, tail
    # the run did load the sanitized libraries, not the ordinary ones
    built = native._build_dir()
    assert os.path.exists(os.path.join(built, "libllmrs_host_san.so")) and os.path.exists(os.path.join(built, "libllmrs_plain_san.so"))


def test_the_sanitizer_sees_a_fault_in_such_a_library(tmp_path):
    """The equipment itself: a library built with the same flags that reads one element past an array ends the Python
    that calls it, with the sanitizer's report (so a green run above means something)."""
    try:
        env = native.sanitizer_env()
    except native.BuildError as e:
        pytest.skip(str(e))
    src = tmp_path / "past.cpp"
    src.write_text('#include <vector>\nextern "C" int past(int n) { std::vector<int> v(n, 1); int* p = v.data(); return p[n]; }\n')
    lib = tmp_path / "libpast.so"
    subprocess.run(["g++", *native.SANITIZE_FLAGS, "-shared", "-fPIC", "-o", str(lib), str(src)], check=True)
    p = subprocess.run([sys.executable, "-c", f"import ctypes; print(ctypes.CDLL({str(lib)!r}).past(8))"],
                       env=env, capture_output=True, text=True, timeout=120)
    assert p.returncode != 0 and "heap-buffer-overflow" in p.stderr, p.stderr[-2000:]
