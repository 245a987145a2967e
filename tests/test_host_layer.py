"""Runs the C++ unit tests of the host layer (tests/host/test_host.cpp, built in-tree by
tests/host/build.py): tensor / buffer / allocator / op layer / registry, CPU part here, GPU part on a GPU;
the CPU part a second time under AddressSanitizer + UBSan."""
import importlib.util
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "host", "host_tests")


def _builder():
    spec = importlib.util.spec_from_file_location("host_tests_build", os.path.join(ROOT, "tests", "host", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _run(which):
    if not os.path.exists(EXE):
        from llminfer_amd import build
        build.build_all()
        _builder().build()
    res = subprocess.run([EXE, which], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(res.stdout)
    failed = [l for l in res.stdout.splitlines() if l.startswith("FAIL")]
    assert res.returncode == 0 and not failed, res.stdout[-3000:]
    assert "0 failed" in res.stdout


def test_host_layer_cpu():
    _run("cpu")


@pytest.mark.gpu
def test_host_layer_gpu(dev):
    _run("gpu")


def test_host_layer_cpu_under_sanitizers():
    """The same CPU tests with the host layer, the pool and the C ABI compiled with -fsanitize=address,undefined
    (host code only; leak checking is off because the HIP runtime the program links keeps its own allocations)."""
    exe = _builder().build(asan=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    res = subprocess.run([exe, "cpu"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600, env=env)
    print(res.stdout[-4000:])
    assert res.returncode == 0, res.stdout[-4000:]
    assert "0 failed" in res.stdout and "ERROR: AddressSanitizer" not in res.stdout and "runtime error" not in res.stdout
