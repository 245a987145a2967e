"""Runs the C++ unit tests of the host layer (tests/host/test_host.cpp, built in-tree by
llminfer_amd.build): tensor / buffer / allocator / op layer / registry, CPU part here, GPU part on a GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "host", "host_tests")


def _run(which):
    if not os.path.exists(EXE):
        from llminfer_amd import build
        build.build_all()
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
