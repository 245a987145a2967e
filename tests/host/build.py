"""Builds tests/host/host_tests, the C++ unit tests of the host layer: test infrastructure, linked against
the two product libraries and the CPU oracle (which the tests register as the registry's CPU arm).

    python tests/host/build.py          the test program the test suite runs
    python tests/host/build.py --asan   the CPU part again with AddressSanitizer + UBSan: the host layer, the
                                        pool and the C ABI are compiled into the program itself so that they
                                        are instrumented; only the kernels' launchers come from libllmi_hip.so.
                                        Host code only: it is never run on a GPU box.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
PKG = os.path.join(ROOT, "llminfer_amd")
CSRC = os.path.join(PKG, "csrc")
ORACLE = os.path.join(ROOT, "oracle")
EXE = os.path.join(HERE, "host_tests")
EXE_ASAN = os.path.join(HERE, "host_tests_asan")


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return res.stdout


def build(asan=False):
    subprocess.run(["make", "-C", ORACLE, "libllmi_oracle.so"], check=True, stdout=subprocess.DEVNULL)
    hipcc = os.environ.get("HIPCC", "hipcc")
    host_dir = os.path.join(CSRC, "host")
    common = ["-std=c++17", "-Wall", "-Wno-unused-command-line-argument", "-I" + os.path.join(ROOT, "include"),
              "-I" + host_dir, "-I" + CSRC, "-I" + ORACLE]
    rpath = ["-Wl,-rpath,$ORIGIN/../../llminfer_amd", "-Wl,-rpath,$ORIGIN/../../oracle"]
    if not asan:
        cmd = [hipcc, "-O1"] + common + [os.path.join(HERE, "test_host.cpp"), "-L" + PKG, "-lllmi_host", "-lllmi_hip",
                                         "-L" + ORACLE, "-lllmi_oracle"] + rpath + ["-o", EXE]
        _run(cmd)
        return EXE
    host_srcs = sorted(os.path.join(host_dir, f) for f in os.listdir(host_dir) if f.endswith(".cpp"))
    srcs = [os.path.join(HERE, "test_host.cpp")] + host_srcs + [os.path.join(CSRC, "pool.cpp"), os.path.join(CSRC, "c_api.cpp")]
    cmd = [hipcc, "-O1", "-g", "-fno-omit-frame-pointer", "-fno-gpu-sanitize", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined"] + common + srcs
    cmd += ["-L" + PKG, "-lllmi_hip", "-L" + ORACLE, "-lllmi_oracle"] + rpath + ["-o", EXE_ASAN]
    _run(cmd)
    return EXE_ASAN


if __name__ == "__main__":
    print("built", build(asan="--asan" in sys.argv[1:]))
