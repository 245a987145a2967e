"""Builds libllmi_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libllmi_hip.so")
HOST_LIB_PATH = os.path.join(HERE, "libllmi_host.so")
DIAG_LIB_PATH = os.path.join(HERE, "libllmi_diag.so")

HIP_SOURCES = ["mha_decode_group4.hip", "mha_decode_group8.hip", "mha_decode_group16.hip", "mha_decode_group2.hip", "mha_decode_group1.hip", "mha_stack.hip",
               "mha_decode.hip", "qk_norm_rope.hip", "gemv.hip", "probes.hip", "c_api.cpp", "pool.cpp"]
DIAG_SOURCES = ["diag_probes.hip"]

# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU ops.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


def kernels_using_scratch(compiler_output):
    """Names of the kernels the compiler gave private (scratch) memory, from its resource-usage remarks. None of the
    kernels here may have any: a kernel with a private segment pays for its set-up at every launch, also when the
    path that spilled never runs (an indexed local array in a rarely taken branch cost 0.1 us per decode call)."""
    bad, name = [], None
    for line in compiler_output.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            if int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0]) != 0:
                bad.append(name)
    return bad


def _compile_objects(sources, defines, tag):
    """Each source to an object file (in parallel: the kernels' file takes minutes, the others seconds), the
    compiler's remarks of all of them joined."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "hipcc")
    obj_dir = os.path.join(HERE, "build", tag)
    os.makedirs(obj_dir, exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]

    def one(src):
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        cmd = [hipcc] + flags + ["-c", "-Rpass-analysis=kernel-resource-usage"] + ["-D" + d for d in defines]
        cmd += ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC, src, "-o", obj]
        return obj, _run(cmd)

    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        results = list(pool.map(one, sources))
    return [o for o, _ in results], "\n".join(out for _, out in results)


def _link_shared(objects, output):
    hipcc = os.environ.get("HIPCC", "hipcc")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objects + ["-o", output])
    return output


def _check_remarks(out, verbose):
    bad = kernels_using_scratch(out)
    if bad:
        raise RuntimeError("kernels with a private (scratch) segment: %s" % ", ".join(sorted(set(bad))))
    # (the remarks themselves are not worth printing: a dozen lines for each of a hundred kernels)
    out = "\n".join(l for l in out.splitlines() if "-Rpass-analysis" not in l and not re.match(r"^\s*\d*\s*\|", l)
                    and not l.startswith("In file included from"))
    if verbose and out.strip():
        print(out)


def build_hip_library(verbose=False, defines=(), output=None, only=()):
    """`defines`: extra NAME=VALUE macros (the kernels' build-time switches, e.g. LLMI_PV_VALU=1);
    `output`: where to write a variant build instead of the in-tree library; `only`: the sources the defines
    matter to (the others are taken from the in-tree build's objects, which must exist)."""
    tag = "hip" if not (defines or output) else "variant_" + re.sub(r"[^A-Za-z0-9_.-]", "_", os.path.basename(output or "x"))
    sources = [s for s in HIP_SOURCES if not only or s in only]
    objects, out = _compile_objects([os.path.join(CSRC, s) for s in sources], list(defines), tag)
    _check_remarks(out, verbose)
    objects += [os.path.join(HERE, "build", "hip", s + ".o") for s in HIP_SOURCES if s not in sources]
    return _link_shared(objects, output or LIB_PATH)


def build_diag_library(verbose=False):
    """libllmi_diag.so: the two diagnostic probes (include/llmi_hip_diag.h), a library of their own."""
    objects, out = _compile_objects([os.path.join(CSRC, "diag", s) for s in DIAG_SOURCES], [], "diag")
    _check_remarks(out, verbose)
    return _link_shared(objects, DIAG_LIB_PATH)


def build_host_library(verbose=False):
    """The C++17 mirror of the reference's tensor/op/registry interface, linked against libllmi_hip.so."""
    host_dir = os.path.join(CSRC, "host")
    if not os.path.isdir(host_dir):
        return None
    srcs = sorted(os.path.join(host_dir, f) for f in os.listdir(host_dir) if f.endswith(".cpp"))
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-command-line-argument",
           "-I" + os.path.join(ROOT, "include"), "-I" + host_dir] + srcs
    cmd += ["-L" + HERE, "-lllmi_hip", "-Wl,-rpath,$ORIGIN", "-o", HOST_LIB_PATH]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return HOST_LIB_PATH


def build_all(verbose=False):
    paths = [build_hip_library(verbose), build_diag_library(verbose)]
    host = build_host_library(verbose)
    if host:
        paths.append(host)
    return paths


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="Builds the gfx950 library and the host layer in-tree, or a variant of the library.")
    ap.add_argument("--define", action="append", default=[], metavar="NAME=VALUE",
                    help="build-time switch of the kernels (LLMI_PV_VALU=1, LLMI_STAGES=3, ...); needs --output")
    ap.add_argument("--output", default=None, help="write a variant of libllmi_hip.so here (load it with LLMI_HIP_LIBRARY)")
    ap.add_argument("--only", action="append", default=[], metavar="SOURCE",
                    help="recompile only this source (e.g. mha_stack.hip) for the variant; the rest comes from the in-tree build")
    cli = ap.parse_args()
    if cli.define or cli.output:
        if not cli.output:
            ap.error("--define needs --output: the in-tree library is always the default build")
        print("built", build_hip_library(verbose=True, defines=cli.define, output=os.path.abspath(cli.output), only=cli.only))
        sys.exit(0)
    for p in build_all(verbose=True):
        print("built", p)
    sys.exit(0)
