"""Builds libhyena_mi355x.so (gfx950) in-tree with hipcc.

    python -m vortex_amd.build            # compile every source, link the shared library
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhyena_mi355x.so")
PROBE = os.path.join(HERE, "libhyena_probe.so")          # copy kernel for counter calibration; not part of the ABI
SELFTEST = os.path.join(HERE, "abi_selftest")          # plain C++ program that exercises the C ABI without torch
SOURCES = ["api.hip", "se_fir.hip", "mr_fir.hip", "li_modal.hip", "decode.hip", "featurizer.hip", "fir_cl.hip",
           "fir_cl_direct.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=True, jobs=4):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def compile_one(s):
        o = os.path.join(objdir, s.replace(".hip", ".o"))
        out = _run([HIPCC] + FLAGS + ["-c", os.path.join(CSRC, s), "-o", o])
        if verbose and out.strip():
            print(out)
        return o

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, srcs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    _run([HIPCC] + FLAGS + ["-shared", os.path.join(CSRC, "copy_probe.hip"), "-o", PROBE])
    _run([HIPCC, "-O2", "-std=c++17", os.path.join(CSRC, "abi_selftest.cpp"), "-o", SELFTEST, "-ldl"])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
