"""Build recipe of libtwgemm.so (HIP, gfx950 only) and of the C++ perf driver.

    python -m tilesparsity_amd.build            # compile everything in-tree

hipcc cross-compiles for gfx950 without a GPU; the built library sits next to this
file so that it travels with the source tree.
"""
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libtwgemm.so")
PERF_PATH = os.path.join(PKG_DIR, "test_basic_nn")

SOURCES = ["tw_host.cpp", "tw_plan.hip", "tw_gemm.hip", "tw_prune.hip", "tw_cell.hip", "tw_layout.hip", "tw_side.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept off for this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unused-value", "-Wno-unused-result",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass prints a note that it does not know the packed-fp32 feature; drop it
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        sys.stderr.write(out + "\n")


def build_library(verbose=False):
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    cmd = [hipcc()] + HIPCC_FLAGS + ["-shared", "-o", LIB_PATH]
    for s in srcs:
        cmd += ["-x", "hip", s]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    return LIB_PATH


def build_perf_driver(verbose=False):
    src = os.path.join(CSRC, "perf", "test_basic_nn.cpp")
    if not os.path.exists(src):
        return None
    cmd = [hipcc()] + HIPCC_FLAGS + ["-x", "hip", src, "-o", PERF_PATH,
                                     "-L", PKG_DIR, "-ltwgemm", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    return PERF_PATH


def build_all(verbose=False):
    build_library(verbose)
    build_perf_driver(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
