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

SOURCES = ["tw_host.cpp", "tw_plan.hip", "tw_gemm.hip", "tw_gemm_bs.hip", "tw_prune.hip", "tw_cell.hip", "tw_layout.hip", "tw_side.hip"]

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


def _compile_object(job):
    src, obj = job
    _run([hipcc()] + HIPCC_FLAGS + ["-c", "-x", "hip", src, "-o", obj])
    return obj


def build_library(verbose=False, force=True):
    """Compiles every source to an object of its own (in parallel) and links them.  With
    force=False a source is recompiled only when it, or a header, is newer than its object."""
    from concurrent.futures import ThreadPoolExecutor
    objdir = os.path.join(PKG_DIR, "build")
    os.makedirs(objdir, exist_ok=True)
    headers = [os.path.join(CSRC, "tw_internal.h"), os.path.join(CSRC, "tw_device.h"),
               os.path.join(ROOT, "include", "twgemm.h"),
               os.path.abspath(__file__)]
    newest_header = max(os.path.getmtime(h) for h in headers)
    jobs, objs = [], []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(objdir, os.path.splitext(s)[0] + ".o")
        objs.append(obj)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_header):
            jobs.append((src, obj))
    if verbose:
        print("compiling: %s" % ", ".join(os.path.basename(j[0]) for j in jobs))
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as pool:
        list(pool.map(_compile_object, jobs))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs)
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


def build_all(verbose=False, force=True):
    build_library(verbose, force)
    build_perf_driver(verbose)


if __name__ == "__main__":
    # `--changed` recompiles only the sources that are newer than their objects
    build_all(verbose=True, force="--changed" not in sys.argv[1:])
