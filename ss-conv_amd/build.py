"""Builds libssc.so (the gfx950 kernels behind include/ssc.h) with hipcc.

Usage: python ss-conv_amd/build.py [--force]
The library is written to ss-conv_amd/lib/libssc.so, next to the sources, so
that it travels with the source tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libssc.so")
SOURCES = ["common.hip", "rulebook.hip", "conv.hip", "conv_epi.hip", "conv_tail.hip",
           "conv_tail_epi.hip", "conv_five.hip", "conv_five_epi.hip", "conv_wide.hip", "conv_wide_epi.hip", "conv_small.hip", "conv_bwd.hip", "combine.hip", "pool.hip", "voxel.hip", "bnact.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 VALU ops are kept off for every device function of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # "#pragma unroll" on loops whose trip count is a template parameter that may be a
    # run-time value in the generic instance
    "-Wno-pass-failed",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _stale():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(ROOT, "include", "ssc.h")]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    """Compile every HIP source for gfx950 and link libssc.so."""
    if not force and not _stale():
        return LIB
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        cmd = [_hipcc()] + FLAGS + os.environ.get("SSC_HIPCC_FLAGS", "").split() + ["-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c",
                                    os.path.join(CSRC, src), "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out = p.communicate()[0].decode()
        if p.returncode != 0:
            failed = True
            sys.stderr.write("hipcc failed on %s:\n%s\n" % (src, out))
        elif verbose and out.strip():
            sys.stderr.write(out)
    if failed:
        raise RuntimeError("building libssc.so failed")
    subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs,
                   check=True)
    for o in objs:
        os.remove(o)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
