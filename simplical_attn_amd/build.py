"""Builds the HIP library in-tree with hipcc for gfx950.

    python -m simplical_attn_amd.build        # compile every source, link libsa2_hip.so

One object per .hip file (compiled in parallel), linked into
simplical_attn_amd/lib/libsa2_hip.so.  Cross-compiles without a GPU.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libsa2_hip.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-fp32 VALU forms are switched off for the device pass; the host pass
# does not know the feature and says so, which is harmless.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def _compile(src, extra):
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    return obj, err


def build_library(verbose=True, extra_flags=()):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        results = list(ex.map(lambda s: _compile(s, list(extra_flags)), sources))
    for (obj, err), src in zip(results, sources):
        if verbose and err.strip():
            print("[%s]\n%s" % (os.path.basename(src), err), file=sys.stderr)
    objs = [o for o, _ in results]
    tmp = LIB_PATH + ".tmp"
    res = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(extra_flags=sys.argv[1:]))
