"""Build libfdb_hip.so (gfx950) in-tree with hipcc.

    python -m flashdeberta_amd.csrc.build

The shared object lands next to the package (flashdeberta_amd/libfdb_hip.so) so that it
travels with the source tree; nothing is installed outside it.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "libfdb_hip.so")
SOURCES = ["fdb_api.cpp", "fdb_attn.hip", "fdb_near.hip", "fdb_fp8.hip", "fdb_aux.hip", "fdb_bwd.hip", "fdb_chain.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-x", "hip",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile(src):
    obj = os.path.join(HERE, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=True):
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    for _, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    for o in objs:
        os.remove(o)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
