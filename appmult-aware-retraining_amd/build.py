"""Builds libamr_lutgemm.so (HIP, gfx950) next to this file.

    python appmult-aware-retraining_amd/build.py [--force]

hipcc cross-compiles for gfx950 without a GPU.  The library is built in-tree; it is git-ignored but
travels with the source tree to the GPU box.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libamr_lutgemm.so")
SOURCES = ["lutgemm_fwd.hip", "lutgemm_fwd_slab.hip", "lutgemm_bwd.hip", "lutgemm_bwd_f32tab.hip", "lutgemm_bwd_slab.hip", "lutgemm_bwd_slab8.hip", "lutgemm_gradA_slab.hip", "lutgemm_gradA_rows8.hip", "accgemm.hip", "im2col.hip", "quantize.hip", "fill.hip", "dequant.hip", "conv_glue.hip", "lds_probe.hip", "capi.hip"]
HEADERS = [os.path.join(CSRC, "amr_common.h"), os.path.join(HERE, "..", "include", "amr_lutgemm.h")]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-Wall",
         # packed-fp32 VALU forms are switched off for every device translation unit
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{msgs}")
    return obj, msgs


def up_to_date():
    if not os.path.exists(LIB):
        return False
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, s) for s in SOURCES] + HEADERS
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force=True, verbose=True):
    if not force and up_to_date():
        return LIB
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        results = list(ex.map(_compile, SOURCES))
    for _, msgs in results:
        if msgs and verbose:
            print(msgs)
    objs = [o for o, _ in results]
    r = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force=True)
