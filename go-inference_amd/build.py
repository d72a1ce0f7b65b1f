"""Build libaq_mi355.so (gfx950 only) in-tree with hipcc.

Usage: python go-inference_amd/build.py [--jobs N]
The library lands next to this file as go-inference_amd/libaq_mi355.so.
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libaq_mi355.so")

HIP_SOURCES = ["aq_qmv.hip", "aq_qmv_blk.hip", "aq_qmv_diag.hip", "aq_qmv_tok.hip", "aq_qmv_act.hip", "aq_moe.hip", "aq_qmv_head.hip", "aq_qmm.hip", "aq_qmm_tile.hip", "aq_qmm_half.hip", "aq_qmm_few.hip", "aq_misc.hip", "aq_tile.hip", "aq_gguf.hip", "aq_api.hip"]
CXX_SOURCES = [os.path.join("host", f) for f in ("quant_registry.cc", "quant_weight.cc", "rocm_affine.cc", "safetensors.cc", "host_capi.cc")]

COMMON = ["-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function"]
# packed-fp32 VALU ops are kept off for device code (the host pass does not know the feature and says so)
HIPFLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(jobs=4, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    cc = hipcc()
    tasks = []
    for src in HIP_SOURCES + CXX_SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            raise RuntimeError("missing source " + path)
        obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
        cmd = [cc] + COMMON + (HIPFLAGS if src.endswith(".hip") else ["-x", "c++"]) + ["-I", os.path.join(HERE, "..", "include"), "-I", CSRC, "-c", path, "-o", obj]
        tasks.append((cmd, obj))
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        for out in ex.map(lambda t: run(t[0]), tasks):
            if verbose and out.strip():
                print(out)
    link = [cc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + [t[1] for t in tasks]
    out = run(link)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args()
    print(build(a.jobs, a.verbose))
