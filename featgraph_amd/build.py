"""Builds libfeatgraph_hip.so for gfx950 with hipcc, in-tree.

    python -m featgraph_amd.build            # compile every source and link

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libfeatgraph_hip.so")

SOURCES = ["fg_host.cpp", "fg_plan.hip", "fg_spmm.hip", "fg_sddmm.hip", "fg_softmax.hip", "fg_attention.hip", "fg_attention_bwd.hip", "fg_general.hip"]

# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 instructions.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=fast",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wno-unused-function"]
# The broadcasting operators promise separately rounded messages and sums (exact max / min and selected
# positions, sums in stored order): no fused multiply-add in that file.
EXTRA_FLAGS = {"fg_general.hip": ["-ffp-contract=off"]}


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; libfeatgraph_hip.so cannot be built")


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + HIP_FLAGS + EXTRA_FLAGS.get(src, []) + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, obj, res.returncode, res.stdout


def build(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = []
    for src, obj, rc, out in results:
        noise = "is not a recognized feature for this target"   # host pass does not know -packed-fp32-ops
        text = "\n".join(l for l in out.splitlines() if noise not in l and l.strip())
        if rc != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and text:
            print(text)
        objs.append(obj)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs + ["-lpthread"]
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
