"""Compile libfgc_hip.so for gfx950 with hipcc (no torch headers involved).

    python fastgraphcompute_amd/csrc/build.py

-ffp-contract=off keeps every float operation a single IEEE operation (bin
indices and squared distances are bit-identical to a sequential float32
evaluation); packed-FP32 instruction selection is switched off.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
# (source, object, extra flags): the search kernels are compiled a second time with their statistics counters
SOURCES = [("fgc_binning.hip", "fgc_binning.o", []), ("fgc_knn.hip", "fgc_knn.o", []),
           ("fgc_knn.hip", "fgc_knn_stats.o", ["-DFGC_KNN_STATS"]),
           ("fgc_knn_mfma.hip", "fgc_knn_mfma.o", ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]), ("fgc_ops.hip", "fgc_ops.o", []),
           ("fgc_oc.hip", "fgc_oc.o", []), ("fgc_linear.hip", "fgc_linear.o", []), ("fgc_api.hip", "fgc_api.o", [])]
OUT = os.path.join(os.path.dirname(HERE), "libfgc_hip.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         "-Wno-unknown-warning-option"]


def build(verbose=True, extra=()):
    objs = []
    procs = []
    for src, obj_name, more in SOURCES:
        obj = os.path.join(HERE, obj_name)
        cmd = ["hipcc"] + FLAGS + more + list(extra) + ["-c", os.path.join(HERE, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((subprocess.Popen(cmd), src))
        objs.append(obj)
    for p, src in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on " + src)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    for o in objs:
        os.remove(o)
    return OUT


if __name__ == "__main__":
    build(extra=sys.argv[1:])
    print("built", OUT)
