"""Build the CPU checker libraries (test infrastructure, never the product).

  libfgc_oracle.so        the plain-C restatement in oracle/fgc_oracle.c
  _ref/libfgc_ref.so      the reference's own CPU kernels, compiled from the
                          sources where they lie in the reference checkout,
                          plus oracle/ref_driver.cpp (a C-ABI driver, no
                          stand-ins).  Only built where the checkout exists.

Usage: python oracle/build_oracle.py [--ref-root /root/reference] [--no-ref]
"""
import argparse
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REF_TUS = [
    "bin_by_coordinates_cpu.cpp",
    "binned_select_knn_cpu.cpp",
    "binned_select_knn_grad_cpu.cpp",
    "index_replacer_cpu.cpp",
    "oc_helper_cpu.cpp",
    "oc_helper_helper.cpp",
    "select_knn_cpu.cpp",
]


def build_oracle(verbose=True):
    out = os.path.join(HERE, "libfgc_oracle.so")
    cmd = ["gcc", "-O2", "-std=c11", "-ffp-contract=off", "-fopenmp", "-shared",
           "-fPIC", "-o", out, os.path.join(HERE, "fgc_oracle.c"), "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


def build_ref(ref_root, verbose=True):
    """Compile the reference's CPU kernel translation units (they need
    only the installed libtorch headers) and link them with ref_driver.cpp."""
    src_dir = os.path.join(ref_root, "fastgraphcompute", "extensions")
    if not os.path.isdir(src_dir):
        return None
    import torch
    from torch.utils.cpp_extension import include_paths
    out_dir = os.path.join(HERE, "_ref")
    os.makedirs(out_dir, exist_ok=True)
    incs = []
    for p in include_paths():
        incs += ["-I", p]
    import sysconfig
    incs += ["-I", sysconfig.get_paths()["include"]]
    abi = "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    objs = []
    procs = []
    for tu in REF_TUS + ["ref_driver.cpp"]:
        src = os.path.join(HERE if tu == "ref_driver.cpp" else src_dir, tu)
        obj = os.path.join(out_dir, tu.replace(".cpp", ".o"))
        cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-w", abi] + incs + ["-I", src_dir, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append(subprocess.Popen(cmd))
        objs.append(obj)
    for p in procs:
        if p.wait() != 0:
            raise RuntimeError("reference CPU kernel compile failed")
    out = os.path.join(out_dir, "libfgc_ref.so")
    cmd = ["g++", "-shared", "-o", out] + objs + ["-L", tlib, "-ltorch", "-ltorch_cpu", "-lc10",
                                                   "-Wl,-rpath," + tlib]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    for o in objs:
        os.remove(o)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref-root", default="/root/reference")
    ap.add_argument("--no-ref", action="store_true")
    a = ap.parse_args()
    build_oracle()
    if not a.no_ref:
        r = build_ref(a.ref_root)
        print("reference CPU kernels:", r if r else "checkout not present, skipped")
    sys.exit(0)
