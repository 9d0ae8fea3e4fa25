"""Writes tests/golden/ref_cpu_kernels.npz: outputs of the reference's own CPU
kernels (compiled from the reference checkout into oracle/_ref by
oracle/build_oracle.py) on small seeded inputs.  Run in the build container,
where the reference checkout exists:

    python oracle/build_oracle.py && python tests/golden/make_golden.py

The fixture holds inputs and outputs only (data, no code).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as O  # noqa: E402

CASES = [
    # name, n, D, K, row_splits (as fractions), max_bin_dims, distribution
    ("u3_k16", 2000, 3, 16, [0, 0.6, 1.0], 3, "uniform"),
    ("u2_k5", 1000, 2, 5, [0, 1.0], 2, "uniform"),
    ("u4_k10", 1000, 4, 10, [0, 1.0], 3, "uniform"),
    ("u8_k50", 1500, 8, 50, [0, 0.33, 0.5, 1.0], 3, "uniform"),
    ("blobs3_k24", 2500, 3, 24, [0, 0.5, 1.0], 3, "blobs"),
    ("small_events_k20", 300, 3, 20, None, 3, "uniform"),
    ("d5_bins5_k8", 1200, 5, 8, [0, 1.0], 5, "uniform"),
]


def make_inputs(name, n, D, K, rsf, dist):
    rng = np.random.default_rng(sum(map(ord, name)))
    if dist == "uniform":
        c = rng.random((n, D))
    else:
        centres = rng.random((12, D))
        c = centres[rng.integers(0, 12, n)] + rng.normal(0, 0.02, (n, D))
        c[: n // 5] = rng.random((n // 5, D))
    c = c.astype(np.float32)
    if rsf is None:
        rs = np.array([0, 3, 3, 40, 41, n], dtype=np.int64)
    else:
        rs = np.array([int(round(f * n)) for f in rsf], dtype=np.int64)
    return c, rs


def main():
    if O.ref_lib() is None:
        raise SystemExit("oracle/_ref/libfgc_ref.so missing: run python oracle/build_oracle.py first")
    out = {}
    for name, n, D, K, rsf, mbd, dist in CASES:
        c, rs = make_inputs(name, n, D, K, rsf, dist)
        s = O.sorted_space(c, rs, K, None, mbd)
        norm, bw, nb = O.normalise(np.ascontiguousarray(c[:, :min(mbd, D)]), None, s["n_bins"])
        a, f, nper, _ = O.bin_points(norm, rs, bw, nb, use_ref=True)
        idx_s, dist_s, _, _ = O.knn_sorted(s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"], s["n_bins"],
                                           s["bin_width"], K, use_ref=True)
        idx, dsq = O.binned_select_knn(K, c, rs, max_bin_dims=mbd, use_ref=True)
        gd = np.random.default_rng(99).standard_normal((n, K)).astype(np.float32)   # tests regenerate it
        g = O.knn_grad(gd, idx, c, dsq, use_ref=True)
        out[name + "/coords"] = c
        out[name + "/row_splits"] = rs
        out[name + "/K"] = np.int64(K)
        out[name + "/max_bin_dims"] = np.int64(mbd)
        out[name + "/assigned"] = a.astype(np.int16)
        out[name + "/flat"] = f.astype(np.int32)
        out[name + "/n_per_bin"] = nper.astype(np.int32)
        out[name + "/bin_width"] = bw
        out[name + "/n_bins"] = nb
        out[name + "/idx_sorted_space"] = idx_s.astype(np.int32)
        out[name + "/dist_sorted_space"] = dist_s
        out[name + "/idx"] = idx.astype(np.int32)
        out[name + "/distsq"] = dsq
        out[name + "/grad_coords"] = g
    np.savez_compressed(os.path.join(HERE, "ref_cpu_kernels.npz"), **out)
    print("wrote", os.path.join(HERE, "ref_cpu_kernels.npz"))


if __name__ == "__main__":
    main()
