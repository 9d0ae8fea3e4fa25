"""Writes tests/golden/ref_cpu_kernels.npz, ref_oc_helper.npz and ref_select_knn.npz:
outputs of the reference's own CPU kernels (compiled from the reference
checkout into oracle/_ref by oracle/build_oracle.py) on small seeded inputs.  Run in the build container,
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


def oc_cases():
    """name -> (association indices, row splits) of the object-condensation helper cases."""
    import torch
    cases = {}
    cases["hand"] = (np.array([3, 7, 3, -1, -1, 3, 7, 1, 1, 0, 0, -1, 1, 1, -1, 3, -1, 19, 3, 2, -1, 19]),
                     np.array([0, 15, 22]))               # tests/test_oc_helper.py:31-37
    torch.manual_seed(42)                                 # tests/test_oc_helper.py:201-210
    a = (torch.randint(0, 100, (1000,), dtype=torch.int64, device="cpu") - 1).numpy()
    cases["stored"] = (a, np.array([0, 250, 500, 1000]))
    rng = np.random.default_rng(4242)
    a = rng.integers(-3, 400, 6000)
    cases["ragged"] = (a, np.array([0, 1, 1, 700, 2500, 2501, 6000]))
    a = rng.integers(0, 60, 3000) * 1234567890123 + 5     # values that need more than 32 bits
    a[rng.random(3000) < 0.2] = -1
    cases["wide_values"] = (a, np.array([0, 1000, 3000]))
    cases["all_negative"] = (np.full(50, -1), np.array([0, 20, 50]))
    cases["single"] = (np.array([7]), np.array([0, 1]))
    cases["one_object"] = (np.full(300, 5), np.array([0, 300]))
    return {k: (np.asarray(v[0], np.int64), np.asarray(v[1], np.int64)) for k, v in cases.items()}


def make_oc():
    out = {}
    for name, (a, rs) in oc_cases().items():
        uv, ur, gmax, lengths, max_len, nobj = O.oc_helper_inputs(a, rs, True)
        M, M_not = O.oc_calc_m(a, uv, ur, rs, gmax, max_len, True, use_ref=True)
        out[name + "/asso"] = a
        out[name + "/row_splits"] = rs
        out[name + "/unique_idx"] = uv
        out[name + "/unique_rs"] = ur
        out[name + "/M"] = M
        out[name + "/M_not"] = M_not.astype(np.int32)
        for flt in (True, False):
            mx, g, no = O.max_same_valued_entries_per_row_split(a, rs, flt, use_ref=True)
            tag = "/filter" if flt else "/nofilter"
            out[name + tag + "_max_per_split"] = mx
            out[name + tag + "_global_max"] = np.int64(g)
            out[name + tag + "_objects_per_split"] = no
    np.savez_compressed(os.path.join(HERE, "ref_oc_helper.npz"), **out)
    print("wrote", os.path.join(HERE, "ref_oc_helper.npz"))


def make_select_knn():
    out = {}
    rng = np.random.default_rng(777)
    for name, n, D, K, rs, radius in (("u3", 1500, 3, 12, [0, 600, 1500], 0.08), ("u3_nolimit", 700, 3, 9, [0, 700], -1.0),
                                      ("u5", 1200, 5, 20, [0, 5, 5, 1200], 0.35), ("tiny", 6, 2, 8, [0, 6], 0.5)):
        c = rng.random((n, D)).astype(np.float32)
        idx, dist = O.select_knn(K, c, np.array(rs), radius, use_ref=True)
        out[name + "/coords"] = c
        out[name + "/row_splits"] = np.array(rs, dtype=np.int64)
        out[name + "/K"] = np.int64(K)
        out[name + "/max_radius"] = np.float64(radius)
        out[name + "/idx"] = idx.astype(np.int32)
        out[name + "/distsq"] = dist
    np.savez_compressed(os.path.join(HERE, "ref_select_knn.npz"), **out)
    print("wrote", os.path.join(HERE, "ref_select_knn.npz"))


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
    make_oc()
    make_select_knn()


if __name__ == "__main__":
    main()
