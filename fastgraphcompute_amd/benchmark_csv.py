"""Timing sweep of binned_select_knn in the CSV layout of the reference's published measurements
(graphing/master_data.csv: size,k,dimension,...,fgc_time,...,count; written by
performance/generate_faiss_performance.py:95-135).

    python -m fastgraphcompute_amd.benchmark_csv --out fgc_times.csv --sizes 100000 1000000 --dims 2 3 4 5 --k 40

Data as in the reference's scripts: standard-normal points from numpy's legacy generator seeded with 42 + offset,
one event.  fgc_time is the wall time in milliseconds of the whole call including the final synchronisation
(the reference times exactly that, performance/generate_faiss_performance.py:68-87), here the median of
`--repeat` calls after one warm-up call; count is the number of timed calls."""
import argparse
import csv
import time

import numpy as np
import torch


def time_call(n, dim, k, repeat, seed_offset=0):
    from . import binned_select_knn
    np.random.seed(42 + seed_offset)
    coords = torch.from_numpy(np.random.randn(n, dim).astype(np.float32)).cuda().contiguous()
    rs = torch.tensor([0, n], dtype=torch.int64, device="cuda")
    binned_select_knn(k, coords, rs)
    torch.cuda.synchronize()
    times = []
    for _ in range(repeat):
        t0 = time.time()
        binned_select_knn(k, coords, rs, direction=None, n_bins=None)
        torch.cuda.synchronize()
        times.append((time.time() - t0) * 1e3)
    return float(np.median(times))


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--out", default="fgc_times.csv")
    ap.add_argument("--sizes", type=int, nargs="+", default=[1000, 10000, 100000, 1000000])
    ap.add_argument("--dims", type=int, nargs="+", default=[2, 3, 4, 5, 6])
    ap.add_argument("--k", type=int, nargs="+", default=[40])
    ap.add_argument("--repeat", type=int, default=5)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("benchmark_csv needs a HIP device")
    with open(a.out, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["size", "k", "dimension", "fgc_time", "count"])
        for n in a.sizes:
            for k in a.k:
                for d in a.dims:
                    if not 1 <= k <= 1024:
                        raise SystemExit("benchmark_csv: k must be in 1..1024 (the library's limit), got %d" % k)
                    t = time_call(n, d, k, a.repeat)                 # the K that is written is the K that is timed
                    w.writerow([float(n), float(k), float(d), t, float(a.repeat)])
                    f.flush()
                    print("size %d k %d dimension %d: %.3f ms" % (n, k, d, t), flush=True)


if __name__ == "__main__":
    main()
