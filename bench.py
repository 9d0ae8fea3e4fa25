#!/usr/bin/env python3
"""Benchmark of the graph-building hot path on one MI355X.

One step = one pass of the path over the headline workload (N = 1 000 000
points, D = 3, K = 64, one event of Zipf-sized Gaussian blobs + 20 % noise):
the whole `binned_select_knn` forward call (binning, sort, search, un-sort)
followed by its gradient for an upstream dL/d(distsq) ~ N(0,1).  Inputs are
resident in HBM before the timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4]
                    [--no-cpu-baseline]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published peak
N_SIMD = 1024           # 256 compute units x 4 SIMDs; a VALU wavefront instruction occupies its SIMD for 4 cycles
GPU_CLOCK_HZ = 2.4e9    # MI355X peak engine clock (published); used only to turn instruction counts into a time share


def kernel_source_hash():
    """First 12 hex digits of the SHA-256 over the library's HIP sources and headers (names and contents, in name
    order): the `src=` field of a `#bench-fact` line says which sources the profiled library was built from."""
    import hashlib
    cdir = os.path.join(ROOT, "fastgraphcompute_amd", "csrc")
    h = hashlib.sha256()
    try:
        names = sorted(n for n in os.listdir(cdir) if n.endswith((".hip", ".h")))
        for n in names + ["../../include/fgc_hip.h"]:
            with open(os.path.join(cdir, n), "rb") as fh:
                h.update(os.path.basename(n).encode() + b"\0" + fh.read() + b"\0")
    except OSError:
        return None
    return h.hexdigest()[:12]


def profile_facts():
    """Per-kernel figures that only a profiler run gives (HBM bytes per launch from FETCH_SIZE / WRITE_SIZE,
    VALU wavefront instructions per launch), read from the `#bench-fact` lines of the committed rocprofv3 summaries
    under profiles/: {(kernel, workload): {key: value, "files": names, "src": source hashes}}.  Both are properties
    of the kernel and the input, not of the run, so they are combined here with the kernel time measured live - as
    long as the kernel is the one that was profiled: a line whose `src=` differs from the hash of the sources in this
    tree is reported as stale (`profile_stale` in the roofline object)."""
    facts = {}
    pdir = os.path.join(ROOT, "profiles")
    if not os.path.isdir(pdir):
        return facts
    for name in sorted(os.listdir(pdir)):
        if not name.endswith(".txt"):
            continue
        with open(os.path.join(pdir, name)) as fh:
            for line in fh:
                if not line.startswith("#bench-fact"):
                    continue
                kv = dict(tok.split("=", 1) for tok in line.split()[1:] if "=" in tok)
                key = (kv.pop("kernel", ""), kv.pop("workload", ""))
                ent = facts.setdefault(key, {"files": [], "src": set()})
                ent["src"].add(kv.pop("src", None))
                for k, v in kv.items():
                    ent[k] = float(v)
                ent["files"].append("profiles/" + name)
    return facts


def roofline_entry(kernel, workload, alg_bytes, kernel_ms, clock_hz, useful_valu_insts=None, facts=None):
    """The roofline object of one kernel: `achieved` / `frac` on ALGORITHMIC bytes (what a kernel without reuse
    would have to move), and beside them what the hardware counters say: physical HBM traffic and its share of the
    peak, and the share of the kernel's duration its SIMDs spend issuing VALU instructions."""
    achieved = alg_bytes / (kernel_ms * 1e-3) / 1e9
    r = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
         "frac": round(achieved / HBM_PEAK_GBS, 4),
         "frac_kind": "effective: algorithmic bytes / measured kernel time (reads served from registers, LDS and L2 "
                      "count as if they came from memory; it can exceed the physical share, and 1)",
         "algorithmic_bytes": alg_bytes, "kernel_ms": round(kernel_ms, 4), "traffic": None, "physical_gbs": None,
         "physical_frac": None, "valu_issue_frac": None, "useful_valu_frac": None, "profile": None}
    f = (facts or {}).get((kernel, workload))
    if f:
        r["profile"] = sorted(set(f["files"]))
        # counters taken from a library built from other sources than the ones in this tree describe another kernel
        r["profile_stale"] = f["src"] != {kernel_source_hash()}
        if "traffic_bytes" in f:
            r["traffic"] = f["traffic_bytes"]
            r["physical_gbs"] = round(f["traffic_bytes"] / (kernel_ms * 1e-3) / 1e9, 1)
            r["physical_frac"] = round(r["physical_gbs"] / HBM_PEAK_GBS, 4)
        if "valu_wave_insts" in f:
            r["valu_issue_frac"] = round(f["valu_wave_insts"] * 4.0 / (N_SIMD * kernel_ms * 1e-3 * clock_hz), 4)
            if useful_valu_insts is not None:
                r["useful_valu_frac"] = round(useful_valu_insts / f["valu_wave_insts"], 4)
            r["binding_resource"] = "valu_issue" if r["valu_issue_frac"] >= 0.6 else "latency / atomic-update rate"
    return r


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg4", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "oc_helper", "gravnet_model"])
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the short GravNetOp / model-step measurements appended to the default line")
    ap.add_argument("--cpu-sample-seconds", type=float, default=15.0)
    ap.add_argument("--cpu-reference-full", action="store_true",
                    help="also time the reference's own compiled CPU kernel (oracle/_ref) on ALL queries of the "
                         "workload, one core; minutes at the default workload")
    ap.add_argument("--matrix-search", default="auto", choices=["auto", "off", "always"],
                    help="config.matrix_search: let the library decide whether a search with 5 to 8 coordinates screens "
                         "its candidates on the matrix cores (auto), never, or wherever that search can run")
    ap.add_argument("--sorted-neighbours", action="store_true",
                    help="ask for neighbour rows by increasing distance (config.sorted_neighbours) instead of the "
                         "default, rows in the order the search found them, as the reference returns them")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no multi-GPU part); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import fastgraphcompute_amd as fgc
    from fastgraphcompute_amd import _lib, config, workloads
    from fastgraphcompute_amd.extensions.binned_select_knn import (binned_select_knn_grad,
                                                                   calculate_optimal_bins)
    from fastgraphcompute_amd._ops import choose_search_grid, knn_grad_sorted

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = _lib.lib()
    config.sorted_neighbours = bool(args.sorted_neighbours)
    config.matrix_search = {"auto": True, "off": False, "always": "always"}[args.matrix_search]

    if args.workload == "oc_helper":
        print(json.dumps(oc_helper_workload(args, dev)), flush=True)
        return
    if args.workload == "gravnet_model":
        print(json.dumps(gravnet_model_workload(args, dev)), flush=True)
        return
    w = workloads.CONFIGS[args.workload](args.scale)
    if args.workload == "cfg3":
        print(json.dumps(gravnet_workload(args, w, dev)), flush=True)
        return
    K = int(w["K"])
    coords_h = w["coords"]
    n, D = coords_h.shape
    coords = torch.from_numpy(coords_h).to(dev)
    rs = torch.from_numpy(w["row_splits"]).to(dev).to(torch.int64)
    gd_h = w.get("grad_distsq")
    if gd_h is None:
        gd_h = np.random.default_rng(2000).standard_normal((n, K)).astype(np.float32)
    grad_d = torch.from_numpy(gd_h).to(dev)
    config.sync_checks = True

    coords_g = coords.clone().requires_grad_(True)

    def step():
        # the user-visible path: forward through the autograd op, backward with the upstream gradient
        idx, dist = fgc.binned_select_knn(K, coords_g, rs)
        coords_g.grad = None
        dist.backward(grad_d)
        return idx, dist, coords_g.grad

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    t_step = (time.perf_counter() - t0) / args.steps
    del out

    # ---- stage timings with events on the launch stream (torch's current stream) ----
    rs_host = rs.cpu()
    if config.auto_grid:                       # the grid binned_select_knn itself picks when n_bins is None
        nbd, nb1 = choose_search_grid(rs_host, D, 3)
        nb = [nb1] * nbd
    else:
        nbd = min(3, D)
        nb = [calculate_optimal_bins(rs_host, K, nbd)] * nbd
    nb_arr, rs_arr = _lib.host_i64(nb), _lib.host_i64(rs_host.tolist())
    n_rs = rs_host.numel()
    ws_bytes = L.fgc_binned_select_knn_workspace_bytes(n, D, nbd, nb_arr, n_rs, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    status = torch.zeros(4, dtype=torch.int32, device=dev)
    stats = torch.zeros(8, dtype=torch.int64, device=dev)
    idx = torch.empty((n, K), dtype=torch.int64, device=dev)
    dist = torch.empty((n, K), dtype=torch.float32, device=dev)
    nbr_sorted = torch.empty((n, K), dtype=torch.int32, device=dev)   # as the autograd path requests it
    st = _lib.stream_ptr()
    knn_flags = 0 if config.sorted_neighbours else _lib.KNN_ANY_ORDER     # the row order binned_select_knn asks for
    knn_flags |= {"auto": 0, "off": _lib.KNN_NO_MATRIX, "always": _lib.KNN_FORCE_MATRIX}[args.matrix_search]

    def prepare():
        _lib.check(L.fgc_binned_knn_prepare_f32(_lib.ptr(coords), n, D, _lib.ptr(rs), rs_arr, n_rs, K, nbd, nb_arr,
                                                None, _lib.ptr(status), _lib.ptr(ws), ws_bytes, st))

    def search(with_stats):
        _lib.check(L.fgc_binned_knn_search_f32(n, D, rs_arr, n_rs, K, nbd, nb_arr, 0, knn_flags, _lib.ptr(idx), _lib.ptr(dist),
                                               _lib.ptr(nbr_sorted),
                                               _lib.ptr(stats) if with_stats else None, _lib.ptr(ws), ws_bytes, st))

    def timed(fn, reps):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return [a.elapsed_time(b) for a, b in ev]

    prepare()
    search(True)
    torch.cuda.synchronize()
    c_eval = int(stats[0].item())
    chunks = int(stats[1].item())
    inserts = int(stats[2].item())
    handed_over, collected = int(stats[3].item()), int(stats[5].item())
    matrix = collected > 0          # the search ran on the matrix cores (k_knn_mf); k_knn only took what it handed over
    reps = max(3, args.steps)
    t_prep = float(np.mean(timed(prepare, reps)))
    t_knn = float(np.mean(timed(lambda: search(False), reps)))
    order = torch.empty(n, dtype=torch.int32, device=dev)
    _lib.check(L.fgc_binned_knn_export_order_i32(n, D, rs_arr, n_rs, K, nbd, nb_arr, 0, _lib.ptr(ws), ws_bytes,
                                                 _lib.ptr(order), st))
    t_grad = float(np.mean(timed(lambda: knn_grad_sorted(grad_d, nbr_sorted, coords, order), reps)))

    # algorithmic bytes of one search launch: every distance evaluation reads one
    # D-float candidate, every query is read once, every (idx, distsq) slot written once
    facts = profile_facts() if args.scale == 1.0 else {}
    clock_hz = GPU_CLOCK_HZ
    # (the matrix-core search screens pairs in float16 and evaluates exact distances only for the candidates it collects:
    # those are its distance evaluations; the screened pairs are reported separately)
    n_exact = collected if matrix else c_eval
    bytes_alg = 4.0 * D * n_exact + 4.0 * D * n + 12.0 * K * n
    # VALU wavefront instructions that are distance arithmetic: per 64 evaluations D subtractions (the query's
    # coordinates are scalar operands), D multiplications, D - 1 additions and the compare
    roofline = roofline_entry("k_knn_mf" if matrix else "k_knn", w["name"], bytes_alg, t_knn, clock_hz,
                              None if matrix else (c_eval / 64.0) * (3 * D), facts)
    if matrix:
        # one v_mfma_f32_32x32x16_f16 per 32 x 32 pairs: 32 flops per evaluated pair, against the dense float16 peak
        roofline["screened_pairs"] = c_eval
        roofline["binding_resource"] = "valu_issue (histogram and collection of the screened pairs)"
        roofline["matrix_core"] = {"mfma_tflops": round(32.0 * c_eval / (t_knn * 1e-3) / 1e12, 1), "peak_tflops": 2500.0,
                                   "frac": round(32.0 * c_eval / (t_knn * 1e-3) / 1e12 / 2500.0, 4),
                                   "candidates_collected_per_query": round(collected / max(1, n - handed_over), 1),
                                   "queries_handed_to_the_vector_search": handed_over}
    achieved = roofline["achieved"]
    roofline["distance_evaluations"] = n_exact
    # inputs + outputs of the timed launch: queries, int64 indices, distances, int32 sorted-space rows
    roofline["io_floor_bytes"] = 4.0 * D * n + 16.0 * K * n
    # gradient kernel: upstream gradient + neighbour rows + one D-float gather per pair + coordinates in, gradient out
    grad_alg = 4.0 * K * n + 8.0 * K * n + 4.0 * D * n * K + 8.0 * D * n
    roofline_grad = roofline_entry("k_knn_grad_sorted", w["name"], grad_alg, t_grad, clock_hz, None, facts)
    roofline_grad["kernel_ms_includes"] = "k_sorted_points, k_knn_grad_sorted, k_unsort_grad (one library call)"
    if roofline_grad["traffic"] is not None:       # the two small kernels of the same call move bytes too
        extra = sum(facts.get((k, w["name"]), {}).get("traffic_bytes", 0.0) for k in ("k_sorted_points", "k_unsort_grad"))
        roofline_grad["traffic"] += extra
        roofline_grad["physical_gbs"] = round(roofline_grad["traffic"] / (t_grad * 1e-3) / 1e9, 1)
        roofline_grad["physical_frac"] = round(roofline_grad["physical_gbs"] / HBM_PEAK_GBS, 4)
    # what a plain device-to-device copy reaches on this box (1 GiB read + 1 GiB written), for orientation
    del idx, dist, nbr_sorted
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    t_copy = float(np.median(timed(lambda: dst.copy_(src), 7)[2:]))
    roofline["copy_gbs"] = round(2.0 * src.numel() * 4 / (t_copy * 1e-3) / 1e9, 1)
    roofline["frac_of_copy"] = round(achieved / roofline["copy_gbs"], 4)
    del src, dst

    result = {
        "metric": ("kNN queries/sec and neighbours/sec at N=1M,D=3,K=64; % of HBM roofline"
                   if (args.workload == "cfg4" and args.scale == 1.0) else
                   "kNN queries/sec and neighbours/sec at N=%d,D=%d,K=%d; %% of HBM roofline" % (n, D, K)),
        "value": round(n / t_step, 1), "unit": "queries/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(t_step * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": w["name"], "n_points": n, "n_coords": D, "K": K, "events": int(n_rs - 1),
                   "n_bins": nb, "step": "binned_select_knn forward (whole call) + gradient",
                   "row_order": "by distance" if config.sorted_neighbours else "any (as the reference)",
                   "search_kernel": "k_knn_mf (candidates screened on the matrix cores)" if matrix else "k_knn"},
        "neighbours_per_s": round(n * K / t_step, 1),
        "forward_call_ms": round(t_prep + t_knn, 4),
        "forward_queries_per_s": round(n / ((t_prep + t_knn) * 1e-3), 1),
        "stages_ms": {"bin_sort_gather": round(t_prep, 4), "knn_search": round(t_knn, 4),
                      "gradient": round(t_grad, 4)},
        "search_counters": {"distance_evaluations": c_eval, "candidate_chunks": chunks, "pool_prunes": inserts},
        "roofline": roofline,
        "roofline_gradient": roofline_grad,
    }

    if not args.no_cpu_baseline:
        result["cpu_baseline"], result["cpu_baseline_allcores"] = cpu_baseline(w, K, n, args.cpu_sample_seconds)
    if args.cpu_reference_full:
        result["cpu_baseline_reference_full"] = cpu_reference_full(w, K, n)
    if args.workload == "cfg4" and args.scale == 1.0 and not args.no_secondary:
        # the steps either side of the path, a few iterations each: the GravNetOp layer at the cfg3 shape and the
        # training step of the reference's 4-layer model benchmark
        del coords, coords_g, grad_d, ws
        torch.cuda.empty_cache()
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup = 5, 2
        g = gravnet_workload(sub, workloads.CONFIGS["cfg3"](1.0), dev)
        m = gravnet_model_workload(sub, dev)
        result["secondary"] = {
            "cfg3_gravnet_op_ms_per_step": g["ms_per_step"], "cfg3_stages_ms": g["stages_ms"],
            "cfg3_roofline_aggregate_bwd": {k: g["roofline"][k] for k in ("achieved", "frac", "kernel_ms")},
            "gravnet_model_ms_per_step": m["ms_per_step"],
            "gravnet_model_ms_per_step_with_use_dense_layers": m["ms_per_step_with_use_dense_layers"]}
    print(json.dumps(result), flush=True)


def gravnet_workload(args, w, dev):
    """Secondary workload: one GravNetOp forward + backward (N = 300 000 x 64 features, S=4, P=32, k=40)."""
    import torch
    from fastgraphcompute_amd.gnn_ops import GravNetOp
    torch.manual_seed(w["weight_seed"])
    op = GravNetOp(w["in_channels"], w["out_channels"], w["space_dimensions"], w["propagate_dimensions"],
                   w["K"]).to(dev)
    x = torch.from_numpy(w["x"]).to(dev).requires_grad_(True)
    rs = torch.from_numpy(w["row_splits"]).to(dev)
    g = torch.from_numpy(w["out_grad"]).to(dev)

    def step():
        x.grad = None
        op.zero_grad(set_to_none=True)
        out = op(x, rs)[0]
        out.backward(g)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / args.steps
    n = w["x"].shape[0]
    result = {
        "metric": "GravNetOp forward+backward points/sec", "value": round(n / t, 1), "unit": "points/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(t * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": w["name"], "n_points": n, "events": 2}}
    result.update(gravnet_stage_times(op, x, rs, w, dev))
    return result


def gravnet_stage_times(op, x, rs, w, dev):
    """The two aggregation kernels of the layer on their own (events on the launch stream, through the C ABI) and
    the roofline entry of the backward one, the largest kernel of the step."""
    import ctypes
    import numpy as np
    import torch
    from fastgraphcompute_amd import _lib
    L = _lib.lib()
    with torch.no_grad():
        space = op.space_transformations(x).contiguous()
        feat = op.propagate_transformations(x).contiguous()
    from fastgraphcompute_amd import _ops
    idx, dist, nbr_sorted, order = _ops._knn_forward(space, space.shape[1], rs, int(w["K"]), None, None, 3, False, True)
    n, K = idx.shape
    P = feat.shape[1]
    agg = torch.empty((n, 2 * P), device=dev)
    am = torch.empty((n, P), dtype=torch.int32, device=dev)
    g_agg = torch.randn((n, 2 * P), device=dev)
    g_feat = torch.zeros((n, P), device=dev)
    g_dsq = torch.empty((n, K), device=dev)
    st = _lib.stream_ptr()

    def fwd():
        _lib.check(L.fgc_gravnet_aggregate_fwd_ld_f32(_lib.ptr(idx), _lib.ptr(dist), _lib.ptr(feat), P, n, _lib.ptr(agg),
                                                      ctypes.c_void_p(agg.data_ptr() + 4 * P), 2 * P, _lib.ptr(am), n,
                                                      K, P, None, st))

    def bwd_pairs():     # one atomic row update per (point, slot) pair: the stand-alone op's kernel
        _lib.check(L.fgc_gravnet_aggregate_bwd_ld_f32(_lib.ptr(idx), _lib.ptr(dist), _lib.ptr(feat), P, n, _lib.ptr(am),
                                                      _lib.ptr(g_agg), ctypes.c_void_p(g_agg.data_ptr() + 4 * P),
                                                      2 * P, _lib.ptr(g_feat), P, _lib.ptr(g_dsq), n, K, P, None, st))

    def bwd():           # what GravNetOp's backward runs: rows of a sorted tile combined on chip
        _lib.check(L.fgc_gravnet_aggregate_bwd_sorted_f32(_lib.ptr(nbr_sorted), _lib.ptr(order), _lib.ptr(dist),
                                                          _lib.ptr(feat), P, _lib.ptr(am), _lib.ptr(g_agg),
                                                          ctypes.c_void_p(g_agg.data_ptr() + 4 * P), 2 * P,
                                                          _lib.ptr(g_feat), P, _lib.ptr(g_dsq), n, K, P, None, st))

    def timed(fn, reps=8):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return float(np.median([a.elapsed_time(b) for a, b in ev][2:]))

    fwd()                # the backward kernels read the arg-max slots the forward writes
    tiled = K <= 64 and 8 < P <= 64
    t_fwd, t_bwd_pairs = timed(fwd), timed(bwd_pairs)
    t_bwd = timed(bwd) if tiled else t_bwd_pairs
    clock_hz = GPU_CLOCK_HZ
    facts = profile_facts()
    # index + distance rows, one P-float gather per pair, features / outputs once; the backward gathers and scatters
    fwd_alg = 12.0 * K * n + 4.0 * P * n * K + 8.0 * P * n
    bwd_alg = fwd_alg + 4.0 * P * n * K
    return {"stages_ms": {"aggregate_fwd": round(t_fwd, 4), "aggregate_bwd": round(t_bwd, 4),
                          "aggregate_bwd_per_pair_kernel": round(t_bwd_pairs, 4)},
            "roofline": roofline_entry("k_gravnet_bwd_tile" if tiled else "k_gravnet_bwd", w["name"], bwd_alg, t_bwd,
                                       clock_hz, None, facts),
            "roofline_aggregate_fwd": roofline_entry("k_gravnet_fwd", w["name"], fwd_alg, t_fwd, clock_hz, None, facts)}


def gravnet_model_workload(args, dev):
    """Secondary workload: the training step of the reference's model benchmark (performance/gravnet_perfm.py:
    20-96,110-163): two dense layers, 4 x (GravNetOp(k=64, S=4, P=32) + three dense layers), two dense layers;
    hidden 128, 200 000 nodes in one event, loss = sum(output) * 0, SGD step."""
    import torch
    import torch.nn as nn
    from fastgraphcompute_amd.gnn_ops import GravNetOp

    in_dim, prop_dim, space_dim, k, hidden, out_dim, layers = 64, 32, 4, 64, 128, 10, 4

    class GravNetModel(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = nn.Linear(in_dim, hidden)
            self.fc2 = nn.Linear(hidden, hidden)
            self.gravnet_layers = nn.ModuleList(
                GravNetOp(hidden if i == 0 else 2 * prop_dim, 2 * prop_dim, space_dim, prop_dim, k)
                for i in range(layers))
            self.dense_after_gravnet = nn.ModuleList(
                nn.Sequential(nn.Linear(2 * prop_dim, hidden), nn.ReLU(), nn.Linear(hidden, hidden), nn.ReLU(),
                              nn.Linear(hidden, 2 * prop_dim), nn.ReLU()) for _ in range(layers))
            self.fc3 = nn.Linear(2 * prop_dim, hidden)
            self.fc4 = nn.Linear(hidden, out_dim)

        def forward(self, x, row_splits):
            x = torch.relu(self.fc2(torch.relu(self.fc1(x))))
            for g, d in zip(self.gravnet_layers, self.dense_after_gravnet):
                x = d(g(x, row_splits)[0])
            return self.fc4(torch.relu(self.fc3(x)))

    n = int(round(200000 * args.scale))
    torch.manual_seed(1007)
    model = GravNetModel().to(dev)
    opt = torch.optim.SGD(model.parameters(), lr=0.01)
    x = torch.randn(n, in_dim, device=dev)
    rs = torch.tensor([0, n], dtype=torch.int64, device=dev)

    def step():
        opt.zero_grad(set_to_none=True)
        out = model(x, rs)
        (out.sum() * 0.0).backward()
        opt.step()

    def timed_steps():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    t = timed_steps()                      # the model as the reference defines it: torch.nn.Linear layers
    from fastgraphcompute_amd.gnn_ops import use_dense_layers
    use_dense_layers(model)                # same parameters, weight gradients by the library's kernel
    t_dense = timed_steps()
    return {
        "metric": "GravNet model training step nodes/sec", "value": round(n / t, 1), "unit": "nodes/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(t * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "gravnet_model_4layers_h128_k64", "n_points": n, "events": 1},
        "ms_per_step_with_use_dense_layers": round(t_dense * 1e3, 4)}


def oc_helper_workload(args, dev):
    """Secondary workload: oc_helper_matrices on 200 000 vertices in 4 events with 500 objects each (M_not is
    [2000, 50000] int64 = 800 MB).  The roofline entry is the M_not kernel's HBM write stream."""
    import numpy as np
    import torch
    import fastgraphcompute_amd as fgc
    from fastgraphcompute_amd import _lib, workloads
    L = _lib.lib()
    a_h, rs_h = workloads.oc_workload(args.scale)
    a = torch.from_numpy(a_h).to(dev)
    rs = torch.from_numpy(rs_h).to(dev)

    def step():
        return fgc.oc_helper_matrices(a, rs)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        M, M_not, _n = step()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / args.steps

    # the two library calls on their own, timed with events on the stream they are enqueued on
    n, n_rs = a.numel(), rs.numel()
    ws_bytes = L.fgc_oc_helper_workspace_bytes(n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    summary = torch.empty(4, dtype=torch.int64, device=dev)
    mx = torch.empty(n_rs - 1, dtype=torch.int64, device=dev)
    no = torch.empty_like(mx)
    U, W, R = M.shape[0], M.shape[1], M_not.shape[1]

    def objects():
        _lib.check(L.fgc_oc_helper_objects_i64(_lib.ptr(a), n, _lib.ptr(rs), n_rs, 1, 0, _lib.ptr(mx), _lib.ptr(no),
                                               _lib.ptr(summary), _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))

    def fill(m, m_not):
        _lib.check(L.fgc_oc_helper_fill_i64(n, _lib.ptr(rs), n_rs, U, W, R, None, None, _lib.ptr(summary),
                                            _lib.ptr(M) if m else None, _lib.ptr(M_not) if m_not else None, None,
                                            None, None, _lib.ptr(ws), ws_bytes, _lib.stream_ptr()))

    def timed(fn, reps=20):
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e-3

    t_obj = timed(objects)
    t_m = timed(lambda: fill(True, False))
    t_not = timed(lambda: fill(False, True))
    bytes_not = 8.0 * U * R + 4.0 * n                # every int64 written once + one read of the object ids
    result = {
        "metric": "oc_helper_matrices vertices/sec", "value": round(n / t, 1), "unit": "vertices/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(t * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": "oc_helper_200k_4events_500objects", "n_vertices": n, "events": int(n_rs - 1),
                   "n_objects": int(U), "M_columns": int(W), "M_not_columns": int(R)},
        "stages_ms": {"objects": round(t_obj * 1e3, 4), "fill_M": round(t_m * 1e3, 4),
                      "fill_M_not": round(t_not * 1e3, 4)},
        "roofline": {"bound": "hbm", "achieved": round(bytes_not / t_not / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                     "frac": round(bytes_not / t_not / 8e12, 4), "traffic": None, "kernel": "k_oc_fill_m_not"},
    }
    if not args.no_cpu_baseline:
        from oracle import oracle as O
        uv, ur, gmax, _l, max_len, _nobj = O.oc_helper_inputs(a_h, rs_h, True)
        sel = np.arange(uv.size)
        O.oc_calc_m(a_h, uv[:8], ur[:8], rs_h, gmax, max_len, True)     # page in the library
        t0 = time.perf_counter()
        for _ in range(3):
            O.oc_calc_m(a_h, uv, ur, rs_h, gmax, max_len, True)
        tc = (time.perf_counter() - t0) / 3
        result["cpu_baseline"] = {"value": round(n * (sel.size / uv.size) / tc, 1), "unit": "vertices/s", "cores": 1,
                                  "kind": "port", "sample": "calc_m restatement on %d of %d objects (%.2f s per pass, 3 passes), "
                                  "object analysis excluded" % (sel.size, uv.size, tc)}
    return result


def cpu_reference_full(w, K, n):
    """The reference's own CPU kernel (its sources compiled unmodified into oracle/_ref) on every query of the
    workload, single-threaded as it is written (binned_select_knn_cpu.cpp:56-208 has no parallel loop), with the
    reference's own grid (calculate_optimal_bins).  Search kernel only, like cpu_baseline."""
    from oracle import oracle as O
    if O.ref_lib() is None:
        return {"value": None, "kind": "reference", "sample": "oracle/_ref is not built on this machine"}
    s = O.sorted_space(w["coords"], w["row_splits"], K)
    a = (s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"], s["n_bins"], s["bin_width"], K)
    import threading
    done = threading.Event()

    def heartbeat():            # minutes of silent CPU work: say so now and then
        while not done.wait(30.0):
            print("bench.py: reference CPU kernel still running (%.0f s)" % (time.perf_counter() - t0),
                  file=sys.stderr, flush=True)

    t0 = time.perf_counter()
    threading.Thread(target=heartbeat, daemon=True).start()
    try:
        O.knn_sorted(*a, use_ref=True)
    finally:
        done.set()
    t = time.perf_counter() - t0
    return {"value": round(n / t, 1), "unit": "queries/s", "cores": 1, "kind": "reference",
            "sample": "all %d queries of the bin-sorted workload, %.1f s, n_bins %s; kNN search kernel only"
                      % (n, t, [int(v) for v in s["n_bins"]])}


def cpu_baseline(w, K, n, budget_s):
    """The reference's CPU search on this box's host cores, on a bounded sample of the workload's queries.

    Headline (`kind: "reference"`): the reference's own kernel (binned_select_knn_cpu.cpp:56-208, compiled unmodified
    into oracle/_ref), single-threaded as it is written, with the reference's own grid.  The kernel has no query
    stride, but it skips a query whose direction flag is 0 and still takes that point as a neighbour
    (binned_select_knn_cpu.cpp:80-83,157-160): all points but every s-th get flag 0, the sampled ones a flag that
    allows both roles, and use_direction is set - the unmodified kernel then searches the sampled queries among ALL
    points.  The rows of the sampled queries are compared with the restatement's (oracle/, `kind: "port"`), which is
    timed on the same queries; where oracle/_ref is not built the restatement is the headline.
    Returns (one-core entry, all-cores entry of the restatement with OpenMP over the queries)."""
    import numpy as np
    from oracle import oracle as O
    s = O.sorted_space(w["coords"], w["row_splits"], K)
    args = (s["scoords"], s["sbin"], s["sdbin"], s["bin_boundaries"], s["n_bins"], s["bin_width"], K)
    stride = max(1, n // 2000)
    t0 = time.perf_counter()
    O.knn_sorted(*args, n_threads=1, query_stride=stride)
    probe = time.perf_counter() - t0
    per_query = probe / max(1, (n + stride - 1) // stride)
    have_ref = O.ref_lib() is not None
    # the reference's kernel takes about twice the restatement's time per query; both run on the same sample
    want = max(1, int(budget_s / max((2.2 if have_ref else 1.0) * per_query, 1e-9)))
    stride2 = max(1, n // want)
    t0 = time.perf_counter()
    pi, pd, ev2, _ = O.knn_sorted(*args, n_threads=1, query_stride=stride2)
    t = time.perf_counter() - t0
    nq = (n + stride2 - 1) // stride2
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    import torch
    host = {"cpu_model": cpu_model, "nproc": os.cpu_count(), "usable_cores": len(os.sched_getaffinity(0)),
            "torch_threads": torch.get_num_threads()}
    sample = ("every %d-th query of the bin-sorted workload (%d queries) among all %d points, n_bins %s; kNN search "
              "kernel only, binning and sort excluded" % (stride2, nq, n, [int(v) for v in s["n_bins"]]))
    port = {"value": round(nq / t, 1), "unit": "queries/s", "cores": 1, "kind": "port", "seconds": round(t, 1),
            "distance_evaluations": int(ev2)}
    if have_ref:
        tiny = O.sorted_space(w["coords"][:256], np.array([0, 256], dtype=np.int64), 4)   # loads the library, untimed
        O.knn_sorted(tiny["scoords"], tiny["sbin"], tiny["sdbin"], tiny["bin_boundaries"], tiny["n_bins"],
                     tiny["bin_width"], 4, use_ref=True)
        direction = np.zeros(n, dtype=np.int64)           # 0: may only be a neighbour
        direction[::stride2] = 3                          # neither 0, 1 nor 2: query and neighbour
        t0 = time.perf_counter()
        ri, rd, _, _ = O.knn_sorted(*args, sdirection=direction, use_ref=True)
        t_ref = time.perf_counter() - t0
        same = bool((ri[::stride2] == pi[::stride2]).all() and (rd[::stride2] == pd[::stride2]).all())
        one = {"value": round(nq / t_ref, 1), "unit": "queries/s", "cores": 1, "kind": "reference", "host": host,
               "seconds": round(t_ref, 1),
               "sample": sample + "; the reference's compiled kernel, unmodified, the other queries switched off "
                                  "through its direction flags",
               "rows_identical_to_port_on_the_sample": same, "port_on_the_same_sample": port}
    else:
        one = dict(port, host=host, sample=sample + "; oracle/_ref is not built on this machine")
    # the restatement with OpenMP over the queries on the cores this process may use (the reference's CPU kernel
    # itself is single-threaded); a second, shorter sample
    threads = max(1, min(O.lib().fgc_oracle_max_threads(), len(os.sched_getaffinity(0)), 16))
    stride3 = max(1, stride2 // max(1, threads // 2))
    t0 = time.perf_counter()
    O.knn_sorted(*args, n_threads=threads, query_stride=stride3)
    t3 = time.perf_counter() - t0
    nq3 = (n + stride3 - 1) // stride3
    many = {"value": round(nq3 / t3, 1), "unit": "queries/s", "cores": threads, "kind": "port",
            "sample": "every %d-th query (%d queries, %.1f s), OpenMP over queries" % (stride3, nq3, t3)}
    return one, many


if __name__ == "__main__":
    main()
