#!/usr/bin/env python3
"""Headline benchmark: QPS @ recall@10 of the flat SQ8 scan (1M x 128 codes, 10 000 queries, k = 10).

One step = one pass of the hot path (query preparation + scan with fused top-k + merge) over the whole
query batch, inputs resident in HBM.  Prints ONE JSON line with the metric, the roofline of the dominant
kernel (HIP events recorded by the library around that kernel on its own stream) and the CPU baseline
(the reference's own SIMD kernel compiled from its sources when oracle/_ref is present, else the CPU
restatement), timed on this host's cores on a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0


def mixture(seed_means, seed_rows, n, d, components, sigma, means=None):
    """Gaussian mixture drawn from MT19937 streams (means uniform[0,1)^d, isotropic sigma)."""
    if means is None:
        means = np.random.Generator(np.random.MT19937(seed_means)).random((components, d), dtype=np.float32)
    rng = np.random.Generator(np.random.MT19937(seed_rows))
    out = np.empty((n, d), np.float32)
    step = 1 << 17
    for s in range(0, n, step):
        e = min(n, s + step)
        which = rng.integers(0, components, e - s)
        out[s:e] = means[which] + np.float32(sigma) * rng.standard_normal((e - s, d), dtype=np.float32)
    return out, means


def exact_topk_host(x, q, k, metric):
    """Exact ground truth on the host, independent of the library: an fp32 GEMM pre-selects 8k candidates
    per query, their distances are then recomputed directly in fp64 and the k nearest kept."""
    n = x.shape[0]
    pre = min(n, 8 * k)
    cand_d = np.full((q.shape[0], 0), np.inf, np.float32)
    cand_i = np.zeros((q.shape[0], 0), np.int64)
    xn = None
    chunk = 1 << 17
    for s in range(0, n, chunk):
        xb = x[s:s + chunk]
        ip = q @ xb.T
        if metric == "l2":
            xn = np.einsum("ij,ij->i", xb, xb)
            dist = xn[None, :] - 2.0 * ip
        else:
            dist = -ip
        m = min(pre, dist.shape[1])
        part = np.argpartition(dist, m - 1, axis=1)[:, :m]
        cand_d = np.concatenate([cand_d, np.take_along_axis(dist, part, 1)], 1)
        cand_i = np.concatenate([cand_i, part + s], 1)
        if cand_d.shape[1] > pre:
            keep = np.argpartition(cand_d, pre - 1, axis=1)[:, :pre]
            cand_d = np.take_along_axis(cand_d, keep, 1)
            cand_i = np.take_along_axis(cand_i, keep, 1)
    out = np.empty((q.shape[0], k), np.int64)
    for i in range(q.shape[0]):
        xs = x[cand_i[i]].astype(np.float64)
        qq = q[i].astype(np.float64)
        dd = ((xs - qq) ** 2).sum(1) if metric == "l2" else 1.0 - xs @ qq
        order = np.lexsort((cand_i[i], dd))[:k]
        out[i] = cand_i[i][order]
    return out


def recall_at_k(ids, gt):
    hits = 0
    for a, b in zip(ids, gt):
        hits += len(set(int(v) for v in a) & set(int(v) for v in b))
    return hits / float(gt.size)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--n", type=int, default=1000000)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--nq", type=int, default=10000)
    ap.add_argument("--k", type=int, default=10)
    ap.add_argument("--tile", type=int, default=0, help="query tile override (0 = library default)")
    ap.add_argument("--chunks", type=int, default=0, help="base chunk override (0 = library default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-recall", action="store_true", help="skip the recall check")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the search core is single-GPU by design (see DESIGN.md); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from vsag_amd import capi
    lib = capi.load_library()
    capi.init(0)
    dev_name, cus, hbm = capi.device_info()
    n, d, nq, k = args.n, args.dim, args.nq, args.k

    t0 = time.time()
    x, means = mixture(315, 47, n, d, 1000, 0.05)
    q, _ = mixture(315, 165, nq, d, 1000, 0.05, means=means)
    t_gen = time.time() - t0

    # Build on the device: train bounds, encode, re-tile (Index::Build of the reference's brute_force).
    x_dev = capi.DeviceBuffer.from_numpy(x)
    lb_dev, diff_dev = capi.DeviceBuffer(d * 4), capi.DeviceBuffer(d * 4)
    wsb = lib.vsag_amd_sq_train_workspace_bytes(n, d, 0)
    ws = capi.DeviceBuffer(wsb)
    t0 = time.time()
    capi.check(lib.vsag_amd_sq_train(x_dev.ptr, n, d, 8, capi.METRIC_L2, capi.SQ_TRAIN_TRUNC_BOUND, 0.05, 0,
                                     lb_dev.ptr, diff_dev.ptr, ws.ptr, wsb, None))
    codes_dev = capi.DeviceBuffer(n * d)
    capi.check(lib.vsag_amd_sq_encode(x_dev.ptr, n, d, 8, capi.METRIC_L2, lb_dev.ptr, diff_dev.ptr, codes_dev.ptr,
                                      None))
    stores = {}
    for name, metric in (("l2", capi.METRIC_L2), ("ip", capi.METRIC_IP)):
        p = capi.StoreParams()
        p.kind, p.metric, p.dim = capi.KIND_SQ8, metric, d
        p.lower_bound_dev, p.diff_dev = lb_dev.ptr, diff_dev.ptr
        h = C.c_void_p()
        capi.check(lib.vsag_amd_store_create(C.byref(p), C.byref(h)))
        capi.check(lib.vsag_amd_store_append(h, codes_dev.ptr, n, None))
        stores[name] = h
    capi.synchronize()
    t_build = time.time() - t0
    ws.free()

    q_dev = capi.DeviceBuffer.from_numpy(q)
    ids_dev, ds_dev = capi.DeviceBuffer(nq * k * 4), capi.DeviceBuffer(nq * k * 4)
    capi.check(lib.vsag_amd_set_scan_tuning(args.tile, args.chunks))
    capi.check(lib.vsag_amd_set_kernel_timing(1))

    results = {}
    for name in ("ip", "l2"):  # l2 last: it is the headline line
        h = stores[name]
        wsb = lib.vsag_amd_flat_scan_workspace_bytes(h, nq, k)
        ws = capi.DeviceBuffer(wsb)

        def step():
            capi.check(lib.vsag_amd_flat_scan_topk(h, q_dev.ptr, nq, k, ids_dev.ptr, ds_dev.ptr, ws.ptr, wsb, None))

        for _ in range(args.warmup):
            step()
        capi.synchronize()
        kernel_ms = []
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
            ms = C.c_float()
            capi.check(lib.vsag_amd_last_kernel_ms(C.byref(ms)))
            kernel_ms.append(ms.value)
        capi.synchronize()
        wall = time.perf_counter() - t0
        tile, passes, bytes_per_pass = C.c_int(), C.c_uint64(), C.c_uint64()
        lib.vsag_amd_last_scan_info(C.byref(tile), C.byref(passes), C.byref(bytes_per_pass))
        ids = ids_dev.to_numpy(np.uint32, (nq, k))
        results[name] = dict(ms_per_step=1e3 * wall / args.steps, qps=nq * args.steps / wall,
                             kernel_ms=float(np.mean(kernel_ms)), tile=tile.value, passes=passes.value,
                             bytes_per_pass=bytes_per_pass.value, ids=ids)
        ws.free()

    # recall@10 against exact brute force on the raw fp32 vectors (host, fp64 distances) on the first queries
    recall = {}
    if not args.no_recall:
        nrec = min(nq, 500)
        for name in ("l2", "ip"):
            gt = exact_topk_host(x, q[:nrec], k, name)
            recall[name] = recall_at_k(results[name]["ids"][:nrec], gt)

    # CPU baseline on a bounded sample of the same workload
    cpu = None
    if not args.no_cpu:
        import oracle as orc
        codes = codes_dev.to_numpy(np.uint8, (n, d))
        lb = lb_dev.to_numpy(np.float32, (d,))
        diff = diff_dev.to_numpy(np.float32, (d,))
        threads = min(os.cpu_count() or 1, 16)
        isa = orc.ref_best_isa()
        fn = orc.ref_sq8_fn(orc.L2, isa)
        sample = min(nq, 8 * threads)
        kind = "reference" if fn is not None else "port"

        def run_cpu(qs, th):
            if fn is not None:
                return orc.flat_scan_topk_fn(fn, orc.L2, d, codes, qs, k, lb, diff, threads=th)
            return orc.flat_scan_topk(orc.SQ8, orc.L2, d, codes, qs, k, lb=lb, diff=diff, threads=th)

        run_cpu(q[:threads], threads)  # thread pool and page warm-up
        t0 = time.perf_counter()
        cids, _ = run_cpu(q[:sample], threads)
        t_all = time.perf_counter() - t0
        t0 = time.perf_counter()
        run_cpu(q[:2], 1)
        t_one = (time.perf_counter() - t0) / 2
        same = float(np.mean([len(set(a) & set(b)) / float(k) for a, b in zip(cids, results["l2"]["ids"][:sample])]))
        cpu = {"value": sample / t_all, "unit": "queries/s", "cores": threads, "kind": kind,
               "sample": "%d of the %d queries over all %d codes, one query per call, OpenMP dynamic over queries; "
                         "distance = %s, loop and heap = restated BruteForce::SearchWithRequest" %
                         (sample, nq, n, ("vsag::%s::SQ8ComputeL2Sqr compiled from the reference sources" % isa)
                          if fn is not None else "CPU restatement (oracle)"),
               "single_thread_qps": 1.0 / t_one, "topk_overlap_with_gpu": same}

    r = results["l2"]
    algo_bytes = r["passes"] * r["bytes_per_pass"]
    achieved = algo_bytes / (r["kernel_ms"] * 1e-3) / 1e9
    ri = results["ip"]
    out = {
        "metric": "QPS @ recall@10 (1M x 128 SQ8 scan)",
        "value": r["qps"],
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": r["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8 codes, f32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: flat SQ8 scan, N=%d, d=%d, %d queries, k=%d, L2 (headline) and IP" % (n, d, nq, k),
            "recall_at_10_l2": recall.get("l2"), "recall_at_10_ip": recall.get("ip"),
            "ip_qps": ri["qps"], "ip_ms_per_step": ri["ms_per_step"], "ip_query_tile": ri["tile"],
            "ip_kernel_ms": ri["kernel_ms"],
            "ip_algorithmic_gbs": ri["passes"] * ri["bytes_per_pass"] / (ri["kernel_ms"] * 1e-3) / 1e9,
            "query_tile": r["tile"], "passes_per_step": r["passes"], "bytes_per_pass": r["bytes_per_pass"],
            "build_seconds": t_build, "datagen_seconds": t_gen, "device": dev_name, "compute_units": cus,
        },
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "flat_scan_kernel<sq8, l2, T=%d>" % r["tile"], "kernel_ms": r["kernel_ms"],
                     "algorithmic_bytes_per_launch": algo_bytes},
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
