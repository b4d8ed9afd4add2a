#!/usr/bin/env python3
"""Benchmarks of the MI355X search core on the reference's five configurations.

Default (what the driver runs): --config c2, the headline metric "QPS @ recall@10 (1M x 128 SQ8 scan)":
one step = one pass of the hot path (query preparation + scan with fused top-k + merge) over the whole
query batch, inputs resident in HBM.  Prints ONE JSON line with the metric, the roofline of the dominant
kernel (HIP events recorded by the library around that kernel on its own stream) and the CPU baseline
(the reference's own SIMD kernel compiled from its sources when oracle/_ref is present, else the CPU
restatement), timed on this host's cores on a bounded sample of the same workload.  The same line carries
one block per other configuration -- "kmeans" (configs[2]), "c1" (configs[0]), "c4" (configs[3]), "c5"
(configs[4]) -- each with its own value, recall, roofline and CPU baseline (--only leaves them out).

--config c1 | c3 | c4 | c5 print one line each in the same shape for the fp32 brute-force scan, k-means
assignment, the IVF SQ4-uniform search and the RaBitQ scan + rerank alone.
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
MFMA_F32_PEAK_TFLOPS = 157.3
MFMA_I8_PEAK_TOPS = 5000.0  # dense int8, published
MFMA_F6F4_PEAK_TFLOPS = 10100.0  # dense fp6 / fp4, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16 / bf16, published
# HBM/fabric bytes of the last-level launch of prefilter_i8_kernel<l2> on configs[1] (profiles/prefilter_i8_sq8_c2.md)
PROFILE_TRAFFIC_I8_C2 = 235670.3 * 2.00 * 1024 + 60099.9 * 1024


def mt(seed):
    return np.random.Generator(np.random.MT19937(seed))


def mixture_chunks(seed_rows, n, d, means, sigma, step=1 << 17):
    """Gaussian-mixture rows in chunks, drawn from one MT19937 stream."""
    rng = mt(seed_rows)
    for s in range(0, n, step):
        e = min(n, s + step)
        which = rng.integers(0, means.shape[0], e - s)
        yield s, means[which] + np.float32(sigma) * rng.standard_normal((e - s, d), dtype=np.float32)


def mixture(seed_means, seed_rows, n, d, components, sigma, means=None, normal_means=False):
    if means is None:
        g = mt(seed_means)
        means = g.standard_normal((components, d), dtype=np.float32) if normal_means else \
            g.random((components, d), dtype=np.float32)
    out = np.empty((n, d), np.float32)
    for s, blk in mixture_chunks(seed_rows, n, d, means, sigma):
        out[s:s + blk.shape[0]] = blk
    return out, means


def exact_topk_host(x, q, k, metric):
    """Exact ground truth on the host, independent of the library: an fp32 GEMM pre-selects 8k candidates
    per query, their distances are then recomputed directly in fp64 and the k nearest kept."""
    n = x.shape[0]
    pre = min(n, 8 * k)
    cand_d = np.full((q.shape[0], 0), np.inf, np.float32)
    cand_i = np.zeros((q.shape[0], 0), np.int64)
    chunk = 1 << 17
    for s in range(0, n, chunk):
        xb = x[s:s + chunk]
        ip = q @ xb.T
        dist = np.einsum("ij,ij->i", xb, xb)[None, :] - 2.0 * ip if metric == "l2" else -ip
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


def blas_name():
    try:
        cfg = np.show_config(mode="dicts")
        b = cfg["Build Dependencies"]["blas"]
        return "%s %s" % (b.get("name", "blas"), b.get("version", ""))
    except Exception:  # noqa: BLE001 - older numpy: no dict form
        return "numpy's BLAS"


def cpu_assign_sgemm(x, cent, threads):
    """KMeansCluster::find_nearest_one_with_blas (impl/cluster/kmeans_cluster.cpp:193-305) with the BLAS numpy links:
    per chunk of 65 536 rows distances = -2 C X^T by SGEMM, then per row (blocks of 1024 rows on the thread pool)
    += |c|^2, first minimum, error += double(float(min + |x|^2)).  Returns (labels, error / n)."""
    from concurrent.futures import ThreadPoolExecutor
    n, k = x.shape[0], cent.shape[0]
    y_sqr = np.einsum("ij,ij->i", cent, cent).astype(np.float32)
    labels = np.empty(n, np.int32)
    ct = np.ascontiguousarray(cent.T)
    err = 0.0

    def block(args):
        dist, xb, lo, hi = args
        blk = dist[lo:hi]
        blk += y_sqr[None, :]
        idx = blk.argmin(1)
        labels_chunk[lo:hi] = idx
        x_sqr = np.einsum("ij,ij->i", xb[lo:hi], xb[lo:hi]).astype(np.float32)
        return float((blk[np.arange(hi - lo), idx] + x_sqr).astype(np.float64).sum())

    with ThreadPoolExecutor(max_workers=threads) as pool:
        for s in range(0, n, 65536):
            xb = x[s:s + 65536]
            dist = np.matmul(xb, ct)
            dist *= np.float32(-2.0)
            labels_chunk = labels[s:s + 65536]
            m = xb.shape[0]
            err += sum(pool.map(block, [(dist, xb, lo, min(lo + 1024, m)) for lo in range(0, m, 1024)]))
    return labels, err / float(n)


def device_rows(env, x_dev, rows, d):
    """Rows of a device-resident n x d fp32 matrix, copied one by one (a few thousand at most)."""
    rows = np.asarray(rows, np.int64)
    out = np.empty((rows.size, d), np.float32)
    for i, r in enumerate(rows):
        env.capi.check(env.lib.vsag_amd_memcpy_d2h(out[i].ctypes.data, x_dev.ptr + int(r) * d * 4, d * 4, None))
    return out


def recall_at_k(ids, gt):
    hits = 0
    for a, b in zip(ids, gt):
        hits += len(set(int(v) for v in a) & set(int(v) for v in b))
    return hits / float(gt.size)


class Env:
    def __init__(self, args):
        from vsag_amd import capi
        self.capi = capi
        self.lib = capi.load_library()
        capi.init(0)
        self.dev_name, self.cus, self.hbm = capi.device_info()
        self.args = args
        self.stores = []
        capi.check(self.lib.vsag_amd_set_kernel_timing(1))

    def buf(self, nbytes):
        return self.capi.DeviceBuffer(nbytes)

    def upload(self, arr):
        return self.capi.DeviceBuffer.from_numpy(arr)

    def kernel_ms(self):
        ms = C.c_float()
        self.capi.check(self.lib.vsag_amd_last_kernel_ms(C.byref(ms)))
        return ms.value

    def make_store(self, kind, metric, dim, lb=None, diff=None, bounds=None, rot=None, cen=None, qbits=4, pq_dim=0,
                   codebooks=None):
        p = self.capi.StoreParams()
        p.kind, p.metric, p.dim, p.rabitq_query_bits = kind, metric, dim, qbits
        if codebooks is not None:
            p.pq_dim, p.codebooks_dev = pq_dim, codebooks.ptr
        if lb is not None:
            p.lower_bound_dev, p.diff_dev = lb.ptr, diff.ptr
        if bounds is not None:
            p.lower_bound_dev = bounds.ptr
        if rot is not None:
            p.rotation_dev, p.centroid_dev = rot.ptr, cen.ptr
        h = C.c_void_p()
        self.capi.check(self.lib.vsag_amd_store_create(C.byref(p), C.byref(h)))
        self.stores.append(h)
        return h

    def release(self):
        """Destroys the stores of the configuration that just ran (its buffers go with their Python objects)."""
        import gc
        self.capi.synchronize()
        for h in self.stores:
            self.lib.vsag_amd_store_destroy(h)
        self.stores = []
        gc.collect()

    def timed(self, step, steps, warmup):
        for _ in range(warmup):
            step()
        self.capi.synchronize()
        kms = []
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
            kms.append(self.kernel_ms())
        self.capi.synchronize()
        wall = time.perf_counter() - t0
        return wall / steps, float(np.mean(kms))

    def flat_scan_fn(self, store, q_dev, nq, k, ids_dev, ds_dev):
        wsb = self.lib.vsag_amd_flat_scan_workspace_bytes(store, nq, k)
        ws = self.buf(wsb)

        def step():
            self.capi.check(self.lib.vsag_amd_flat_scan_topk(store, q_dev.ptr, nq, k, ids_dev.ptr, ds_dev.ptr, ws.ptr,
                                                             wsb, None))
        return step, ws

    def scan_info(self):
        tile, passes, bpp = C.c_int(), C.c_uint64(), C.c_uint64()
        self.lib.vsag_amd_last_scan_info(C.byref(tile), C.byref(passes), C.byref(bpp))
        return tile.value, passes.value, bpp.value

    def base_line(self, metric, unit, value, sec_per_step, dtype, workload, extra, roofline, cpu):
        cfg = {"workload": workload, "device": self.dev_name, "compute_units": self.cus}
        cfg.update(extra)
        if roofline is not None and "traffic_source" not in roofline:
            roofline["traffic_source"] = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, from the committed "
                                          "summary under profiles/; not measured in this run"
                                          if roofline.get("traffic") is not None else None)
        return {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": self.args.steps,
                "warmup": self.args.warmup, "ms_per_step": 1e3 * sec_per_step, "higher_is_better": True,
                "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": cfg,
                "roofline": roofline, "cpu_baseline": cpu}


# ------------------------------------------------------------------------------------------- C2 (headline)
def run_c2(env):
    args, capi, lib = env.args, env.capi, env.lib
    n, d, nq, k = args.n or 1000000, args.dim or 128, args.nq or 10000, args.k
    t0 = time.time()
    x, means = mixture(315, 47, n, d, 1000, 0.05)
    q, _ = mixture(315, 165, nq, d, 1000, 0.05, means=means)
    t_gen = time.time() - t0

    # Build on the device: train bounds, encode, re-tile (Index::Build of the reference's brute_force).
    x_dev = env.upload(x)
    lb_dev, diff_dev = env.buf(d * 4), env.buf(d * 4)
    wsb = lib.vsag_amd_sq_train_workspace_bytes(n, d, 0)
    ws = env.buf(wsb)
    t0 = time.time()
    capi.check(lib.vsag_amd_sq_train(x_dev.ptr, n, d, 8, capi.METRIC_L2, capi.SQ_TRAIN_TRUNC_BOUND, 0.05, 0,
                                     lb_dev.ptr, diff_dev.ptr, ws.ptr, wsb, None))
    codes_dev = env.buf(n * d)
    capi.check(lib.vsag_amd_sq_encode(x_dev.ptr, n, d, 8, capi.METRIC_L2, lb_dev.ptr, diff_dev.ptr, codes_dev.ptr,
                                      None))
    stores = {}
    for name, metric in (("l2", capi.METRIC_L2), ("ip", capi.METRIC_IP)):
        stores[name] = env.make_store(capi.KIND_SQ8, metric, d, lb=lb_dev, diff=diff_dev)
        capi.check(lib.vsag_amd_store_append(stores[name], codes_dev.ptr, n, None))
    capi.synchronize()
    t_build = time.time() - t0
    ws.free()
    x_dev.free()

    q_dev = env.upload(q)
    ids_dev, ds_dev = env.buf(nq * k * 4), env.buf(nq * k * 4)
    capi.check(lib.vsag_amd_set_scan_tuning(args.tile, args.chunks))
    results = {}
    for name in ("ip", "l2"):  # l2 last: it is the headline line
        step, ws = env.flat_scan_fn(stores[name], q_dev, nq, k, ids_dev, ds_dev)
        sec, kms = env.timed(step, args.steps, args.warmup)
        tile, passes, bpp = env.scan_info()
        results[name] = dict(sec=sec, qps=nq / sec, kernel_ms=kms, tile=tile, passes=passes, bytes_per_pass=bpp,
                             ids=ids_dev.to_numpy(np.uint32, (nq, k)))
        ws.free()

    # one query per call (the reference's own call pattern): a single streaming pass over the codes
    single = None
    if not args.no_single:
        step, ws = env.flat_scan_fn(stores["l2"], q_dev, 1, k, ids_dev, ds_dev)
        sec, kms = env.timed(step, 50, 5)
        _, _, bpp = env.scan_info()
        single = {"latency_us": 1e6 * sec, "kernel_us": 1e3 * kms, "hbm_gbs": bpp / (kms * 1e-3) / 1e9,
                  "hbm_frac": bpp / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        ws.free()

    # The same search through the index API with host buffers on both sides, as a user of the reference calls it
    # (tools/eval/case/search_eval_case.cpp:233-277): Factory::CreateIndex("brute_force") -> Build -> KnnSearch.
    # A step uploads the queries, runs the scan above, downloads ids and distances and maps inner ids to labels.
    api = None
    if not args.no_api:
        from vsag_amd import pyvsag
        params = json.dumps({"dtype": "float32", "metric_type": "l2", "dim": d,
                             "index_param": {"base_quantization_type": "sq8"}})
        index = pyvsag.Index("brute_force", params)
        labels = np.arange(n, dtype=np.int64) + 1000000007
        t0 = time.perf_counter()
        index.build(x, labels, n, d)
        api_build = time.perf_counter() - t0
        for _ in range(max(1, args.warmup)):
            aids, adist = index.knn_search_batch(q, k, "{}")
        capi.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            aids, adist = index.knn_search_batch(q, k, "{}")
        api_sec = (time.perf_counter() - t0) / args.steps
        # one query per call, the reference evaluator's protocol (tools/eval/case/search_eval_case.cpp:233-277): from
        # one caller thread, then from as many as the CPU baseline uses, all on the one index
        index.eval_knn_search(q[:64], k, "{}", 1)
        e_ids, _, e_sec = index.eval_knn_search(q[:2000], k, "{}", 1)
        api_one = e_sec / 2000
        threads = min(os.cpu_count() or 1, 16)
        index.eval_knn_search(q[:256], k, "{}", threads)
        c_ids, _, c_sec = index.eval_knn_search(q, k, "{}", threads)
        api = {"qps": nq / api_sec, "ms_per_step": 1e3 * api_sec, "build_seconds": api_build,
               "one_query_per_call_us": 1e6 * api_one,
               "concurrent_one_query_qps": nq / c_sec, "concurrent_threads": threads,
               "concurrent_same_ids_as_batch": float(np.mean(c_ids == aids)),
               "same_ids_as_resident_path": float(np.mean(aids - 1000000007 == results["l2"]["ids"])),
               "what": "vsag::Factory::CreateIndex(brute_force, sq8) -> Build(%d x %d host floats) -> KnnSearch(%d host "
                       "queries, k=%d) -> host ids / distances, PCIe copies and label mapping included" % (n, d, nq, k)}
        index.close()

    recall = {}
    if not args.no_recall:
        nrec = min(nq, 500)
        for name in ("l2", "ip"):
            gt = exact_topk_host(x, q[:nrec], k, name)
            recall[name] = recall_at_k(results[name]["ids"][:nrec], gt)

    cpu = None
    if not args.no_cpu:
        import oracle as orc
        codes = codes_dev.to_numpy(np.uint8, (n, d))
        lb = lb_dev.to_numpy(np.float32, (d,))
        diff = diff_dev.to_numpy(np.float32, (d,))
        threads = min(os.cpu_count() or 1, 16)
        isa = orc.ref_best_isa()
        fn = orc.ref_sq8_fn(orc.L2, isa)
        sample = min(nq, 64 * threads)

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
        cpu = {"value": sample / t_all, "unit": "queries/s", "cores": threads,
               "kind": "reference" if fn is not None else "port",
               "sample": "%d of the %d queries over all %d codes, one query per call, OpenMP dynamic over queries; "
                         "distance = %s, loop and heap = restated BruteForce::SearchWithRequest" %
                         (sample, nq, n, ("vsag::%s::SQ8ComputeL2Sqr compiled from the reference sources" % isa)
                          if fn is not None else "CPU restatement (oracle)"),
               "single_thread_qps": 1.0 / t_one, "topk_overlap_with_gpu": same}

    r, ri = results["l2"], results["ip"]
    algo_bytes = r["passes"] * r["bytes_per_pass"]
    achieved = algo_bytes / (r["kernel_ms"] * 1e-3) / 1e9
    extra = {"recall_at_10_l2": recall.get("l2"), "recall_at_10_ip": recall.get("ip"),
             "ip_qps": ri["qps"], "ip_ms_per_step": 1e3 * ri["sec"], "ip_query_tile": ri["tile"],
             "ip_kernel_ms": ri["kernel_ms"],
             "ip_algorithmic_gbs": ri["passes"] * ri["bytes_per_pass"] / (ri["kernel_ms"] * 1e-3) / 1e9,
             "query_tile": r["tile"], "passes_per_step": r["passes"], "bytes_per_pass": r["bytes_per_pass"],
             "single_query_l2": single, "index_api_l2": api, "build_seconds": t_build, "datagen_seconds": t_gen}
    # HBM/fabric bytes of one launch of this exact configuration come from rocprofv3 --pmc runs of this command
    # (FETCH_SIZE x 2.00, the factor that makes kernels of known size read their size, + WRITE_SIZE x 1.00); they are
    # constants of the committed profile, not measurements of this run, and are labelled so.
    traffic, traffic_source = None, None
    if (n, d, nq, k, r["tile"]) == (1000000, 128, 10000, 10, 4):
        traffic, traffic_source = 115043826 * 2.00 * 1024 + 28593 * 1024, "profiles/flat_scan_sq8_c2.md"
    elif (n, d, nq, k, r["tile"]) == (1000000, 128, 10000, 10, 256):
        traffic, traffic_source = PROFILE_TRAFFIC_I8_C2, "profiles/prefilter_i8_sq8_c2.md"
    if traffic_source is not None:
        traffic_source += " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command; not measured in this run)"
    roof = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
            "kernel": "flat_scan_kernel<sq8, l2, T=%d>" % r["tile"], "kernel_ms": r["kernel_ms"],
            "algorithmic_bytes_per_launch": algo_bytes}
    if r["tile"] >= 64:
        # The batch went through a matrix-core pre-selection (query tile 256: int8, 128: fp32): the timed kernel meets
        # every code of the last level (bytes_per_pass / padded code bytes of them) with every query.  Algorithmic work
        # of the launch = 2 d operations per (query, code) pair; the int8 kernel executes twice that (two int8 planes
        # per query), reported beside it.  The same launch by the memory figure: passes x code bytes.
        i8 = r["tile"] == 256
        # (beyond 128 dimensions the fp16 matrix cores take the code bytes and one fp16 part of the scaled query)
        h16 = not i8 and d > 128 and args.contraction != 2
        codes = r["bytes_per_pass"] / float(-(-d // 16) * 16)
        ops = 2.0 * codes * d * nq
        rate = ops / (r["kernel_ms"] * 1e-3) / 1e12
        peak = MFMA_I8_PEAK_TOPS if i8 else MFMA_F16_PEAK_TFLOPS if h16 else MFMA_F32_PEAK_TFLOPS
        roof = {"bound": "mfma", "achieved": rate, "peak": peak, "unit": "TOP/s" if i8 else "TFLOP/s",
                "frac": rate / peak, "traffic": traffic, "traffic_source": traffic_source,
                "kernel": "prefilter_i8_kernel<l2> (int8 MFMA, last level)" if i8 else
                          "prefilter_h16_kernel (fp16 MFMA, last level)" if h16 else "prefilter_kernel<sq8> (fp32 MFMA)",
                "kernel_ms": r["kernel_ms"], "ops_per_launch": ops, "codes_per_launch": codes,
                "mfma_frac": rate / peak,
                "executed_ops_per_launch": (2.0 if i8 else 1.0) * 2.0 * codes * (-(-d // 32) * 32) * nq,
                "executed_frac": (2.0 if i8 else 1.0) * 2.0 * codes * (-(-d // 32) * 32) * nq /
                                 (r["kernel_ms"] * 1e-3) / 1e12 / peak,
                "algorithmic_bytes_per_launch": algo_bytes, "algorithmic_gbs": achieved,
                "hbm_frac_algorithmic": achieved / HBM_PEAK_GBS}
    return env.base_line("QPS @ recall@10 (1M x 128 SQ8 scan)", "queries/s", r["qps"], r["sec"],
                         "u8 codes; i8 x i8 -> i32 pre-selection, f32 results" if r["tile"] == 256 else
                         "u8 codes, f32 accumulate",
                         "configs[1]: flat SQ8 scan, N=%d, d=%d, %d queries, k=%d, L2 (headline) and IP" % (n, d, nq, k),
                         extra, roof, cpu)


# ------------------------------------------------------------------------------------------- C1
def run_c1(env):
    args, capi, lib = env.args, env.capi, env.lib
    n, d, nq, k = args.n or 100000, args.dim or 128, args.nq or 1000, args.k
    x = mt(47).random((n, d), dtype=np.float32)
    q = mt(165).random((nq, d), dtype=np.float32)
    store = env.make_store(capi.KIND_FP32, capi.METRIC_L2, d)
    x_dev = env.upload(x)
    capi.check(lib.vsag_amd_store_append(store, x_dev.ptr, n, None))
    q_dev = env.upload(q)
    ids_dev, ds_dev = env.buf(nq * k * 4), env.buf(nq * k * 4)
    capi.check(lib.vsag_amd_set_scan_tuning(args.tile, args.chunks))
    step, ws = env.flat_scan_fn(store, q_dev, nq, k, ids_dev, ds_dev)
    sec, kms = env.timed(step, args.steps, args.warmup)
    tile, passes, bpp = env.scan_info()
    ids = ids_dev.to_numpy(np.uint32, (nq, k))
    rec = None if args.no_recall else recall_at_k(ids[:200], exact_topk_host(x, q[:200], k, "l2"))
    cpu = None
    if not args.no_cpu:
        import oracle as orc
        threads = min(os.cpu_count() or 1, 16)
        sample = nq
        codes = x.view(np.uint8).reshape(n, 4 * d)
        ref = orc.use_reference_kernels(orc.ref_best_isa())
        orc.flat_scan_topk(orc.FP32, orc.L2, d, codes, q[:threads], k, threads=threads)
        t0 = time.perf_counter()
        cids, _ = orc.flat_scan_topk(orc.FP32, orc.L2, d, codes, q[:sample], k, threads=threads)
        t_cpu = time.perf_counter() - t0
        orc.use_reference_kernels(None)
        cpu = {"value": sample / t_cpu, "unit": "queries/s", "cores": threads,
               "kind": "reference" if ref else "port",
               "sample": "%d of the %d queries over all %d vectors, one query per call, OpenMP dynamic over queries; "
                         "distance = %s, loop and heap = restated BruteForce::SearchWithRequest" %
                         (sample, nq, n, (ref["FP32ComputeL2Sqr"] + " compiled from the reference sources") if ref
                          else "CPU restatement of generic::FP32ComputeL2Sqr"),
               "topk_overlap_with_gpu": float(np.mean([len(set(a) & set(b)) / float(k)
                                                       for a, b in zip(cids, ids[:sample])]))}
    algo = passes * bpp
    achieved = algo / (kms * 1e-3) / 1e9
    roof = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": None, "kernel": "flat_scan_kernel<fp32, l2, T=%d>" % tile, "kernel_ms": kms,
            "algorithmic_bytes_per_launch": algo, "flops_per_launch": 2.0 * n * d * nq,
            "tflops": 2.0 * n * d * nq / (kms * 1e-3) / 1e12}
    if tile >= 64:
        # The timed kernel is the last level of the contraction: bpp bytes of fp32 codes against every query.
        codes = bpp / (4.0 * d)
        tf = 2.0 * codes * d * nq / (kms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": tf, "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": tf / MFMA_F32_PEAK_TFLOPS,
                # rocprofv3 --pmc FETCH_SIZE (x 2.00) + WRITE_SIZE of this launch: profiles/prefilter_fp32_c1.md
                "traffic": 87735.7 * 2.00 * 1024 + 23281.8 * 1024 if (n, d, nq, k) == (100000, 128, 1000, 10) else None,
                "kernel": "prefilter_kernel<fp32> (fp32 MFMA, last level)", "kernel_ms": kms,
                "flops_per_launch": 2.0 * codes * d * nq, "codes_per_launch": codes}
    return env.base_line("QPS @ recall@10 (100k x 128 fp32 brute force)", "queries/s", nq / sec, sec, "f32",
                         "configs[0]: brute_force fp32 L2, N=%d, d=%d, %d queries, k=%d" % (n, d, nq, k),
                         {"recall_at_10": rec, "query_tile": tile, "passes_per_step": passes, "bytes_per_pass": bpp},
                         roof, cpu)


# ------------------------------------------------------------------------------------------- C3
def run_c3(env):
    args, capi, lib = env.args, env.capi, env.lib
    n, d, k, iters = args.n or 1000000, args.dim or 960, args.nlist or 4096, 10
    means = mt(315).standard_normal((k, d), dtype=np.float32)
    x_dev = env.buf(n * d * 4)
    pick = np.sort(mt(7).choice(n, k, replace=False))  # seeded random-sample initial centroids
    init = np.empty((k, d), np.float32)
    sample_rows = []
    t0 = time.time()
    for s, blk in mixture_chunks(47, n, d, means, 0.2, step=1 << 15):
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
        lo, hi = np.searchsorted(pick, [s, s + blk.shape[0]])
        init[lo:hi] = blk[pick[lo:hi] - s]
        if s < (1 << 18):
            sample_rows.append(blk.copy())  # the first 262 144 rows stay on the host for the CPU legs
    t_gen = time.time() - t0
    cent = env.upload(init)
    labels, loss = env.buf(n * 4), env.buf(8)
    wsb = lib.vsag_amd_kmeans_assign_workspace_bytes(n, d, k)
    ws = env.buf(wsb)

    def step():
        capi.check(lib.vsag_amd_kmeans_assign(x_dev.ptr, n, d, cent.ptr, k, labels.ptr, None, loss.ptr, ws.ptr, wsb,
                                              None))
    sec, kms = env.timed(step, args.steps, args.warmup)
    ws_a, wsb_a = ws, wsb
    # the full Lloyd run: 10 iterations from the same initial centroids
    cent2 = env.upload(init)
    wsb = lib.vsag_amd_kmeans_run_workspace_bytes(n, d, k)
    ws = env.buf(wsb)
    final = C.c_double()
    t0 = time.perf_counter()
    capi.check(lib.vsag_amd_kmeans_run(x_dev.ptr, n, d, cent2.ptr, k, iters, 7, labels.ptr, C.byref(final), ws.ptr, wsb,
                                       None))
    t_run = time.perf_counter() - t0
    cpu = None
    inertia = None
    if not args.no_cpu:
        import oracle as orc
        threads = min(os.cpu_count() or 1, 16)
        orc.set_threads(threads)
        # (1) Assignment as the reference does it (find_nearest_one_with_blas): SGEMM per 65 536-row chunk through the
        # OpenBLAS that numpy links, + |c|^2, first minimum, loss in double.  Timed on the first rows of the workload.
        xs = np.concatenate(sample_rows)
        cpu_assign_sgemm(xs[:4096], init, threads)  # BLAS thread pool and page warm-up
        t0 = time.perf_counter()
        ol, oloss = cpu_assign_sgemm(xs, init, threads)
        t_cpu = time.perf_counter() - t0
        step()
        capi.synchronize()
        glabels = labels.to_numpy(np.int32, (n,))[:xs.shape[0]]
        sl, _, _ = orc.kmeans_assign(xs[:1024], init)  # the scalar restatement on a few rows, for the record
        cpu = {"value": xs.shape[0] / t_cpu, "unit": "rows/s", "cores": threads, "kind": "port",
               "blas": blas_name(),
               "sample": "first %d of the %d rows against all %d centroids; find_nearest_one_with_blas restated with "
                         "its own steps: chunks of 65 536 rows, -2 C X^T by SGEMM (%s through numpy, %d threads), + |c|^2, "
                         "std::min_element per row in blocks of 1024 rows on %d threads, loss in double" %
                         (xs.shape[0], n, k, blas_name(), threads, threads),
               "label_agreement_with_gpu": float((ol == glabels).mean()),
               "label_agreement_sgemm_vs_scalar_restatement": float((ol[:1024] == sl).mean())}
        # (2) Final inertia against the CPU: ten Lloyd iterations by both sides on one slice of the workload (its
        # first 65 536 rows), from the same initial centroids (a seeded sample of the slice) and with the same
        # re-seeding of empty clusters; the CPU side assigns through SGEMM as above.
        ns = min(n, xs.shape[0], 65536)
        xsl = np.ascontiguousarray(xs[:ns])
        init_s = xsl[np.sort(mt(7).choice(ns, k, replace=False))].copy()
        xs_dev, cs_dev = env.upload(xsl), env.upload(init_s)
        ls_dev = env.buf(ns * 4)
        wsb_s = lib.vsag_amd_kmeans_run_workspace_bytes(ns, d, k)
        ws_s = env.buf(wsb_s)
        g_loss = C.c_double()
        capi.check(lib.vsag_amd_kmeans_run(xs_dev.ptr, ns, d, cs_dev.ptr, k, iters, 7, ls_dev.ptr, C.byref(g_loss),
                                           ws_s.ptr, wsb_s, None))
        g_lab = ls_dev.to_numpy(np.int32, (ns,))
        g_cent = cs_dev.to_numpy(np.float32, (k, d))
        t0 = time.perf_counter()
        c_cent, c_lab, c_loss = orc.kmeans_run_with(xsl, init_s, iters, 7,
                                                    lambda cc: cpu_assign_sgemm(xsl, np.array(cc), threads))
        t_lloyd_cpu = time.perf_counter() - t0
        # inertia of the final centroids (after the tenth update), by one more SGEMM assignment of the slice
        _, g_final = cpu_assign_sgemm(xsl, g_cent, threads)
        _, c_final = cpu_assign_sgemm(xsl, c_cent, threads)
        inertia = {"slice_rows": int(ns), "iterations": iters,
                   "gpu_loss_of_last_assignment": g_loss.value, "cpu_loss_of_last_assignment": float(c_loss),
                   "relative_difference": abs(g_loss.value - c_loss) / abs(c_loss),
                   "gpu_inertia_of_final_centroids": float(g_final), "cpu_inertia_of_final_centroids": float(c_final),
                   "relative_difference_final": abs(g_final - c_final) / abs(c_final),
                   "label_agreement_after_10_iterations": float((g_lab == c_lab).mean()),
                   "cpu_lloyd_seconds": t_lloyd_cpu,
                   "gpu_all_rows_loss_after_10_iterations": final.value,
                   "what": "KMeansCluster::Run restated (SGEMM assignment, mean update, empty clusters re-seeded from "
                           "mt19937(7)) on the CPU against vsag_amd_kmeans_run on the same %d x %d slice" % (ns, d)}
        for b in (xs_dev, cs_dev, ls_dev, ws_s):
            b.free()
    flops = 2.0 * n * k * d
    tf = flops / (kms * 1e-3) / 1e12
    roof = {"bound": "mfma", "achieved": tf, "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": tf / MFMA_F32_PEAK_TFLOPS,
            # rocprofv3 --pmc FETCH_SIZE (x 2.00) + WRITE_SIZE of one launch: profiles/kmeans_assign_c3.md.  Above the
            # 3.9 GB of inputs: an XCD's L2 holds the k-slices of one macro tile (1024 rows x 2048 centroids) at a time.
            "traffic": 11786276.4 * 2.00 * 1024 + 2125360.1 * 1024 if (n, d, k) == (1000000, 960, 4096) else None,
            "kernel": "kmeans_assign_tile_kernel<4>" if d % 4 == 0 and k > 384 else
                      "kmeans_assign_tile_kernel<2>" if d % 4 == 0 else "kmeans_assign_kernel", "kernel_ms": kms,
            "flops_per_launch": flops}
    return env.base_line("k-means assign rows/s", "rows/s", n / sec, sec, "f32",
                         "configs[2]: k-means assignment, N=%d, d=%d, k=%d (one step = one assignment pass)" % (n, d, k),
                         {"lloyd_iterations": iters, "lloyd_seconds": t_run, "final_loss": final.value,
                          "final_inertia_vs_cpu": inertia, "datagen_seconds": t_gen}, roof, cpu)


# ------------------------------------------------------------------------------------------- C4
def run_c4(env):
    args, capi, lib = env.args, env.capi, env.lib
    n, d, nq, k = args.n or 10000000, args.dim or 128, args.nq or 10000, args.k
    nlist, nprobe, kcand = args.nlist or 4096, 64, 100
    # --list-codes sq8_uniform / sq8: the same search over lists of a byte per dimension (one range for all
    # dimensions / a range per dimension)
    bits = 4 if args.list_codes == "sq4_uniform" else 8
    per_dim = args.list_codes == "sq8"
    one_bit = args.list_codes == "rabitq"  # 1-bit codes, 4-bit queries, a seeded random rotation
    pqfs = args.list_codes == "pqfs"       # 4-bit product quantization, --pq-dim subspaces (default: one per dimension)
    raw32 = args.list_codes == "fp32"      # the reference's default ivf codec: the vectors themselves
    pq_dim = (args.pq_dim or d) if pqfs else 0
    kind = (capi.KIND_FP32 if raw32 else capi.KIND_PQFS if pqfs else capi.KIND_RABITQ if one_bit else capi.KIND_SQ8 if per_dim
            else capi.KIND_SQ8_UNIFORM if bits == 8 else capi.KIND_SQ4_UNIFORM)
    kind_name = args.list_codes
    means = mt(315).random((10000, d), dtype=np.float32)
    x_dev = env.buf(n * d * 4)
    pick = np.sort(mt(7).choice(n, nlist, replace=False))
    init = np.empty((nlist, d), np.float32)
    for s, blk in mixture_chunks(47, n, d, means, 0.05):
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
        lo, hi = np.searchsorted(pick, [s, s + blk.shape[0]])
        init[lo:hi] = blk[pick[lo:hi] - s]
    q, _ = mixture(315, 165, nq, d, 10000, 0.05, means=means)
    t0 = time.perf_counter()
    # train on a sample (the first 262144 rows), assign everything, encode, build the lists
    ns = min(n, 64 * nlist)
    cent = env.upload(init)
    slabels = env.buf(ns * 4)
    wsb = lib.vsag_amd_kmeans_run_workspace_bytes(ns, d, nlist)
    ws = env.buf(wsb)
    capi.check(lib.vsag_amd_kmeans_run(x_dev.ptr, ns, d, cent.ptr, nlist, 10, 7, slabels.ptr, None, ws.ptr, wsb, None))
    ws.free()
    labels = env.buf(n * 4)
    wsb = lib.vsag_amd_kmeans_assign_workspace_bytes(n, d, nlist)
    ws = env.buf(wsb)
    capi.check(lib.vsag_amd_kmeans_assign(x_dev.ptr, n, d, cent.ptr, nlist, labels.ptr, None, None, ws.ptr, wsb, None))
    ws.free()
    bounds = env.buf(8)
    lb_dev, diff_dev = env.buf(d * 4), env.buf(d * 4)
    wsb = lib.vsag_amd_sq_train_workspace_bytes(ns, d, 0)
    ws = env.buf(wsb)
    cs = int(lib.vsag_amd_code_size(kind, capi.METRIC_L2, pq_dim if pqfs else d, 4 if one_bit else 0))
    codes = x_dev if raw32 else env.buf(n * cs)
    rot = None
    if raw32:
        lists = env.make_store(kind, capi.METRIC_L2, d)
    elif pqfs:
        cb_dev = env.buf(d * 16 * 4)
        wsp = lib.vsag_amd_pq_train_workspace_bytes(ns, d, pq_dim)
        wp = env.buf(wsp)
        capi.check(lib.vsag_amd_pq_train(x_dev.ptr, ns, d, pq_dim, capi.METRIC_L2, 11, cb_dev.ptr, wp.ptr, wsp, None))
        wp.free()
        capi.check(lib.vsag_amd_pq_encode(x_dev.ptr, n, d, pq_dim, cb_dev.ptr, capi.METRIC_L2, codes.ptr, None, None))
        lists = env.make_store(kind, capi.METRIC_L2, d, pq_dim=pq_dim, codebooks=cb_dev)
    elif one_bit:
        g = mt(316).standard_normal((d, d))
        rot, r = np.linalg.qr(g)
        rot = (rot * np.sign(np.diag(r))).astype(np.float32)
        rot_dev, cen_dev = env.upload(rot), env.buf(d * 4)
        capi.check(lib.vsag_amd_rabitq_train(x_dev.ptr, ns, d, rot_dev.ptr, cen_dev.ptr, None))
        capi.check(lib.vsag_amd_rabitq_encode(x_dev.ptr, n, d, rot_dev.ptr, cen_dev.ptr, capi.METRIC_L2, 4, codes.ptr, None))
        lists = env.make_store(kind, capi.METRIC_L2, d, rot=rot_dev, cen=cen_dev, qbits=4)
    elif per_dim:
        capi.check(lib.vsag_amd_sq_train(x_dev.ptr, ns, d, 8, capi.METRIC_L2, capi.SQ_TRAIN_TRUNC_BOUND, 0.05, 0,
                                         lb_dev.ptr, diff_dev.ptr, ws.ptr, wsb, None))
        capi.check(lib.vsag_amd_sq_encode(x_dev.ptr, n, d, 8, capi.METRIC_L2, lb_dev.ptr, diff_dev.ptr, codes.ptr, None))
        lists = env.make_store(kind, capi.METRIC_L2, d, lb=lb_dev, diff=diff_dev)
    else:
        capi.check(lib.vsag_amd_sq_train_uniform(x_dev.ptr, ns, d, bits, capi.METRIC_L2, capi.SQ_TRAIN_TRUNC_BOUND, 0.05,
                                                 0, bounds.ptr, ws.ptr, wsb, None))
        capi.check(lib.vsag_amd_squ_encode(x_dev.ptr, n, d, bits, capi.METRIC_L2, bounds.ptr, codes.ptr, None))
        lists = env.make_store(kind, capi.METRIC_L2, d, bounds=bounds)
    ws.free()
    capi.check(lib.vsag_amd_store_set_lists(lists, codes.ptr, labels.ptr, n, nlist, None))
    cstore = env.make_store(capi.KIND_FP32, capi.METRIC_L2, d)
    capi.check(lib.vsag_amd_store_append(cstore, cent.ptr, nlist, None))
    capi.synchronize()
    t_build = time.perf_counter() - t0
    sizes = np.zeros(nlist, np.uint32)
    capi.check(lib.vsag_amd_store_list_sizes(lists, sizes.ctypes.data, nlist))

    q_dev = env.upload(q)
    buckets, bd = env.buf(nq * nprobe * 4), env.buf(nq * nprobe * 4)
    cand, cand_d = env.buf(nq * kcand * 4), env.buf(nq * kcand * 4)
    out_i, out_d = env.buf(nq * k * 4), env.buf(nq * k * 4)
    wr = lib.vsag_amd_ivf_route_workspace_bytes(cstore, nq, nprobe)
    wsc = lib.vsag_amd_ivf_scan_workspace_bytes(lists, nq, nprobe, kcand)
    ws = env.buf(max(wr, wsc))

    def step():
        capi.check(lib.vsag_amd_ivf_route(cstore, q_dev.ptr, nq, nprobe, buckets.ptr, bd.ptr, ws.ptr, wr, None))
        capi.check(lib.vsag_amd_ivf_scan_topk(lists, q_dev.ptr, nq, buckets.ptr, nprobe, kcand, cand.ptr, cand_d.ptr,
                                              ws.ptr, wsc, None))
        capi.check(lib.vsag_amd_rerank_fp32(x_dev.ptr, n, d, capi.METRIC_L2, q_dev.ptr, nq, cand.ptr, kcand, k,
                                            out_i.ptr, out_d.ptr, None))
    # one query per call (the reference's own call pattern): route + scan of 64 lists + rerank, synchronised per query
    single = None
    if not args.no_single:
        t_one = []
        for i in range(5 + 50):
            qp = q_dev.ptr + (i % nq) * d * 4
            t0 = time.perf_counter()
            capi.check(lib.vsag_amd_ivf_route(cstore, qp, 1, nprobe, buckets.ptr, bd.ptr, ws.ptr, wr, None))
            capi.check(lib.vsag_amd_ivf_scan_topk(lists, qp, 1, buckets.ptr, nprobe, kcand, cand.ptr, cand_d.ptr, ws.ptr,
                                                  wsc, None))
            capi.check(lib.vsag_amd_rerank_fp32(x_dev.ptr, n, d, capi.METRIC_L2, qp, 1, cand.ptr, kcand, k, out_i.ptr,
                                                out_d.ptr, None))
            capi.synchronize()
            if i >= 5:
                t_one.append(time.perf_counter() - t0)
        single = {"latency_us": 1e6 * float(np.mean(t_one)), "queries_per_second_one_at_a_time": 1.0 / float(np.mean(t_one))}
    sec, kms = env.timed(step, args.steps, args.warmup)
    tile = C.c_int()
    lib.vsag_amd_last_scan_info(C.byref(tile), None, None)  # 256: the int8 matrix cores took columns 1..nprobe-1
    ids = out_i.to_numpy(np.uint32, (nq, k))
    b = buckets.to_numpy(np.int32, (nq, nprobe))
    scanned = sizes[b.clip(0)].astype(np.int64).sum()  # codes scanned per step, summed over queries
    algo = float(scanned) * (cs + 4)
    rec = None
    gt_ids = None
    if not args.no_recall:
        # exact fp32 ground truth from the library's own fp32 flat scan (checked against the CPU checker in tests)
        flat = env.make_store(capi.KIND_FP32, capi.METRIC_L2, d)
        capi.check(lib.vsag_amd_store_append(flat, x_dev.ptr, n, None))
        nrec = min(nq, 1000)
        gi, gd = env.buf(nrec * k * 4), env.buf(nrec * k * 4)
        st, w2 = env.flat_scan_fn(flat, q_dev, nrec, k, gi, gd)
        st()
        gt_ids = gi.to_numpy(np.uint32, (nrec, k))
        rec = recall_at_k(ids[:nrec], gt_ids)
        w2.free()
    cpu = None
    if not args.no_cpu:
        # CPU restatement of IVF::search + reorder on a sample of the same queries, routing injected (the GPU's
        # exact routing), same codes and lists: candidates, reranked ids and recall must agree.
        import oracle as orc
        threads = min(os.cpu_count() or 1, 16)
        sample = min(nq, 64 * threads)
        hcodes = codes.to_numpy(np.uint8, (n, cs))
        hlabels = labels.to_numpy(np.int32, (n,))
        offsets, order = orc.ivf_build_lists(hlabels, nlist)
        posting = hcodes[order]
        od = d
        if raw32:
            hb = (None, None)
            okind, qcodes = orc.FP32, q[:sample]
        elif pqfs:
            hb = (None, None)
            okind, od = orc.PQFS, pq_dim
            qcodes = orc.pqfs_process_query(q[:sample], pq_dim, cb_dev.to_numpy(np.float32, (pq_dim, 16, d // pq_dim)), orc.L2)
        elif one_bit:
            hb = (None, None)
            okind = orc.RABITQ
            qcodes = orc.rabitq_process_query(q[:sample], rot, cen_dev.to_numpy(np.float32, (d,)), orc.L2)
        elif per_dim:
            hb = (lb_dev.to_numpy(np.float32, (d,)), diff_dev.to_numpy(np.float32, (d,)))
            okind, qcodes = orc.SQ8, q[:sample]
        else:
            hb = bounds.to_numpy(np.float32, (2,))
            okind = orc.SQ8U if bits == 8 else orc.SQ4U
            qcodes = orc.squ_encode(q[:sample], bits, hb[0], hb[1], orc.L2)
        ref = orc.use_reference_kernels(orc.ref_best_isa())
        ref_name = {orc.SQ4U: "SQ4UniformComputeCodesIP", orc.SQ8U: "SQ8UniformComputeCodesIP",
                    orc.RABITQ: "RaBitQSQ4UBinaryIP", orc.FP32: "FP32ComputeL2Sqr"}.get(okind)
        ref = ref if ref and ref_name in ref else None
        orc.ivf_scan(okind, orc.L2, od, posting, offsets, order, qcodes[:threads], b[:threads], kcand,
                     lb=hb[0], diff=hb[1], threads=threads)
        t0 = time.perf_counter()
        cids, cds = orc.ivf_scan(okind, orc.L2, od, posting, offsets, order, qcodes, b[:sample], kcand,
                                 lb=hb[0], diff=hb[1], threads=threads)
        t_cpu = time.perf_counter() - t0
        orc.use_reference_kernels(None)
        gcand = cand.to_numpy(np.uint32, (nq, kcand))[:sample]
        gcd = cand_d.to_numpy(np.float32, (nq, kcand))[:sample]
        uniq = np.unique(cids[cids != 0xFFFFFFFF])
        raw = device_rows(env, x_dev, uniq, d)
        pos = {int(v): i for i, v in enumerate(uniq)}
        rids = np.empty((sample, k), np.uint32)
        for i in range(sample):
            rows = raw[[pos[int(v)] for v in cids[i]]]
            dd = ((rows.astype(np.float64) - q[i].astype(np.float64)) ** 2).sum(1)
            rids[i] = cids[i][np.lexsort((cids[i], dd))[:k]]
        cpu = {"value": sample / t_cpu, "unit": "queries/s", "cores": threads, "kind": "reference" if ref else "port",
               "sample": "%d of the %d queries, one query per call, OpenMP dynamic over queries; restated IVF::search "
                         "(scan of the same %d probed lists per query with the strict-< heap) on the same %s codes, lists "
                         "and routing; distance kernel = %s; rerank in fp64 on the host (not timed)" %
                         (sample, nq, nprobe, kind_name, (ref[ref_name] + " compiled from the reference sources") if ref
                          else "CPU restatement"),
               "candidate_distances_bit_equal": bool(np.array_equal(cds.view(np.uint32), gcd.view(np.uint32))),
               "candidate_distances_max_abs_difference": float(np.abs(cds.astype(np.float64) - gcd).max()),
               "candidate_overlap_with_gpu": float(np.mean([len(set(a) & set(bb)) / float(kcand)
                                                            for a, bb in zip(cids, gcand)])),
               "topk_overlap_with_gpu": float(np.mean([len(set(a) & set(bb)) / float(k)
                                                       for a, bb in zip(rids, ids[:sample])])),
               "recall_at_10": None if gt_ids is None else recall_at_k(rids, gt_ids[:sample]),
               "gpu_recall_at_10_same_queries": None if gt_ids is None else recall_at_k(ids[:sample], gt_ids[:sample])}
    if not raw32:
        codes.free()
    achieved = algo / (kms * 1e-3) / 1e9
    # One step launches the scan kernel twice (nearest list of every query first, then the other lists); kernel_ms,
    # the algorithmic bytes (76 B per (query, scanned code), the reference's per-query list reads) and the traffic
    # are the sums over both launches.  Traffic: rocprofv3 --pmc FETCH_SIZE (x 2.00) + WRITE_SIZE of this exact
    # configuration, profiles/ivf_scan_sq4u_c4.md.  Work items that share a list are co-scheduled and read it
    # through L2 once per <= 4 queries, so the fraction against HBM exceeds 1: this kernel is bound by VALU issue.
    traffic = None
    if (n, d, nq, k, nlist, bits) == (10000000, 128, 10000, 10, 4096, 4) and tile.value != 256:
        traffic = (482513.06 + 1698762.06) * 2.00 * 1024 + (9817.03 + 19915.53) * 1024
    roof = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic, "kernel": "ivf_scan_kernel<%s, l2> (2 launches per step)" % kind_name, "kernel_ms": kms,
            "algorithmic_bytes_per_launch": algo,
            "distance_evaluations_per_second": float(scanned) / (kms * 1e-3)}
    if tile.value == 256:
        # The probe columns behind the first went through the int8 matrix cores; the timed kernel is that pass alone:
        # every code of those lists against every query probing them, 2 x 128 integer operations per pair.
        rest = sizes[b[:, 1:].clip(0)].astype(np.int64).sum() - (b[:, 1:] < 0).sum() * int(sizes[0])
        # (pqfs: a pair is a contraction of the one-hot centroid indices with the byte table, 16 products per subspace)
        ops = 2.0 * (16 * (-(-pq_dim // 32) * 32) if pqfs else -(-d // 32) * 32) * float(rest)
        tops = ops / (kms * 1e-3) / 1e12
        # (sq8 lists beyond 128 dimensions: the fp16 matrix cores, unless --contraction 2 keeps the fp32 ones)
        h16 = per_dim and d > 128 and bits == 8 and args.contraction != 2
        peak = (MFMA_F16_PEAK_TFLOPS if h16 else MFMA_F32_PEAK_TFLOPS if raw32 or (per_dim and d > 128) else
                MFMA_F6F4_PEAK_TFLOPS if one_bit else MFMA_I8_PEAK_TOPS)
        roof = {"bound": "mfma", "achieved": tops, "peak": peak, "unit": "TOP/s" if peak == MFMA_I8_PEAK_TOPS else "TFLOP/s",
                "frac": tops / peak,
                # rocprofv3 --pmc FETCH_SIZE (x 2.00) + WRITE_SIZE of this launch: profiles/ivf_i8_sq4u_c4.md
                "traffic": 491061.0 * 2.00 * 1024 + 73550.7 * 1024
                if (n, d, nq, k, nlist, bits) == (10000000, 128, 10000, 10, 4096, 4) else None,
                "kernel": "%s<%s> (%s MFMA, probe columns 1..%d)" % ("ivf_h16_kernel" if h16 else
                                                                        "ivf_f32_kernel" if peak == MFMA_F32_PEAK_TFLOPS else
                                                                        "ivf_pq_kernel" if pqfs else
                                                                        "prefilter_rb_kernel<lists>" if one_bit else
                                                                        "ivf_sq8_i8_kernel" if per_dim else "ivf_i8_kernel",
                                                                        kind_name, "fp16" if h16 else
                                                                        "fp32" if peak == MFMA_F32_PEAK_TFLOPS else
                                                                        "fp4 x fp6" if one_bit else "int8",
                                                                        nprobe - 1), "kernel_ms": kms,
                "ops_per_launch": ops, "distance_evaluations_per_launch": float(rest),
                "distance_evaluations_per_second": float(rest) / (kms * 1e-3)}
    return env.base_line("QPS @ recall@10 (IVF %s, %s x %d)" % ({"sq4_uniform": "SQ4-uniform", "sq8_uniform": "SQ8-uniform",
                                                                "sq8": "SQ8", "rabitq": "RaBitQ", "pqfs": "PQFS",
                                                                "fp32": "FP32"}[kind_name],
                                                               "%dM" % (n // 1000000) if n % 1000000 == 0 else str(n), d),
                         "queries/s", nq / sec, sec, "f32" if raw32 else "4-bit pq codes, u8 table sums in i32" if pqfs else
                         "1-bit codes x u4 queries, i32 popcount sums, f32 estimator" if one_bit else
                         "u8 codes x f32 scale, f32 (pre-selection: i8 x i8, i32 sums)" if per_dim else "u%d codes, i32 dot" % bits,
                         "configs[3]%s: IVF search, N=%d, d=%d, nlist=%d, nprobe=%d, rerank %d, %d queries, k=%d"
                         % ("" if bits == 4 else " with %s lists" % kind_name, n, d, nlist, nprobe, kcand, nq, k),
                         {"recall_at_10": rec, "build_seconds": t_build, "scanned_codes_per_query": float(scanned) / nq,
                          "bytes_per_scanned_code": cs + 4, "single_query": single,
                          "list_sizes": {"mean": float(sizes.mean()), "max": int(sizes.max()), "min": int(sizes.min()),
                                         "p99": float(np.percentile(sizes, 99))},
                          "queries_per_first_list": {"max": int(np.bincount(b[:, 0].clip(0), minlength=nlist).max()),
                                                     "mean": float(nq) / nlist}}, roof, cpu)


# ------------------------------------------------------------------------------------------- C5
def run_c5(env):
    args, capi, lib = env.args, env.capi, env.lib
    n, d, nq, k, kcand = args.n or 5000000, args.dim or 768, args.nq or 10000, args.k, 200
    x_dev = env.buf(n * d * 4)
    rng = mt(47)
    step_rows = 1 << 15
    for s in range(0, n, step_rows):
        blk = rng.standard_normal((min(step_rows, n - s), d), dtype=np.float32)
        blk /= np.linalg.norm(blk, axis=1, keepdims=True)
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
    q = mt(165).standard_normal((nq, d), dtype=np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    g = mt(315).standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)  # seeded Gaussian -> QR, passed to CPU and GPU alike
    t0 = time.perf_counter()
    rot_dev = env.upload(rot)
    cen = env.buf(d * 4)
    capi.check(lib.vsag_amd_rabitq_train(x_dev.ptr, n, d, rot_dev.ptr, cen.ptr, None))
    cs = int(lib.vsag_amd_code_size(capi.KIND_RABITQ, capi.METRIC_IP, d, 4))
    codes = env.buf(n * cs)
    capi.check(lib.vsag_amd_rabitq_encode(x_dev.ptr, n, d, rot_dev.ptr, cen.ptr, capi.METRIC_IP, 4, codes.ptr, None))
    store = env.make_store(capi.KIND_RABITQ, capi.METRIC_IP, d, rot=rot_dev, cen=cen, qbits=4)
    capi.check(lib.vsag_amd_store_append(store, codes.ptr, n, None))
    capi.synchronize()
    t_build = time.perf_counter() - t0
    q_dev = env.upload(q)
    cand, cand_d = env.buf(nq * kcand * 4), env.buf(nq * kcand * 4)
    out_i, out_d = env.buf(nq * k * 4), env.buf(nq * k * 4)
    capi.check(lib.vsag_amd_set_scan_tuning(args.tile, args.chunks))
    scan, ws = env.flat_scan_fn(store, q_dev, nq, kcand, cand, cand_d)

    def step():
        scan()
        capi.check(lib.vsag_amd_rerank_fp32(x_dev.ptr, n, d, capi.METRIC_IP, q_dev.ptr, nq, cand.ptr, kcand, k,
                                            out_i.ptr, out_d.ptr, None))
    sec, kms = env.timed(step, args.steps, args.warmup)
    tile, passes, bpp = env.scan_info()
    ids = out_i.to_numpy(np.uint32, (nq, k))
    rec = None
    gt_ids = None
    if not args.no_recall:
        flat = env.make_store(capi.KIND_FP32, capi.METRIC_IP, d)
        capi.check(lib.vsag_amd_store_append(flat, x_dev.ptr, n, None))
        nrec = min(nq, 500)
        gi, gd = env.buf(nrec * k * 4), env.buf(nrec * k * 4)
        st, w2 = env.flat_scan_fn(flat, q_dev, nrec, k, gi, gd)
        st()
        gt_ids = gi.to_numpy(np.uint32, (nrec, k))
        rec = recall_at_k(ids[:nrec], gt_ids)
        w2.free()
    cpu = None
    if not args.no_cpu:
        # CPU restatement of the RaBitQ scan (ProcessQueryImpl + ComputeQueryBaseImpl + heap) on a sample of the same
        # queries against the same codes, then fp64 rerank of its 200 candidates.
        import oracle as orc
        threads = min(os.cpu_count() or 1, 16)
        sample = min(nq, 8 * threads)
        hcodes = codes.to_numpy(np.uint8, (n, cs))
        hcen = cen.to_numpy(np.float32, (d,))
        qcodes = orc.rabitq_process_query(q[:sample], rot, hcen, orc.IP, 4)
        ref = orc.use_reference_kernels(orc.ref_best_isa())
        ref = ref if ref and "RaBitQSQ4UBinaryIP" in ref else None
        t0 = time.perf_counter()
        cids, cds = orc.flat_scan_topk(orc.RABITQ, orc.IP, d, hcodes, qcodes, kcand, qbits=4, threads=threads)
        t_cpu = time.perf_counter() - t0
        orc.use_reference_kernels(None)
        gcand = cand.to_numpy(np.uint32, (nq, kcand))[:sample]
        uniq = np.unique(cids)
        raw = device_rows(env, x_dev, uniq, d)
        pos = {int(v): i for i, v in enumerate(uniq)}
        rids = np.empty((sample, k), np.uint32)
        for i in range(sample):
            rows = raw[[pos[int(v)] for v in cids[i]]]
            dd = 1.0 - rows.astype(np.float64) @ q[i].astype(np.float64)
            rids[i] = cids[i][np.lexsort((cids[i], dd))[:k]]
        cpu = {"value": sample / t_cpu, "unit": "queries/s", "cores": threads, "kind": "reference" if ref else "port",
               "sample": "%d of the %d queries over all %d codes, one query per call, OpenMP dynamic over queries; restated "
                         "RaBitQuantizer::ComputeQueryBaseImpl + BruteForce heap, popcount kernel = %s; rerank in fp64 on "
                         "the host (not timed)" %
                         (sample, nq, n, (ref["RaBitQSQ4UBinaryIP"] + " compiled from the reference sources") if ref
                          else "CPU restatement"),
               "candidate_overlap_with_gpu": float(np.mean([len(set(a) & set(bb)) / float(kcand)
                                                            for a, bb in zip(cids, gcand)])),
               "topk_overlap_with_gpu": float(np.mean([len(set(a) & set(bb)) / float(k)
                                                       for a, bb in zip(rids, ids[:sample])])),
               "recall_at_10": None if gt_ids is None else recall_at_k(rids, gt_ids[:sample]),
               "gpu_recall_at_10_same_queries": None if gt_ids is None else recall_at_k(ids[:sample], gt_ids[:sample])}
    codes.free()
    algo = passes * n * float(cs)
    achieved = algo / (kms * 1e-3) / 1e9
    # rocprofv3 --pmc FETCH_SIZE (x 2.00) + WRITE_SIZE of this exact configuration, profiles/flat_scan_rabitq_c5.md
    traffic = None
    if (n, d, nq, k, tile) == (5000000, 768, 10000, 10, 2):
        traffic = 1142603761.9 * 2.00 * 1024 + 242555.2 * 1024
    roof = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic, "kernel": "flat_scan_kernel<rabitq, ip, T=%d>" % tile, "kernel_ms": kms,
            "algorithmic_bytes_per_launch": algo}
    dtype = "1-bit codes x 4-bit queries, u32 popcount"
    if tile >= 64:
        # The batch was pre-selected on the matrix cores (1-bit codes as fp4, 4-bit queries as fp6, exact sums in
        # fp32) and the survivors rescored with the popcount arithmetic.  The timed kernel is the last level: bpp
        # bytes of d / 8-byte codes against every query.
        lcodes = bpp / (d / 8.0)
        ops = 2.0 * lcodes * d * nq
        tops = ops / (kms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": tops, "peak": MFMA_F6F4_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": tops / MFMA_F6F4_PEAK_TFLOPS,
                # rocprofv3 --pmc FETCH_SIZE (x 2.00) + WRITE_SIZE of this launch: profiles/prefilter_rb_rabitq_c5.md
                "traffic": 951461.0 * 2.00 * 1024 + 218608.0 * 1024 if (n, d, nq, k) == (5000000, 768, 10000, 10) else None,
                "kernel": "prefilter_rb_kernel<ip> (fp4 x fp6 MFMA, last level)", "kernel_ms": kms, "ops_per_launch": ops,
                "codes_per_launch": lcodes}
        dtype = "1-bit codes x 4-bit queries: fp4 x fp6 MFMA pre-selection (exact fp32 sums), u32 popcount rescoring"
    return env.base_line("QPS @ recall@10 (RaBitQ 1-bit scan + rerank 200, 5M x 768)", "queries/s", nq / sec, sec,
                         dtype,
                         "configs[4]: RaBitQ full scan + fp32 rerank of %d, N=%d, d=%d, %d queries, k=%d, IP" %
                         (kcand, n, d, nq, k),
                         {"recall_at_10": rec, "build_seconds": t_build, "query_tile": tile, "passes_per_step": passes,
                          "bytes_per_code": cs}, roof, cpu)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--n", type=int, default=0)
    ap.add_argument("--dim", type=int, default=0)
    ap.add_argument("--nq", type=int, default=0)
    ap.add_argument("--nlist", type=int, default=0)
    ap.add_argument("--k", type=int, default=10)
    ap.add_argument("--tile", type=int, default=0, help="query tile override (0 = library default)")
    ap.add_argument("--chunks", type=int, default=0, help="base chunk override (0 = library default)")
    ap.add_argument("--contraction", type=int, default=0, choices=[-1, 0, 1, 2],
                    help="matrix-core path of the flat scans: -1 never, 0 library default, 1 whenever supported, 2 the fp32 matrix cores only")
    ap.add_argument("--list-codes", default="sq4_uniform", choices=["sq4_uniform", "sq8_uniform", "sq8", "rabitq", "pqfs", "fp32"],
                    help="c4 only: the quantizer of the posting lists (configs[3] names sq4_uniform)")
    ap.add_argument("--pq-dim", type=int, default=0, help="c4 with --list-codes pqfs: subspaces (default: the dimension)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-recall", action="store_true", help="skip the recall check")
    ap.add_argument("--no-single", action="store_true", help="skip the one-query-per-call measurement")
    ap.add_argument("--no-api", action="store_true", help="skip the index-API leg (host buffers on both sides)")
    ap.add_argument("--no-kmeans", action="store_true", help="default line only: skip the k-means block (configs[2])")
    ap.add_argument("--only", action="store_true", help="--config c2 alone, without the blocks of the other configurations")
    ap.add_argument("--skip", default="", help="default line only: blocks to leave out, e.g. c4,c5")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the search core is single-GPU by design (sharding it means splitting "
              "the base rows or posting lists and merging nq x k results); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    env = Env(args)
    env.capi.check(env.lib.vsag_amd_set_scan_contraction(args.contraction))
    runs = {"c1": run_c1, "c2": run_c2, "c3": run_c3, "c4": run_c4, "c5": run_c5}
    line = runs[args.config](env)
    env.release()
    if args.config == "c2" and not args.only and not (args.n or args.dim or args.nq):
        # The default line carries all five configurations: configs[1] is the line itself (the headline metric), the
        # others are blocks of the same shape -- "kmeans" (configs[2], the metric's second figure), "c1" (configs[0]),
        # "c4" (configs[3]) and "c5" (configs[4]) -- each timed with the same --steps / --warmup, with its own roofline
        # and its own CPU baseline on a bounded sample.
        def block(cfg):
            env.capi.check(env.lib.vsag_amd_set_scan_tuning(0, 0))
            t0 = time.perf_counter()
            full = runs[cfg](env)
            env.release()
            c = full["config"]
            out = {"metric": full["metric"], "value": full["value"], "unit": full["unit"],
                   "ms_per_step": full["ms_per_step"], "steps": full["steps"], "warmup": full["warmup"],
                   "dtype": full["dtype"], "workload": c["workload"]}
            out.update({k: v for k, v in c.items() if k not in ("workload", "device", "compute_units")})
            out["roofline"] = full["roofline"]
            out["cpu_baseline"] = full["cpu_baseline"]
            out["block_wall_seconds"] = time.perf_counter() - t0
            return out
        if not args.no_kmeans:
            line["kmeans"] = block("c3")
        for cfg in ("c1", "c4", "c5"):
            if cfg not in args.skip:
                line[cfg] = block(cfg)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
