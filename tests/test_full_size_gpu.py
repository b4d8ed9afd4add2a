"""Parity at the full sizes of the five benchmark configurations, through the C ABI.

At these sizes the CPU checker can only afford a few queries (it is compared on those, on the same codes),
so each test adds properties that do not depend on size: the same result bit for bit whatever the query
tile / batch split, ascending distances, distinct in-range ids, exact fp64 recomputation on samples.
The data are the benchmark's own seeded generators.
"""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from bench import mixture, mixture_chunks, mt
from gpu_helpers import Store, assert_topk_close, dev
from vsag_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    lib = capi.load_library()
    capi.init(0)
    yield lib
    capi.check(lib.vsag_amd_set_scan_tuning(0, 0))


def check_result_shape(ids, dists, n):
    assert np.all(np.diff(dists.astype(np.float64), axis=1) >= 0), "distances must ascend"
    assert np.all(ids < n), "ids must be inner ids of the store"
    srt = np.sort(ids, axis=1)
    assert np.all(srt[:, 1:] != srt[:, :-1]), "ids of one query must be distinct"


def scan_with_tile(lib, store, queries, k, tile):
    """A flat scan with the store's own query-tile setting (process-wide settings stay untouched)."""
    capi.check(lib.vsag_amd_store_set_scan_tuning(store.handle, tile, -1))
    try:
        return store.flat_scan(queries, k)
    finally:
        capi.check(lib.vsag_amd_store_set_scan_tuning(store.handle, -1, -1))


def streaming_only(lib, store):
    """Context manager: the store's scans stay on the streaming kernels (its own setting, not the process-wide one)."""
    import contextlib

    @contextlib.contextmanager
    def cm():
        capi.check(lib.vsag_amd_store_set_scan_contraction(store.handle, -1))
        try:
            yield
        finally:
            capi.check(lib.vsag_amd_store_set_scan_contraction(store.handle, -2))
    return cm()


def test_fp32_bruteforce_100k(lib):
    """configs[0]: 100 000 x 128 uniform rows, 1000 queries, L2."""
    n, d, nq, k = 100000, 128, 1000, 10
    x = mt(47).random((n, d), dtype=np.float32)
    q = mt(165).random((nq, d), dtype=np.float32)
    store = Store(capi.KIND_FP32, capi.METRIC_L2, d)
    store.append(x.view(np.uint8).reshape(n, d * 4))
    ids, dists = store.flat_scan(q, k)
    check_result_shape(ids, dists, n)
    # exact fp64 distances of the returned ids, and no closer vector anywhere (fp64 scan of 64 queries)
    for i in range(0, nq, 16):
        dd = ((x.astype(np.float64) - q[i].astype(np.float64)) ** 2).sum(1)
        order = np.lexsort((np.arange(n), dd))[:k]
        assert np.array_equal(order, ids[i]), i
        np.testing.assert_allclose(dists[i], dd[order], rtol=1e-4)
    oi, od = orc.flat_scan_topk(orc.FP32, orc.L2, d, x.view(np.uint8).reshape(n, d * 4), q[:64], k)
    assert_topk_close(ids[:64], dists[:64], oi, od, label="fp32 100k")
    for tile in (1, 2):
        ti, td = scan_with_tile(lib, store, q[:128], k, tile)
        assert np.array_equal(ti, ids[:128]) and np.array_equal(td.view(np.uint32), dists[:128].view(np.uint32)), tile
    store.destroy()


@pytest.mark.parametrize("metric,ometric", [(capi.METRIC_L2, orc.L2), (capi.METRIC_IP, orc.IP)])
def test_sq8_scan_1m(lib, metric, ometric):
    """configs[1] at the benchmark's own batch: 1 000 000 x 128 mixture rows as SQ8 codes (trained and encoded on the
    device), all 10 000 queries in one call."""
    n, d, nq, k = 1000000, 128, 10000, 10
    x, means = mixture(315, 47, n, d, 1000, 0.05)
    q, _ = mixture(315, 165, nq, d, 1000, 0.05, means=means)
    x_dev = dev(x)
    lb_dev, diff_dev = capi.DeviceBuffer(d * 4), capi.DeviceBuffer(d * 4)
    wsb = lib.vsag_amd_sq_train_workspace_bytes(n, d, 0)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_sq_train(x_dev.ptr, n, d, 8, metric, capi.SQ_TRAIN_TRUNC_BOUND, 0.05, 0, lb_dev.ptr,
                                     diff_dev.ptr, ws.ptr, wsb, None))
    codes_dev = capi.DeviceBuffer(n * d)
    capi.check(lib.vsag_amd_sq_encode(x_dev.ptr, n, d, 8, metric, lb_dev.ptr, diff_dev.ptr, codes_dev.ptr, None))
    lb, diff = lb_dev.to_numpy(np.float32, (d,)), diff_dev.to_numpy(np.float32, (d,))
    codes = codes_dev.to_numpy(np.uint8, (n, d))
    for b in (x_dev, ws, codes_dev, lb_dev, diff_dev):
        b.free()
    # trained bounds and codes equal the checker's, bit for bit, at full size
    olb, odiff = orc.sq_train(x, 8, ometric)
    assert np.array_equal(lb.view(np.uint32), olb.view(np.uint32))
    assert np.array_equal(diff.view(np.uint32), odiff.view(np.uint32))
    assert np.array_equal(codes[::97], orc.sq_encode(x[::97], 8, lb, diff, ometric))

    store = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    store.append(codes)
    ids, dists = store.flat_scan(q, k)
    check_result_shape(ids, dists, n)
    oi, od = orc.flat_scan_topk(orc.SQ8, ometric, d, codes, q[:32], k, lb=lb, diff=diff)
    assert_topk_close(ids[:32], dists[:32], oi, od, label="sq8 1M")
    # the batch goes through the int8 matrix-core pre-selection (40 query groups, the XCD-grouped grid of the
    # benchmark); the streaming kernel alone must return the same bits for every one of the 10 000 queries
    info = capi.C.c_int()
    lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
    assert info.value == 256, "the int8 pre-selection did not run"
    with streaming_only(lib, store):
        si, sd = store.flat_scan(q, k)
        lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
        assert info.value <= 8
    assert np.array_equal(si, ids) and np.array_equal(sd.view(np.uint32), dists.view(np.uint32))
    # a smaller batch takes another grid (2 query groups): same bits again
    pi, pd = store.flat_scan(q[:512], k)
    assert np.array_equal(pi, ids[:512]) and np.array_equal(pd.view(np.uint32), dists[:512].view(np.uint32))
    # the same answer whatever the query tile, and one query per call (a different grid and cold start)
    for tile in (1, 2):
        ti, td = scan_with_tile(lib, store, q[:256], k, tile)
        assert np.array_equal(ti, ids[:256]) and np.array_equal(td.view(np.uint32), dists[:256].view(np.uint32)), tile
    for i in range(24):
        si, sd = store.flat_scan(q[i:i + 1], k)
        assert np.array_equal(si[0], ids[i]) and np.array_equal(sd[0].view(np.uint32), dists[i].view(np.uint32)), i
    store.destroy()


def test_kmeans_assign_1m_x_960(lib):
    """configs[2]: 1 000 000 x 960 rows against 4096 centroids (seeded random-sample initialisation)."""
    n, d, k = 1000000, 960, 4096
    means = mt(315).standard_normal((k, d), dtype=np.float32)
    x_dev = capi.DeviceBuffer(n * d * 4)
    pick = np.sort(mt(7).choice(n, k, replace=False))
    init = np.empty((k, d), np.float32)
    keep_rows, keep_idx = [], []
    for s, blk in mixture_chunks(47, n, d, means, 0.2, step=1 << 15):
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
        lo, hi = np.searchsorted(pick, [s, s + blk.shape[0]])
        init[lo:hi] = blk[pick[lo:hi] - s]
        keep_rows.append(blk[:64].copy())  # 64 rows of every chunk of 32768
        keep_idx.append(np.arange(s, s + 64))
    xs, idx = np.concatenate(keep_rows), np.concatenate(keep_idx)
    cent = dev(init)
    labels, mind, loss = capi.DeviceBuffer(n * 4), capi.DeviceBuffer(n * 4), capi.DeviceBuffer(8)
    wsb = lib.vsag_amd_kmeans_assign_workspace_bytes(n, d, k)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_kmeans_assign(x_dev.ptr, n, d, cent.ptr, k, labels.ptr, mind.ptr, loss.ptr, ws.ptr, wsb,
                                          None))
    gl = labels.to_numpy(np.int32, (n,))
    gm = mind.to_numpy(np.float32, (n,))
    gloss = loss.to_numpy(np.float64, (1,))[0]
    assert gl.min() >= 0 and gl.max() < k
    # the sampled rows against all centroids in fp64: same argmin except at near-ties below 1e-5 relative
    c64 = init.astype(np.float64)
    cn = (c64 ** 2).sum(1)
    x64 = xs.astype(np.float64)
    full = (x64 ** 2).sum(1)[:, None] - 2.0 * x64 @ c64.T + cn[None, :]
    best = full.argmin(1)
    differ = np.nonzero(best != gl[idx])[0]
    for r in differ:
        assert abs(full[r, gl[idx][r]] - full[r, best[r]]) <= 1e-5 * abs(full[r, best[r]]) + 1e-6, r
    assert differ.size <= xs.shape[0] // 100
    # the checker on the same sample (labels of a row do not depend on the other rows)
    ol, _, _ = orc.kmeans_assign(xs[:512], init)
    assert np.mean(ol == gl[idx][:512]) >= 0.995
    # min distance is reported without the row norm (as the reference keeps it); loss adds it back
    xn = (x64 ** 2).sum(1)
    np.testing.assert_allclose(gm[idx] + xn, full[np.arange(xs.shape[0]), gl[idx]], rtol=2e-4, atol=5e-2)
    # loss = mean over rows of (min + |x|^2); compare with the per-row outputs on the sample's scale
    assert np.isfinite(gloss) and gloss > 0
    sample_loss = float(np.mean(full[np.arange(xs.shape[0]), gl[idx]]))
    assert abs(gloss - sample_loss) <= 0.1 * sample_loss
    for b in (x_dev, cent, labels, mind, loss, ws):
        b.free()


def test_kmeans_lloyd_10_iterations_on_a_64k_slice(lib):
    """configs[2], the first 65 536 rows: ten Lloyd iterations from the seeded random-sample initialisation against
    the checker's KMeansCluster::Run restatement (same initial centroids, same re-seeding of empty clusters)."""
    n, d, k, iters = 65536, 960, 4096, 10
    means = mt(315).standard_normal((k, d), dtype=np.float32)
    x = np.empty((n, d), np.float32)
    for s, blk in mixture_chunks(47, n, d, means, 0.2, step=1 << 15):
        x[s:s + blk.shape[0]] = blk
    cent0 = x[np.sort(mt(7).choice(n, k, replace=False))].copy()
    xb, cb = dev(x), dev(cent0)
    labels = capi.DeviceBuffer(n * 4)
    loss = C.c_double()
    wsb = lib.vsag_amd_kmeans_run_workspace_bytes(n, d, k)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_kmeans_run(xb.ptr, n, d, cb.ptr, k, iters, 7, labels.ptr, C.byref(loss), ws.ptr, wsb, None))
    gl = labels.to_numpy(np.int32, (n,))
    gc = cb.to_numpy(np.float32, (k, d))
    rc, rl, rloss = orc.kmeans_run(x, cent0, iters, 7)
    assert np.mean(gl == rl) >= 0.999, float(np.mean(gl == rl))
    assert abs(loss.value - rloss) <= 1e-4 * abs(rloss), (loss.value, rloss)
    # centroids of clusters whose members agree are the same means (fp32 sums in a different order)
    same = np.array([np.array_equal(np.nonzero(gl == j)[0], np.nonzero(rl == j)[0]) for j in range(0, k, 16)])
    assert same.mean() > 0.99
    np.testing.assert_allclose(gc[::16][same], rc[::16][same], rtol=1e-4, atol=1e-4)
    # the inertia went down from that of the initial centroids (estimated on the first 2048 rows)
    _, _, loss0 = orc.kmeans_assign(x[:2048], cent0)
    assert loss.value < loss0
    for b in (xb, cb, labels, ws):
        b.free()


def test_ivf_sq4_uniform_10m(lib):
    """configs[3] at the benchmark's own batch: 10 000 000 x 128 rows, 4096 lists of SQ4-uniform codes, 64 probes,
    rerank of 100, all 10 000 queries in one call (640 000 (query, list) pairs)."""
    n, d, nq, k, nlist, nprobe, kcand = 10000000, 128, 10000, 10, 4096, 64, 100
    means = mt(315).random((10000, d), dtype=np.float32)
    x_dev = capi.DeviceBuffer(n * d * 4)
    pick = np.sort(mt(7).choice(n, nlist, replace=False))
    init = np.empty((nlist, d), np.float32)
    for s, blk in mixture_chunks(47, n, d, means, 0.05):
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
        lo, hi = np.searchsorted(pick, [s, s + blk.shape[0]])
        init[lo:hi] = blk[pick[lo:hi] - s]
    q, _ = mixture(315, 165, nq, d, 10000, 0.05, means=means)
    ns = 64 * nlist
    cent = dev(init)
    slabels = capi.DeviceBuffer(ns * 4)
    wsb = lib.vsag_amd_kmeans_run_workspace_bytes(ns, d, nlist)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_kmeans_run(x_dev.ptr, ns, d, cent.ptr, nlist, 10, 7, slabels.ptr, None, ws.ptr, wsb, None))
    ws.free()
    labels = capi.DeviceBuffer(n * 4)
    wsb = lib.vsag_amd_kmeans_assign_workspace_bytes(n, d, nlist)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_kmeans_assign(x_dev.ptr, n, d, cent.ptr, nlist, labels.ptr, None, None, ws.ptr, wsb, None))
    ws.free()
    bounds = capi.DeviceBuffer(8)
    wsb = lib.vsag_amd_sq_train_workspace_bytes(ns, d, 0)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_sq_train_uniform(x_dev.ptr, ns, d, 4, capi.METRIC_L2, capi.SQ_TRAIN_TRUNC_BOUND, 0.05, 0,
                                             bounds.ptr, ws.ptr, wsb, None))
    ws.free()
    cs = int(lib.vsag_amd_code_size(capi.KIND_SQ4_UNIFORM, capi.METRIC_L2, d, 0))
    codes = capi.DeviceBuffer(n * cs)
    capi.check(lib.vsag_amd_squ_encode(x_dev.ptr, n, d, 4, capi.METRIC_L2, bounds.ptr, codes.ptr, None))
    hb = bounds.to_numpy(np.float32, (2,))
    hcodes = codes.to_numpy(np.uint8, (n, cs))
    hlabels = labels.to_numpy(np.int32, (n,))
    hcent = cent.to_numpy(np.float32, (nlist, d))

    lists = Store(capi.KIND_SQ4_UNIFORM, capi.METRIC_L2, d, bounds=hb)
    capi.check(lib.vsag_amd_store_set_lists(lists.handle, codes.ptr, labels.ptr, n, nlist, None))
    capi.synchronize()
    codes.free()
    assert lists.size() == n
    sizes = np.zeros(nlist, np.uint32)
    capi.check(lib.vsag_amd_store_list_sizes(lists.handle, sizes.ctypes.data, nlist))
    assert np.array_equal(sizes, np.bincount(hlabels, minlength=nlist).astype(np.uint32))

    # routing = exact nearest centroids
    cstore = Store(capi.KIND_FP32, capi.METRIC_L2, d)
    cstore.append(hcent.view(np.uint8).reshape(nlist, d * 4))
    q_dev = dev(q)
    buckets, bd = capi.DeviceBuffer(nq * nprobe * 4), capi.DeviceBuffer(nq * nprobe * 4)
    wr = lib.vsag_amd_ivf_route_workspace_bytes(cstore.handle, nq, nprobe)
    ws = capi.DeviceBuffer(wr)
    capi.check(lib.vsag_amd_ivf_route(cstore.handle, q_dev.ptr, nq, nprobe, buckets.ptr, bd.ptr, ws.ptr, wr, None))
    b = buckets.to_numpy(np.int32, (nq, nprobe))
    ws.free()
    ob, _ = orc.ivf_route(hcent, q[:64], nprobe)
    assert np.mean(ob == b[:64]) >= 0.999  # equal up to near-ties between centroid distances

    cand, cand_d = lists.ivf_scan(q, b, kcand)
    check_result_shape(cand, cand_d, n)
    # a batch of this size sends the probe columns behind the first through the int8 matrix cores (ivf_i8_kernel);
    # the streaming kernel alone must return the same bits
    info = capi.C.c_int()
    lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
    assert info.value == 256, "the int8 pass over the posting lists did not run"
    with streaming_only(lib, lists):
        si, sd = lists.ivf_scan(q, b, kcand)
        lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
        assert info.value <= 8
    assert np.array_equal(si, cand) and np.array_equal(sd.view(np.uint32), cand_d.view(np.uint32))
    # the checker on the same codes, lists and probes: integer distances, so bit-equal; ids up to equal distances
    offsets, order = orc.ivf_build_lists(hlabels, nlist)
    posting = hcodes[order]
    qcodes = orc.squ_encode(q[:64], 4, hb[0], hb[1], orc.L2)
    oi, od = orc.ivf_scan(orc.SQ4U, orc.L2, d, posting, offsets, order, qcodes, b[:64], kcand, lb=hb[0], diff=hb[1])
    assert np.array_equal(od.view(np.uint32), cand_d[:64].view(np.uint32))
    assert_topk_close(cand[:64], cand_d[:64], oi, od, rtol=0, atol=0, tie_rtol=0, label="ivf sq4u 10M")
    # the batch split does not matter: the same queries alone and in groups of 7
    for s, e in ((0, 1), (5, 6), (10, 17), (100, 107), (1000, 2024), (9990, 10000)):
        ci, cd = lists.ivf_scan(q[s:e], b[s:e], kcand)
        assert np.array_equal(ci, cand[s:e]) and np.array_equal(cd.view(np.uint32), cand_d[s:e].view(np.uint32)), (s, e)

    # rerank: exact fp64 distances of the candidates, best k
    cand_dev = dev(cand)
    out_i, out_d = capi.DeviceBuffer(nq * k * 4), capi.DeviceBuffer(nq * k * 4)
    capi.check(lib.vsag_amd_rerank_fp32(x_dev.ptr, n, d, capi.METRIC_L2, q_dev.ptr, nq, cand_dev.ptr, kcand, k,
                                        out_i.ptr, out_d.ptr, None))
    ri, rd = out_i.to_numpy(np.uint32, (nq, k)), out_d.to_numpy(np.float32, (nq, k))
    check_result_shape(ri, rd, n)
    row = np.empty(d, np.float32)
    for i in range(0, nq, 250):
        dd = np.empty(kcand)
        for j, c in enumerate(cand[i]):
            capi.check(lib.vsag_amd_memcpy_d2h(row.ctypes.data, x_dev.ptr + int(c) * d * 4, d * 4, None))
            dd[j] = ((row.astype(np.float64) - q[i].astype(np.float64)) ** 2).sum()
        best = np.lexsort((cand[i], dd))[:k]
        np.testing.assert_allclose(rd[i], dd[best], rtol=1e-4)
        assert set(ri[i]) == set(cand[i][best]) or np.allclose(np.sort(dd[best]), np.sort(rd[i]), rtol=1e-5)
    for x in (x_dev, cent, slabels, labels, bounds, q_dev, buckets, bd, cand_dev, out_i, out_d):
        x.free()
    lists.destroy()
    cstore.destroy()


def test_ivf_sq8_and_rabitq_lists_10m(lib):
    """configs[3]'s rows, lists and probes with sq8 and with RaBitQ codes in the lists: the probe columns behind the
    first go through the int8 matrix cores (two planes per query / expanded code bits), and what they return must be
    the streaming kernel's result bit for bit, the checker's on a sample, and independent of the batch split."""
    n, d, nq, nlist, nprobe, kcand = 10000000, 128, 10000, 4096, 64, 100
    means = mt(315).random((10000, d), dtype=np.float32)
    x_dev = capi.DeviceBuffer(n * d * 4)
    pick = np.sort(mt(7).choice(n, nlist, replace=False))
    init = np.empty((nlist, d), np.float32)
    for s, blk in mixture_chunks(47, n, d, means, 0.05):
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
        lo, hi = np.searchsorted(pick, [s, s + blk.shape[0]])
        init[lo:hi] = blk[pick[lo:hi] - s]
    q, _ = mixture(315, 165, nq, d, 10000, 0.05, means=means)
    ns = 64 * nlist
    cent = dev(init)
    slabels = capi.DeviceBuffer(ns * 4)
    wsb = lib.vsag_amd_kmeans_run_workspace_bytes(ns, d, nlist)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_kmeans_run(x_dev.ptr, ns, d, cent.ptr, nlist, 10, 7, slabels.ptr, None, ws.ptr, wsb, None))
    ws.free()
    labels = capi.DeviceBuffer(n * 4)
    wsb = lib.vsag_amd_kmeans_assign_workspace_bytes(n, d, nlist)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_kmeans_assign(x_dev.ptr, n, d, cent.ptr, nlist, labels.ptr, None, None, ws.ptr, wsb, None))
    ws.free()
    hlabels = labels.to_numpy(np.int32, (n,))
    hcent = cent.to_numpy(np.float32, (nlist, d))
    offsets, order = orc.ivf_build_lists(hlabels, nlist)
    b, _ = orc.ivf_route(hcent, q, nprobe)
    info = capi.C.c_int()

    def both(lists):
        fast = lists.ivf_scan(q, b, kcand)
        lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
        assert info.value == 256, "the int8 pass over the posting lists did not run"
        check_result_shape(fast[0], fast[1], n)
        capi.check(lib.vsag_amd_store_set_scan_contraction(lists.handle, -1))
        plain = lists.ivf_scan(q, b, kcand)
        capi.check(lib.vsag_amd_store_set_scan_contraction(lists.handle, -2))
        assert np.array_equal(plain[0], fast[0]) and np.array_equal(plain[1].view(np.uint32), fast[1].view(np.uint32))
        for s, e in ((0, 1), (10, 17), (1000, 2024), (9990, 10000)):
            ci, cd = lists.ivf_scan(q[s:e], b[s:e], kcand)
            assert np.array_equal(ci, fast[0][s:e]) and np.array_equal(cd.view(np.uint32), fast[1][s:e].view(np.uint32))
        return fast

    # sq8: a range per dimension
    lb_dev, diff_dev = capi.DeviceBuffer(d * 4), capi.DeviceBuffer(d * 4)
    wsb = lib.vsag_amd_sq_train_workspace_bytes(ns, d, 0)
    ws = capi.DeviceBuffer(wsb)
    capi.check(lib.vsag_amd_sq_train(x_dev.ptr, ns, d, 8, capi.METRIC_L2, capi.SQ_TRAIN_TRUNC_BOUND, 0.05, 0, lb_dev.ptr,
                                     diff_dev.ptr, ws.ptr, wsb, None))
    ws.free()
    codes = capi.DeviceBuffer(n * d)
    capi.check(lib.vsag_amd_sq_encode(x_dev.ptr, n, d, 8, capi.METRIC_L2, lb_dev.ptr, diff_dev.ptr, codes.ptr, None))
    hlb, hdiff = lb_dev.to_numpy(np.float32, (d,)), diff_dev.to_numpy(np.float32, (d,))
    hcodes = codes.to_numpy(np.uint8, (n, d))
    lists = Store(capi.KIND_SQ8, capi.METRIC_L2, d, lb=hlb, diff=hdiff)
    capi.check(lib.vsag_amd_store_set_lists(lists.handle, codes.ptr, labels.ptr, n, nlist, None))
    capi.synchronize()
    codes.free()
    fast = both(lists)
    oi, od = orc.ivf_scan(orc.SQ8, orc.L2, d, hcodes[order], offsets, order, q[:32], b[:32], kcand, lb=hlb, diff=hdiff)
    assert_topk_close(fast[0][:32], fast[1][:32], oi, od, atol=4e-6, label="ivf sq8 10M")
    lists.destroy()
    del hcodes

    # RaBitQ: 1-bit codes, 4-bit queries, a seeded rotation
    g = mt(316).standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    rot_dev, cen = dev(rot), capi.DeviceBuffer(d * 4)
    capi.check(lib.vsag_amd_rabitq_train(x_dev.ptr, ns, d, rot_dev.ptr, cen.ptr, None))
    cs = int(lib.vsag_amd_code_size(capi.KIND_RABITQ, capi.METRIC_L2, d, 4))
    codes = capi.DeviceBuffer(n * cs)
    capi.check(lib.vsag_amd_rabitq_encode(x_dev.ptr, n, d, rot_dev.ptr, cen.ptr, capi.METRIC_L2, 4, codes.ptr, None))
    hcen = cen.to_numpy(np.float32, (d,))
    hcodes = codes.to_numpy(np.uint8, (n, cs))
    lists = Store(capi.KIND_RABITQ, capi.METRIC_L2, d, rot=rot, centroid=hcen, qbits=4)
    capi.check(lib.vsag_amd_store_set_lists(lists.handle, codes.ptr, labels.ptr, n, nlist, None))
    capi.synchronize()
    codes.free()
    fast = both(lists)
    qcodes = orc.rabitq_process_query(q[:32], rot, hcen, orc.L2)
    oi, od = orc.ivf_scan(orc.RABITQ, orc.L2, d, hcodes[order], offsets, order, qcodes, b[:32], kcand)
    assert np.array_equal(od.view(np.uint32), fast[1][:32].view(np.uint32))
    lists.destroy()
    for x in (x_dev, cent, slabels, labels, lb_dev, diff_dev, rot_dev, cen):
        x.free()


def test_rabitq_scan_5m_x_768(lib):
    """configs[4] at the benchmark's own batch: 5 000 000 x 768 unit rows, 1-bit codes, 4-bit queries, inner product,
    200 candidates, all 10 000 queries in one call."""
    n, d, nq, kcand = 5000000, 768, 10000, 200
    rng = mt(47)
    x_dev = capi.DeviceBuffer(n * d * 4)
    head = None
    step_rows = 1 << 16
    for s in range(0, n, step_rows):
        blk = rng.standard_normal((min(step_rows, n - s), d), dtype=np.float32)
        blk /= np.linalg.norm(blk, axis=1, keepdims=True)
        capi.check(lib.vsag_amd_memcpy_h2d(x_dev.ptr + s * d * 4, blk.ctypes.data, blk.nbytes, None))
        if head is None:
            head = blk[:4096].copy()
    q = mt(165).standard_normal((nq, d), dtype=np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    g = mt(315).standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    rot_dev = dev(rot)
    cen = capi.DeviceBuffer(d * 4)
    capi.check(lib.vsag_amd_rabitq_train(x_dev.ptr, n, d, rot_dev.ptr, cen.ptr, None))
    cs = int(lib.vsag_amd_code_size(capi.KIND_RABITQ, capi.METRIC_IP, d, 4))
    assert cs == 112
    codes = capi.DeviceBuffer(n * cs)
    capi.check(lib.vsag_amd_rabitq_encode(x_dev.ptr, n, d, rot_dev.ptr, cen.ptr, capi.METRIC_IP, 4, codes.ptr, None))
    hcen = cen.to_numpy(np.float32, (d,))
    hcodes = codes.to_numpy(np.uint8, (n, cs))
    x_dev.free()
    # codes of the first rows equal the checker's bit for bit (same rotation, the device's centroid)
    assert np.array_equal(hcodes[:4096], orc.rabitq_encode(head, rot, hcen, orc.IP, 4))
    store = Store(capi.KIND_RABITQ, capi.METRIC_IP, d, rot=rot, centroid=hcen, qbits=4)
    capi.check(lib.vsag_amd_store_append(store.handle, codes.ptr, n, None))
    capi.synchronize()
    codes.free()
    ids, dists = store.flat_scan(q, kcand)
    check_result_shape(ids, dists, n)
    # the batch takes the matrix-core route (prefilter_rb_kernel: code bits x 4-bit queries on the int8 matrix cores,
    # exact rescoring); the checker on a sample and the streaming kernel alone on 1000 queries spread over the batch
    # must agree with it, and so must a smaller batch (another grid)
    info = capi.C.c_int()
    lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
    assert info.value == 128, "the matrix-core pre-selection did not run"
    qcodes = orc.rabitq_process_query(q[:16], rot, hcen, orc.IP, 4)
    oi, od = orc.flat_scan_topk(orc.RABITQ, orc.IP, d, hcodes, qcodes, kcand, qbits=4)
    assert_topk_close(ids[:16], dists[:16], oi, od, label="rabitq 5M")
    sel = np.arange(0, nq, 10)
    with streaming_only(lib, store):
        si, sd = store.flat_scan(q[sel], kcand)
        lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
        assert info.value <= 8
        ti, td = scan_with_tile(lib, store, q[:32], kcand, 1)
    assert np.array_equal(si, ids[sel]) and np.array_equal(sd.view(np.uint32), dists[sel].view(np.uint32))
    assert np.array_equal(ti, ids[:32]) and np.array_equal(td.view(np.uint32), dists[:32].view(np.uint32))
    pi, pd = store.flat_scan(q[:512], kcand)
    lib.vsag_amd_last_scan_info(capi.C.byref(info), None, None)
    assert info.value == 128
    assert np.array_equal(pi, ids[:512]) and np.array_equal(pd.view(np.uint32), dists[:512].view(np.uint32))
    for b in (rot_dev, cen):
        b.free()
    store.destroy()
