"""IVF route / posting-list scan / rerank on the device against the CPU checker."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _ivf_case(rng, n, d, nlist, nq):
    x, means = gaussian_mixture(rng, n, d, 40, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 40, 0.05, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    return x, q, cent, labels


def test_route_matches_exact_centroid_scan(lib):
    L = lib.load_library()
    rng = np.random.default_rng(5)
    x, q, cent, _ = _ivf_case(rng, 4000, 64, 300, 50)
    st = Store(capi.KIND_FP32, orc.L2, 64)
    st.append(cent.view(np.uint8).reshape(300, 256))
    nprobe = 16
    qb = dev(q)
    b, ds = capi.DeviceBuffer(50 * nprobe * 4), capi.DeviceBuffer(50 * nprobe * 4)
    wsb = L.vsag_amd_ivf_route_workspace_bytes(st.handle, 50, nprobe)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_ivf_route(st.handle, qb.ptr, 50, nprobe, b.ptr, ds.ptr, ws.ptr, wsb, None))
    buckets = b.to_numpy(np.int32, (50, nprobe))
    dists = ds.to_numpy(np.float32, (50, nprobe))
    rb, rd = orc.ivf_route(cent, q, nprobe)
    assert_topk_close(buckets.view(np.uint32), dists, rb.view(np.uint32), rd, atol=2e-6, label="route")
    st.destroy()


@pytest.mark.parametrize("kind,okind,bits", [("sq4u", orc.SQ4U, 4), ("sq8", orc.SQ8, 8), ("fp32", orc.FP32, 32)])
@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand", [(20000, 128, 64, 40, 8, 100), (3000, 33, 200, 7, 200, 10),
                                                       (500, 16, 8, 3, 1, 5)])
def test_ivf_scan_matches_oracle(lib, kind, okind, bits, n, d, nlist, nq, nprobe, kcand):
    rng = np.random.default_rng(n + d + bits)
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    routed, _ = orc.ivf_route(cent, q, min(nprobe, nlist))
    buckets = np.full((nq, nprobe), -1, np.int32)
    buckets[:, :routed.shape[1]] = routed
    lb = diff = None
    if kind == "sq4u":
        l, dd = orc.sq_train_uniform(x, 4, orc.L2, mode=3)
        codes = orc.squ_encode(x, 4, l, dd, orc.L2)
        qproc = orc.squ_encode(q, 4, l, dd, orc.L2)
        lb, diff = l, dd
        st = Store(capi.KIND_SQ4_UNIFORM, orc.L2, d, bounds=[l, dd])
    elif kind == "sq8":
        lb, diff = orc.sq_train(x, 8)
        codes = orc.sq_encode(x, 8, lb, diff)
        qproc = q
        st = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    else:
        codes = x.view(np.uint8).reshape(n, 4 * d)
        qproc = q
        st = Store(capi.KIND_FP32, orc.L2, d)
    st.set_lists(codes, labels, nlist)
    sizes = np.zeros(nlist, np.uint32)
    capi.check(lib.load_library().vsag_amd_store_list_sizes(st.handle, sizes.ctypes.data, nlist))
    assert np.array_equal(sizes, np.diff(offsets).astype(np.uint32))
    ids, ds = st.ivf_scan(q, buckets, kcand)
    rids, rds = orc.ivf_scan(okind, orc.L2, d, codes[order], offsets, order, qproc, buckets, kcand, lb=lb, diff=diff)
    if kind == "sq4u":
        assert np.array_equal(ds.view(np.uint32), rds.view(np.uint32))
        assert_topk_close(ids, ds, rids, rds, rtol=0, atol=0, tie_rtol=0, label="ivf sq4u")
    else:
        assert_topk_close(ids, ds, rids, rds, atol=2e-6, label="ivf " + kind)
    st.destroy()


@pytest.mark.parametrize("kind", ["sq8", "sq4u"])
def test_many_pairs_are_grouped_by_the_counting_sort(lib, kind):
    """From 65 536 (query, list) pairs of a pass on, the pairs are grouped by list with a counting sort in LDS instead of
    an atomic per pair; what a query finds does not depend on where its pairs land inside a list's group.  Streaming
    kernels only (sq8 lists; sq4_uniform with the matrix cores switched off), a ragged bucket table, one list much
    longer than the others."""
    rng = np.random.default_rng(5)
    n, d, nlist, nq, nprobe, kcand = 30000, 32, 48, 10000, 9, 10
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    labels = labels.copy()
    labels[rng.random(n) < 0.3] = 7  # a long list
    offsets, order = orc.ivf_build_lists(labels, nlist)
    routed, _ = orc.ivf_route(cent, q, nprobe)
    buckets = routed.copy()
    buckets[::5, 6:] = -1
    buckets[3, :] = -1
    if kind == "sq4u":
        l, dd = orc.sq_train_uniform(x, 4, orc.L2, mode=3)
        codes = orc.squ_encode(x, 4, l, dd, orc.L2)
        qproc = orc.squ_encode(q, 4, l, dd, orc.L2)
        lb, diff, okind = l, dd, orc.SQ4U
        st = Store(capi.KIND_SQ4_UNIFORM, orc.L2, d, bounds=[l, dd])
    else:
        lb, diff = orc.sq_train(x, 8)
        codes = orc.sq_encode(x, 8, lb, diff)
        qproc, okind = q, orc.SQ8
        st = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    st.set_lists(codes, labels, nlist)
    L = lib.load_library()
    capi.check(L.vsag_amd_store_set_scan_contraction(st.handle, -1))
    ids, ds = st.ivf_scan(q, buckets, kcand)
    rids, rds = orc.ivf_scan(okind, orc.L2, d, codes[order], offsets, order, qproc, buckets, kcand, lb=lb, diff=diff)
    if kind == "sq4u":
        assert np.array_equal(ds.view(np.uint32), rds.view(np.uint32))
        # and the matrix-core pass over the same grouping
        capi.check(L.vsag_amd_store_set_scan_contraction(st.handle, -2))
        fids, fds = st.ivf_scan(q, buckets, kcand)
        tile = capi.C.c_int()
        L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
        assert tile.value == 256
        assert np.array_equal(fids, ids) and np.array_equal(fds.view(np.uint32), ds.view(np.uint32))
    else:
        assert_topk_close(ids, ds, rids, rds, atol=2e-6, label="ivf sq8, many pairs")
    assert np.all(ids[3] == 0xFFFFFFFF)
    st.destroy()


def test_probe_all_lists_equals_flat_scan(lib):
    rng = np.random.default_rng(9)
    n, d, nlist, nq = 5000, 48, 32, 12
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    lb, diff = orc.sq_train(x, 8)
    codes = orc.sq_encode(x, 8, lb, diff)
    flat = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    flat.append(codes)
    lists = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    lists.set_lists(codes, labels, nlist)
    buckets = np.tile(np.arange(nlist, dtype=np.int32), (nq, 1))
    i1, d1 = flat.flat_scan(q, 20)
    i2, d2 = lists.ivf_scan(q, buckets, 20)
    assert np.array_equal(i1, i2) and np.array_equal(d1, d2)
    flat.destroy()
    lists.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
def test_rerank_matches_oracle(lib, metric):
    L = lib.load_library()
    rng = np.random.default_rng(21)
    n, d, nq, kcand, k = 3000, 128, 17, 100, 10
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((nq, d), dtype=np.float32)
    cand = np.stack([rng.choice(n, kcand, replace=False) for _ in range(nq)]).astype(np.uint32)
    cand[0, 5:] = 0xFFFFFFFF  # a short candidate list
    xb, qb, cb = dev(x), dev(q), dev(cand)
    ids, ds = capi.DeviceBuffer(nq * k * 4), capi.DeviceBuffer(nq * k * 4)
    capi.check(L.vsag_amd_rerank_fp32(xb.ptr, n, d, metric, qb.ptr, nq, cb.ptr, kcand, k, ids.ptr, ds.ptr, None))
    gi, gd = ids.to_numpy(np.uint32, (nq, k)), ds.to_numpy(np.float32, (nq, k))
    ri, rd = orc.rerank_fp32(x, q, cand, k, metric)
    assert_topk_close(gi, gd, ri, rd, atol=2e-6, label="rerank")
    assert np.all(gi[0, 5:] == 0xFFFFFFFF)


def _append_lists(lib, store, codes, labels, bias=None):
    cbuf, lbuf = dev(np.ascontiguousarray(codes)), dev(np.ascontiguousarray(labels, np.int32))
    bbuf = dev(np.ascontiguousarray(bias, np.float32)) if bias is not None else None
    capi.check(lib.load_library().vsag_amd_store_append_lists(store.handle, cbuf.ptr, lbuf.ptr,
                                                             bbuf.ptr if bbuf is not None else None, codes.shape[0], None))
    for b in (cbuf, lbuf, bbuf):
        if b is not None:
            b.free()


@pytest.mark.parametrize("kind", ["sq8", "sq4u", "fp32"])
def test_lists_appended_in_pieces_equal_one_fill(lib, kind):
    """IVF::Add on a filled index (ivf.cpp:590-724): codes appended to their lists piece by piece -- the first pieces fit
    the room of the first fill's last tiles, later ones make every list move -- give the lists one fill of everything
    gives: same sizes, and the same scan results bit for bit (in-list order = insertion order either way)."""
    rng = np.random.default_rng(77)
    n, d, nlist, nq, nprobe, kcand = 9000, 64, 37, 25, 9, 50
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    labels[labels == 5] = 6  # an empty list
    if kind == "sq8":
        lb, diff = orc.sq_train(x, 8)
        codes = orc.sq_encode(x, 8, lb, diff)
        make = lambda: Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    elif kind == "sq4u":
        l, dd = orc.sq_train_uniform(x, 4, orc.L2, mode=3)
        codes = orc.squ_encode(x, 4, l, dd, orc.L2)
        make = lambda: Store(capi.KIND_SQ4_UNIFORM, orc.L2, d, bounds=[l, dd])
    else:
        codes = x.view(np.uint8).reshape(n, 4 * d)
        make = lambda: Store(capi.KIND_FP32, orc.L2, d)
    whole = make()
    whole.set_lists(codes, labels, nlist)
    grown = make()
    cuts = [0, 3000, 3001, 3010, 3500, 6000, 9000]
    grown.set_lists(codes[:cuts[1]], labels[:cuts[1]], nlist)
    for s, e in zip(cuts[1:-1], cuts[2:]):
        _append_lists(lib, grown, codes[s:e], labels[s:e])
    assert grown.size() == n
    L = lib.load_library()
    sa, sb = np.zeros(nlist, np.uint32), np.zeros(nlist, np.uint32)
    capi.check(L.vsag_amd_store_list_sizes(whole.handle, sa.ctypes.data, nlist))
    capi.check(L.vsag_amd_store_list_sizes(grown.handle, sb.ctypes.data, nlist))
    assert np.array_equal(sa, sb) and sa[5] == 0
    routed, _ = orc.ivf_route(cent, q, nprobe)
    i1, d1 = whole.ivf_scan(q, routed, kcand)
    i2, d2 = grown.ivf_scan(q, routed, kcand)
    assert np.array_equal(i1, i2) and np.array_equal(d1.view(np.uint32), d2.view(np.uint32))
    # a store that starts empty and is only ever appended to
    empty = make()
    empty.set_lists(codes[:0], labels[:0], nlist)
    assert empty.ivf_scan(q, routed, kcand)[0].max() == 0xFFFFFFFF
    _append_lists(lib, empty, codes[:4000], labels[:4000])
    _append_lists(lib, empty, codes[4000:], labels[4000:])
    i3, d3 = empty.ivf_scan(q, routed, kcand)
    assert np.array_equal(i1, i3) and np.array_equal(d1.view(np.uint32), d3.view(np.uint32))
    for st in (whole, grown, empty):
        st.destroy()


def _store_distances(lib, store, q, ids):
    L = lib.load_library()
    nq, count = ids.shape
    qb, ib = dev(np.ascontiguousarray(q, np.float32)), dev(np.ascontiguousarray(ids, np.uint32))
    out = capi.DeviceBuffer(nq * count * 4)
    wsb = L.vsag_amd_store_distances_workspace_bytes(store.handle, nq)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_store_distances(store.handle, qb.ptr, nq, ib.ptr, count, out.ptr, ws.ptr, wsb, None))
    res = out.to_numpy(np.float32, (nq, count))
    for b in (qb, ib, out, ws):
        b.free()
    return res


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
def test_distances_by_inner_id(lib, metric):
    """CalDistanceById's core: the distance of a query to codes named by inner id equals the scan's distance to the
    same code, on a flat store and on posting lists; unknown ids give -1."""
    rng = np.random.default_rng(31)
    n, d, nlist, nq, count = 5000, 96, 23, 6, 150
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    lb, diff = orc.sq_train(x, 8, metric)
    codes = orc.sq_encode(x, 8, lb, diff, metric)
    ids = rng.integers(0, n, (nq, count)).astype(np.uint32)
    ids[1, 3] = 0xFFFFFFFF
    ids[2, 7] = n + 5
    expect = orc.flat_dists(orc.SQ8, metric, d, codes, q, lb=lb, diff=diff)
    want = np.take_along_axis(expect, np.minimum(ids, n - 1).astype(np.int64), 1)
    want[1, 3] = want[2, 7] = -1.0
    flat = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    flat.append(codes)
    lists = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    lists.set_lists(codes[:3000], labels[:3000], nlist)
    _append_lists(lib, lists, codes[3000:], labels[3000:])
    for st in (flat, lists):
        got = _store_distances(lib, st, q, ids)
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=2e-6)
        st.destroy()


@pytest.mark.parametrize("metric,mname", [(orc.L2, "l2"), (orc.IP, "ip"), (orc.COSINE, "cosine")])
@pytest.mark.parametrize("kind", ["fp32", "sq8", "sq4u"])
def test_residual_lists_match_oracle(lib, kind, metric, mname):
    """use_residual (bucket_datacell.h:527-572,594-639): codes of x - c scanned with the list's bias and <q, c> taken
    off, against the checker's restatement; with fp32 codes that is the plain distance to x again -- except under
    cosine, where FP32Quantizer::EncodeOneImpl (fp32_quantizer.cpp:58-72) normalises what it is given, the residual
    too: the stored code is the unit residual and the figure is 1 - <q, r / |r|> - <q, c>, as in the reference."""
    L = lib.load_library()
    rng = np.random.default_rng(41 + metric)
    n, d, nlist, nq, nprobe, kcand = 6000, 48, 29, 19, 7, 40
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    x = (x - 0.3).astype(np.float32)
    q = (q - 0.3).astype(np.float32)
    res = orc.residual_rows(x, labels, cent, metric)
    xb, lb_dev, cb = dev(x), dev(labels.astype(np.int32)), dev(cent)
    rb = capi.DeviceBuffer(n * d * 4)
    capi.check(L.vsag_amd_residual_rows(xb.ptr, n, d, metric, lb_dev.ptr, cb.ptr, rb.ptr, None))
    assert np.array_equal(rb.to_numpy(np.float32, (n, d)).view(np.uint32), res.view(np.uint32))
    qproc = q if metric != orc.COSINE else (q / np.linalg.norm(q, axis=1, keepdims=True)).astype(np.float32)
    lb = diff = None
    ocodes = None
    if kind == "fp32":
        codes = res.view(np.uint8).reshape(n, 4 * d)
        dec = res
        st = Store(capi.KIND_FP32, metric, d)
        okind = orc.FP32
        if metric == orc.COSINE:
            unit = (res / np.linalg.norm(res.astype(np.float64), axis=1, keepdims=True)).astype(np.float32)
            ocodes = unit.view(np.uint8).reshape(n, 4 * d)
    elif kind == "sq8":
        lb, diff = orc.sq_train(res, 8, metric)
        codes = orc.sq_encode(res, 8, lb, diff, metric)
        dec = orc.sq_decode(codes, d, 8, lb, diff)
        st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
        okind = orc.SQ8
    else:
        l, dd = orc.sq_train_uniform(res, 4, metric, mode=3)
        codes = orc.squ_encode(res, 4, l, dd, metric)
        dec = orc.squ_decode(codes, d, 4, l, dd, metric)
        lb, diff = l, dd
        st = Store(capi.KIND_SQ4_UNIFORM, metric, d, bounds=[l, dd])
        okind = orc.SQ4U
        qproc = orc.squ_encode(q, 4, l, dd, metric)
    bias = orc.residual_bias(dec, labels, cent) if metric == orc.L2 else None
    capi.check(L.vsag_amd_store_set_residual(st.handle, cb.ptr, nlist, None))
    st.set_lists(codes[:0], labels[:0], nlist)
    if metric == orc.L2:
        cdev, bdev, scratch = dev(codes), capi.DeviceBuffer(n * 4), capi.DeviceBuffer(n * d * 4)
        capi.check(L.vsag_amd_residual_bias(st.handle, cdev.ptr, n, lb_dev.ptr, cb.ptr, bdev.ptr, scratch.ptr, None))
        gbias = bdev.to_numpy(np.float32, (n,))
        np.testing.assert_allclose(gbias, bias, rtol=1e-5, atol=1e-5)
        for b in (cdev, bdev, scratch):
            b.free()
    _append_lists(lib, st, codes[:2500], labels[:2500], None if bias is None else bias[:2500])
    _append_lists(lib, st, codes[2500:], labels[2500:], None if bias is None else bias[2500:])
    offsets, order = orc.ivf_build_lists(labels, nlist)
    routed, _ = orc.ivf_route(cent, q, nprobe)
    ids, ds = st.ivf_scan(q, routed, kcand)
    rids, rds = orc.ivf_scan_residual(okind, metric, d, (codes if ocodes is None else ocodes)[order], offsets, order, qproc, q, cent,
                                      None if bias is None else bias[order], routed, kcand, lb=lb, diff=diff)
    assert_topk_close(ids, ds, rids, rds, rtol=2e-4, atol=2e-5, tie_rtol=2e-4, label="residual %s %s" % (kind, mname))
    if kind == "fp32" and metric != orc.COSINE:
        # closed form: the residual scan of fp32 codes is the plain distance to the original vectors
        plain = Store(capi.KIND_FP32, metric, d)
        plain.set_lists(x.view(np.uint8).reshape(n, 4 * d), labels, nlist)
        pi, pd = plain.ivf_scan(q, routed, kcand)
        assert_topk_close(ids, ds, pi, pd, rtol=2e-4, atol=5e-5, tie_rtol=5e-4, label="residual fp32 closed form")
        plain.destroy()
    for b in (xb, lb_dev, cb, rb):
        b.free()
    st.destroy()


@pytest.mark.parametrize("nq,kcand", [(40, 32), (40, 33), (6000, 32), (6000, 7)])
def test_a_list_probed_twice_brings_every_key_twice(lib, nq, kcand):
    """Injected buckets may name a list twice; then every (distance, id) key exists twice, also the k-th one, and the
    closing merge must keep the right number of copies of it: positions 2i and 2i + 1 of a result are equal."""
    rng = np.random.default_rng(kcand)
    n, d, nlist = 20000, 32, 16
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    lb, diff = orc.sq_train(x, 8)
    codes = orc.sq_encode(x, 8, lb, diff)
    st = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    st.set_lists(codes, labels, nlist)
    routed, _ = orc.ivf_route(cent, q, 2)
    buckets = np.ascontiguousarray(routed[:, [0, 1, 0, 1]])
    ids, ds = st.ivf_scan(q, buckets, kcand)
    once, od = st.ivf_scan(q, np.ascontiguousarray(routed), kcand)
    half = kcand // 2
    assert np.array_equal(ids[:, 0:2 * half:2], ids[:, 1:2 * half:2])
    assert np.array_equal(ids[:, 0:2 * half:2], once[:, :half])
    assert np.array_equal(ds[:, 0:2 * half:2].view(np.uint32), od[:, :half].view(np.uint32))
    if kcand % 2:
        assert np.array_equal(ids[:, -1], once[:, half])
    st.destroy()


@pytest.mark.parametrize("metric,mname", [(orc.L2, "l2"), (orc.IP, "ip")])
@pytest.mark.parametrize("qbits", [4, 32])
def test_residual_rabitq_lists_match_oracle(lib, metric, mname, qbits):
    """use_residual with rabitq lists (bucket_datacell.h:594-650): the quantizer is trained on and encodes x - c; under
    l2 the bias of a code comes from RaBitQuantizer::DecodeOneImpl (rabitq_quantizer.cpp:871-899), the sign point
    rotated back.  The decoder and the bias against the checker's, then the scan against its restatement."""
    L = lib.load_library()
    rng = np.random.default_rng(97 + metric + qbits)
    n, d, nlist, nq, nprobe, kcand = 5000, 72, 23, 17, 6, 30
    x, q, cent, labels = _ivf_case(rng, n, d, nlist, nq)
    x = (x - 0.3).astype(np.float32)
    q = (q - 0.3).astype(np.float32)
    res = orc.residual_rows(x, labels, cent, metric)
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(res, rot)
    codes = orc.rabitq_encode(res, rot, cen, metric, qbits)
    dec = orc.rabitq_decode(codes, d, rot, cen, metric, qbits)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen, qbits=qbits)
    cdev, rdev, cendev, out = dev(codes), dev(rot), dev(cen), capi.DeviceBuffer(n * d * 4)
    capi.check(L.vsag_amd_rabitq_decode(cdev.ptr, n, d, rdev.ptr, cendev.ptr, metric, qbits, out.ptr, None))
    np.testing.assert_allclose(out.to_numpy(np.float32, (n, d)), dec, rtol=0, atol=2e-6 * (1 + np.abs(dec).max()))
    cb, lb_dev = dev(cent), dev(labels.astype(np.int32))
    capi.check(L.vsag_amd_store_set_residual(st.handle, cb.ptr, nlist, None))
    st.set_lists(codes[:0], labels[:0], nlist)
    bias = None
    if metric == orc.L2:
        bias = orc.residual_bias(dec, labels, cent)
        bdev = capi.DeviceBuffer(n * 4)
        capi.check(L.vsag_amd_residual_bias(st.handle, cdev.ptr, n, lb_dev.ptr, cb.ptr, bdev.ptr, out.ptr, None))
        np.testing.assert_allclose(bdev.to_numpy(np.float32, (n,)), bias, rtol=1e-5, atol=1e-5)
        bdev.free()
    _append_lists(lib, st, codes[:2000], labels[:2000], None if bias is None else bias[:2000])
    _append_lists(lib, st, codes[2000:], labels[2000:], None if bias is None else bias[2000:])
    offsets, order = orc.ivf_build_lists(labels, nlist)
    routed, _ = orc.ivf_route(cent, q, nprobe)
    ids, ds = st.ivf_scan(q, routed, kcand)
    qproc = orc.rabitq_process_query(q, rot, cen, metric, qbits)
    rids, rds = orc.ivf_scan_residual(orc.RABITQ, metric, d, codes[order], offsets, order, qproc, q, cent,
                                      None if bias is None else bias[order], routed, kcand, qbits=qbits)
    assert_topk_close(ids, ds, rids, rds, rtol=2e-4, atol=5e-5, tie_rtol=2e-4, label="residual rabitq %s" % mname)
    for b in (cdev, rdev, cendev, out, cb, lb_dev):
        b.free()
    st.destroy()
