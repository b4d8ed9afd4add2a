"""pqfs (PQ fast scan, src/quantization/product_quantization/pq_fastscan_quantizer.cpp) on the device against the
CPU checker: codes, processed queries (byte tables), the packaged block order and every distance bit for bit; the
trained codebooks as good as the checker's; flat and posting-list scans with the fused top-k."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu

METRICS = [(orc.L2, "l2"), (orc.IP, "ip"), (orc.COSINE, "cosine")]


def gpu_encode(L, x, pq_dim, cb, metric):
    n, d = x.shape
    cs = (pq_dim + 1) // 2
    xb, cbb, out, norms = dev(x), dev(cb), capi.DeviceBuffer(n * cs), capi.DeviceBuffer(n * 4)
    capi.check(L.vsag_amd_pq_encode(xb.ptr, n, d, pq_dim, cbb.ptr, metric, out.ptr, norms.ptr, None))
    codes = out.to_numpy(np.uint8, (n, cs))
    for b in (xb, cbb, out, norms):
        b.free()
    return codes


@pytest.mark.parametrize("metric,mname", METRICS)
@pytest.mark.parametrize("n,d,pq_dim", [(700, 128, 128), (300, 96, 24), (500, 60, 15), (64, 33, 1)])
def test_pq_encode_decode_and_query_tables_bit_exact(lib, metric, mname, n, d, pq_dim):
    L = lib.load_library()
    rng = np.random.default_rng(n + d + pq_dim + metric)
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((9, d)).astype(np.float32)
    q[3] = 0.0  # a zero query: every entry of an ip table equal (diff 0), cosine divides by 1
    sd = d // pq_dim
    cb = rng.standard_normal((pq_dim, 16, sd)).astype(np.float32)
    ref = orc.pq_encode(x, pq_dim, cb, metric)
    codes = gpu_encode(L, x, pq_dim, cb, metric)
    assert np.array_equal(codes, ref)
    # decode
    cbuf, cbb, out = dev(ref), dev(cb), capi.DeviceBuffer(n * d * 4)
    capi.check(L.vsag_amd_pq_decode(cbuf.ptr, n, d, pq_dim, cbb.ptr, out.ptr, None))
    assert np.array_equal(out.to_numpy(np.float32, (n, d)), orc.pq_decode(ref, d, pq_dim, cb))
    # processed queries in the reference layout
    qs = pq_dim * 16 + 8
    qb, qout = dev(q), capi.DeviceBuffer(q.shape[0] * qs)
    capi.check(L.vsag_amd_pqfs_process_query(qb.ptr, q.shape[0], d, pq_dim, cbb.ptr, metric, qout.ptr, None))
    got = qout.to_numpy(np.uint8, (q.shape[0], qs))
    want = orc.pqfs_process_query(q, pq_dim, cb, metric)
    assert np.array_equal(got, want), np.argwhere(got != want)[:5]
    for b in (cbuf, cbb, out, qb, qout):
        b.free()


@pytest.mark.parametrize("n,pq_dim", [(32, 8), (100, 31), (1000, 128), (5, 2)])
def test_pqfs_package_and_unpack(lib, n, pq_dim):
    L = lib.load_library()
    rng = np.random.default_rng(n + pq_dim)
    cs = (pq_dim + 1) // 2
    codes = rng.integers(0, 256, (n, cs)).astype(np.uint8)
    if pq_dim % 2:
        codes[:, -1] &= 0x0F
    blocks = (n + 31) // 32
    pad = np.zeros((blocks * 32, cs), np.uint8)
    pad[:n] = codes
    want = np.concatenate([orc.pqfs_package32(pad[b * 32:(b + 1) * 32], pq_dim, valid=min(32, n - 32 * b))
                           for b in range(blocks)])
    cbuf, pbuf, back = dev(codes), capi.DeviceBuffer(blocks * 32 * cs), capi.DeviceBuffer(n * cs)
    capi.check(L.vsag_amd_pqfs_package(cbuf.ptr, n, pq_dim, pbuf.ptr, None))
    assert np.array_equal(pbuf.to_numpy(np.uint8, (blocks * 32 * cs,)), want)
    capi.check(L.vsag_amd_pqfs_unpack(pbuf.ptr, n, pq_dim, back.ptr, None))
    assert np.array_equal(back.to_numpy(np.uint8, (n, cs)), codes)
    for b in (cbuf, pbuf, back):
        b.free()


@pytest.mark.parametrize("metric,mname", [(orc.L2, "l2"), (orc.COSINE, "cosine")])
def test_pq_train_is_as_good_as_the_checkers(lib, metric, mname):
    """Same seeds, same draws: the codebooks agree where k-means takes the same path; what must hold in any case is
    the quantisation error (the sum over subspaces of the squared distance to the nearest centroid)."""
    L = lib.load_library()
    rng = np.random.default_rng(5)
    n, d, pq_dim = 4000, 32, 8
    x, _ = gaussian_mixture(rng, n, d, 12, 0.1)
    xb, cbb = dev(x), capi.DeviceBuffer(d * 16 * 4)
    wsb = L.vsag_amd_pq_train_workspace_bytes(n, d, pq_dim)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_pq_train(xb.ptr, n, d, pq_dim, metric, 11, cbb.ptr, ws.ptr, wsb, None))
    cb = cbb.to_numpy(np.float32, (pq_dim, 16, d // pq_dim))
    ref = orc.pq_train(x, pq_dim, metric, 11)
    xn = x / np.linalg.norm(x, axis=1, keepdims=True) if metric == orc.COSINE else x

    def err(books):
        dec = orc.pq_decode(orc.pq_encode(x, pq_dim, books, metric), d, pq_dim, books)
        return float(((xn - dec) ** 2).sum(1).mean())
    e_gpu, e_ref = err(cb), err(ref)
    assert np.isfinite(cb).all()
    assert abs(e_gpu - e_ref) <= 0.02 * e_ref, (e_gpu, e_ref)
    assert np.mean(np.isclose(cb, ref, rtol=1e-3, atol=1e-4)) > 0.9
    for b in (xb, cbb, ws):
        b.free()


@pytest.mark.parametrize("metric,mname", METRICS)
@pytest.mark.parametrize("n,d,pq_dim,nq,k", [(9000, 128, 128, 13, 10), (3000, 64, 16, 5, 100), (700, 30, 15, 3, 7),
                                             (40000, 128, 64, 600, 10)])
def test_pqfs_flat_scan(lib, metric, mname, n, d, pq_dim, nq, k):
    rng = np.random.default_rng(n + d + metric)
    x, means = gaussian_mixture(rng, n, d, 30, 0.1)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.1, means=means)
    cb = orc.pq_train(x[:2000], pq_dim, metric)
    codes = orc.pq_encode(x, pq_dim, cb, metric)
    st = Store(capi.KIND_PQFS, metric, d, pq_dim=pq_dim, codebooks=cb)
    assert st.code_size() == codes.shape[1]
    st.append(codes)
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(orc.PQFS, metric, pq_dim, codes, orc.pqfs_process_query(q, pq_dim, cb, metric), k)
    # integer sums of table bytes and three float operations in the reference's order: the distances are the same bits
    assert np.array_equal(ds.view(np.uint32), rds.view(np.uint32))
    assert_topk_close(ids, ds, rids, rds, rtol=0, atol=0, tie_rtol=0, label="pqfs " + mname)
    # one query per call and a filter / radius go the same way
    i1, d1 = st.flat_scan(q[:1], k)
    assert np.array_equal(i1[0], ids[0]) and np.array_equal(d1[0].view(np.uint32), ds[0].view(np.uint32))
    deny = rng.random(n) < 0.3
    fi, fd = st.flat_scan(q[:4], k, deny=deny)
    assert not deny[fi[fi != capi.INVALID_ID]].any()
    st.destroy()


@pytest.mark.parametrize("metric,mname", METRICS)
def test_pqfs_posting_lists_and_lookup(lib, metric, mname):
    L = lib.load_library()
    rng = np.random.default_rng(77 + metric)
    n, d, pq_dim, nlist, nprobe, nq, kcand = 20000, 64, 32, 40, 7, 50, 60
    x, means = gaussian_mixture(rng, n, d, 40, 0.1)
    q, _ = gaussian_mixture(rng, nq, d, 40, 0.1, means=means)
    cb = orc.pq_train(x[:3000], pq_dim, metric)
    codes = orc.pq_encode(x, pq_dim, cb, metric)
    labels = rng.integers(0, nlist, n).astype(np.int32)
    buckets = np.stack([rng.permutation(nlist)[:nprobe] for _ in range(nq)]).astype(np.int32)
    st = Store(capi.KIND_PQFS, metric, d, pq_dim=pq_dim, codebooks=cb)
    st.set_lists(codes, labels, nlist)
    ids, ds = st.ivf_scan(q, buckets, kcand)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qc = orc.pqfs_process_query(q, pq_dim, cb, metric)
    rids, rds = orc.ivf_scan(orc.PQFS, metric, pq_dim, codes[order], offsets, order, qc, buckets, kcand)
    assert np.array_equal(ds.view(np.uint32), rds.view(np.uint32))
    assert_topk_close(ids, ds, rids, rds, rtol=0, atol=0, tie_rtol=0, label="pqfs lists " + mname)
    # distances by id (Index::CalDistanceById): the same arithmetic
    want = orc.flat_dists(orc.PQFS, metric, pq_dim, codes, qc[:3])
    pick = rng.integers(0, n, (3, 20)).astype(np.uint32)
    qb, ib, out = dev(q[:3]), dev(pick), capi.DeviceBuffer(3 * 20 * 4)
    wsb = L.vsag_amd_store_distances_workspace_bytes(st.handle, 3)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_store_distances(st.handle, qb.ptr, 3, ib.ptr, 20, out.ptr, ws.ptr, wsb, None))
    got = out.to_numpy(np.float32, (3, 20))
    assert np.array_equal(got.view(np.uint32), np.take_along_axis(want, pick.astype(np.int64), 1).view(np.uint32))
    for b in (qb, ib, out, ws):
        b.free()
    st.destroy()


@pytest.mark.parametrize("metric,mname", METRICS)
@pytest.mark.parametrize("d,pq_dim", [(128, 128), (64, 32), (62, 31), (96, 8)])
def test_pqfs_lists_on_the_matrix_cores_equal_the_streaming_scan(lib, metric, mname, d, pq_dim):
    """A large batch sends the probe columns behind the first through the int8 matrix cores (one-hot centroid indices
    against the byte tables, ivf_pq.hip): ids and distance bits must be the streaming kernel's, and the checker's on
    a sample.  Lists shorter than the candidate count (queries without a bound overflow into the streaming fallback),
    missing buckets and a list probed twice are part of the batch."""
    L = lib.load_library()
    rng = np.random.default_rng(d + pq_dim + metric)
    n, nlist, nprobe, nq, kcand = 150000, 256, 12, 3000, 40
    x, means = gaussian_mixture(rng, n, d, 200, 0.08)
    q, _ = gaussian_mixture(rng, nq, d, 200, 0.08, means=means)
    cb = orc.pq_train(x[:4000], pq_dim, metric)
    codes = orc.pq_encode(x, pq_dim, cb, metric)
    labels = rng.integers(0, nlist, n).astype(np.int32)
    labels[labels < 3] = 3 + rng.integers(0, nlist - 3, int((labels < 3).sum()))  # lists 0..2: nearly empty
    labels[:20] = 0
    labels[20:25] = 1
    buckets = np.stack([rng.permutation(nlist)[:nprobe] for _ in range(nq)]).astype(np.int32)
    buckets[:200, 0] = rng.integers(0, 3, 200)   # a first list that leaves no bound
    buckets[200:300, 5] = -1                     # missing buckets
    buckets[300:320, 7] = buckets[300:320, 3]    # a list probed twice
    st = Store(capi.KIND_PQFS, metric, d, pq_dim=pq_dim, codebooks=cb)
    st.set_lists(codes, labels, nlist)
    fast = st.ivf_scan(q, buckets, kcand)
    info = C.c_int()
    L.vsag_amd_last_scan_info(C.byref(info), None, None)
    assert info.value == 256, "the matrix-core pass over the posting lists did not run"
    capi.check(L.vsag_amd_store_set_scan_contraction(st.handle, -1))
    plain = st.ivf_scan(q, buckets, kcand)
    L.vsag_amd_last_scan_info(C.byref(info), None, None)
    assert info.value <= 8
    capi.check(L.vsag_amd_store_set_scan_contraction(st.handle, -2))
    assert np.array_equal(fast[0], plain[0]) and np.array_equal(fast[1].view(np.uint32), plain[1].view(np.uint32))
    offsets, order = orc.ivf_build_lists(labels, nlist)
    sel = np.r_[0:40, 200:240, 300:320, 2900:2940]
    # the checker keeps what it meets first among equal distances and scans a list probed twice twice
    sel = sel[~np.isin(sel, np.arange(300, 320))]
    qc = orc.pqfs_process_query(q[sel], pq_dim, cb, metric)
    rids, rds = orc.ivf_scan(orc.PQFS, metric, pq_dim, codes[order], offsets, order, qc, buckets[sel], kcand)
    assert np.array_equal(fast[1][sel].view(np.uint32), rds.view(np.uint32))
    assert_topk_close(fast[0][sel], fast[1][sel], rids, rds, rtol=0, atol=0, tie_rtol=0, label="pqfs mfma " + mname)
    # the batch split does not matter
    for s, e in ((0, 1), (250, 257), (1000, 2024)):
        ci, cd = st.ivf_scan(q[s:e], buckets[s:e], kcand)
        assert np.array_equal(ci, fast[0][s:e]) and np.array_equal(cd.view(np.uint32), fast[1][s:e].view(np.uint32)), (s, e)
    st.destroy()
