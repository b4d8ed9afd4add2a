"""One query per call against a large flat store: the route that writes every distance, keeps a minimum per run of
tiles and selects in a second launch (scan_one.hip) returns, bit for bit, what the batched streaming kernel returns
(same distance arithmetic, same (distance, id) order), with a pre-filter, with a radius, and when distances tie."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _streaming(lib, st, q, k, **kw):
    capi.check(lib.vsag_amd_store_set_scan_tuning(st.handle, 1, -1))
    try:
        return st.flat_scan(q, k, **kw)
    finally:
        capi.check(lib.vsag_amd_store_set_scan_tuning(st.handle, -1, -1))


def _route(lib):
    tile, passes, nbytes = capi.C.c_int(), capi.C.c_uint64(), capi.C.c_uint64()
    lib.vsag_amd_last_scan_info(capi.C.byref(tile), capi.C.byref(passes), capi.C.byref(nbytes))
    return tile.value, passes.value, nbytes.value


def _rotation(rng, d):
    q, _ = np.linalg.qr(rng.standard_normal((d, d)))
    return q.astype(np.float32)


def _sq8_store(rng, n, d, metric):
    x = rng.standard_normal((n, d)).astype(np.float32)
    lb, diff = orc.sq_train(x, 8)
    codes = orc.sq_encode(x, 8, lb, diff)
    st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    st.append(codes)
    return st, codes, lb, diff


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("n,d,k", [(70000, 128, 10), (65536 + 17, 32, 1), (200000, 64, 100), (131072, 128, 128)])
def test_one_query_sq8_equals_streaming_and_checker(lib, metric, n, d, k):
    lib = lib.load_library()
    rng = np.random.default_rng(n + d + k)
    st, codes, lb, diff = _sq8_store(rng, n, d, metric)
    for i in range(3):
        q = rng.standard_normal((1, d)).astype(np.float32)
        ids, ds = st.flat_scan(q, k)
        tile, passes, _ = _route(lib)
        sids, sds = _streaming(lib, st, q, k)
        assert (tile, passes) == (1, 1)
        assert np.array_equal(ids, sids) and np.array_equal(ds.view(np.uint32), sds.view(np.uint32))
        rids, rds = orc.flat_scan_topk(orc.SQ8, metric, d, codes, q, k, lb=lb, diff=diff)
        assert_topk_close(ids, ds, rids, rds, rtol=2e-5, atol=1e-5, tie_rtol=2e-5, label="one query sq8")
    st.destroy()


def test_one_query_every_kind_equals_streaming(lib):
    lib = lib.load_library()
    rng = np.random.default_rng(5)
    n, d, k = 66000, 64, 10
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((4, d)).astype(np.float32)
    stores = []
    for metric in (orc.L2, orc.IP, orc.COSINE):
        st = Store(capi.KIND_FP32, metric, d)
        st.append(x.view(np.uint8).reshape(n, 4 * d))
        stores.append(("fp32", st))
        lb, diff = orc.sq_train(x, 4)
        st = Store(capi.KIND_SQ4, metric, d, lb=lb, diff=diff)
        st.append(orc.sq_encode(x, 4, lb, diff))
        stores.append(("sq4", st))
        for kind, bits in ((capi.KIND_SQ4_UNIFORM, 4), (capi.KIND_SQ8_UNIFORM, 8)):
            ulb, udiff = orc.sq_train_uniform(x, bits, metric)
            st = Store(kind, metric, d, bounds=np.array([ulb, udiff], np.float32))
            st.append(orc.squ_encode(x, bits, ulb, udiff, metric))
            stores.append(("uniform%d" % bits, st))
        rot = _rotation(rng, d)
        cen = orc.rabitq_train(x, rot)
        for word in (4, 32, orc.rabitq_bits(32, 4)):
            st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen, qbits=word)
            if word >> 8:
                st.append(orc.rabitq_encode_multibit(x, rot, cen, metric, word >> 8))
            else:
                st.append(orc.rabitq_encode(x, rot, cen, metric, word))
            stores.append(("rabitq%d" % word, st))
    for name, st in stores:
        for i in range(q.shape[0]):
            ids, ds = st.flat_scan(q[i:i + 1], k)
            assert _route(lib)[:2] == (1, 1), name
            sids, sds = _streaming(lib, st, q[i:i + 1], k)
            assert np.array_equal(ids, sids) and np.array_equal(ds.view(np.uint32), sds.view(np.uint32)), name
        st.destroy()


def test_one_query_filter_radius_and_ties(lib):
    lib = lib.load_library()
    rng = np.random.default_rng(9)
    n, d, k = 80000, 32, 20
    st, codes, lb, diff = _sq8_store(rng, n, d, orc.L2)
    q = rng.standard_normal((1, d)).astype(np.float32)
    # a pre-filter that keeps one code in fifty, and one that keeps fewer than k
    for keep_every in (50, 7000):
        deny = np.ones(n, bool)
        deny[::keep_every] = False
        ids, ds = st.flat_scan(q, k, deny=deny)
        sids, sds = _streaming(lib, st, q, k, deny=deny)
        assert np.array_equal(ids, sids) and np.array_equal(ds.view(np.uint32), sds.view(np.uint32))
        valid = ids[0] != 0xFFFFFFFF
        assert valid.sum() == min(k, (~deny).sum()) and not deny[ids[0][valid]].any()
    # a radius between the 5th and 6th distance: five results, the rest empty
    ids, ds = st.flat_scan(q, k)
    radius = 0.5 * (float(ds[0, 4]) + float(ds[0, 5]))
    rids, rds = st.flat_scan(q, k, radius=radius)
    sids, sds = _streaming(lib, st, q, k, radius=radius)
    assert np.array_equal(rids, sids) and np.array_equal(rds.view(np.uint32), sds.view(np.uint32))
    assert np.array_equal(rids[0, :5], ids[0, :5]) and np.all(rids[0, 5:] == 0xFFFFFFFF)
    st.destroy()
    # every code the same: all distances tie, the k smallest ids win, and the admitted keys overflow the sort
    same = np.repeat(codes[:1], n, axis=0)
    st = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    st.append(same)
    ids, ds = st.flat_scan(q, k)
    assert np.array_equal(ids[0], np.arange(k, dtype=np.uint32)) and np.all(ds == ds[0, 0])
    sids, sds = _streaming(lib, st, q, k)
    assert np.array_equal(ids, sids) and np.array_equal(ds.view(np.uint32), sds.view(np.uint32))
    st.destroy()


def test_one_query_through_the_entry_point_that_allocates_nothing(lib):
    """Its fixed scratch holds the distance array of a store this size; a larger store streams instead (checked by
    the route the call reports), with the same result."""
    lib = lib.load_library()
    rng = np.random.default_rng(10)
    n, d, k = 70000, 32, 10
    st, codes, lb, diff = _sq8_store(rng, n, d, orc.L2)
    q = rng.standard_normal((1, d)).astype(np.float32)
    ids, ds = st.flat_scan(q, k)
    from gpu_helpers import dev
    qb = dev(q)
    oi, od = capi.DeviceBuffer(k * 4), capi.DeviceBuffer(k * 4)
    capi.check(lib.vsag_amd_flat_scan_topk_noalloc(st.handle, qb.ptr, 1, k, None, oi.ptr, od.ptr, None))
    capi.check(lib.vsag_amd_stream_synchronize(None))
    assert np.array_equal(oi.to_numpy(np.uint32, (1, k)), ids)
    assert np.array_equal(od.to_numpy(np.uint32, (1, k)), ds.view(np.uint32))
    st.destroy()
