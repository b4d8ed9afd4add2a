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
