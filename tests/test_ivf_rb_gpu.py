"""Large batches on RaBitQ posting lists (1-bit codes, 4-bit queries): the probe columns behind the first are
pre-selected on the int8 matrix cores from the expanded code bits and what passes is rescored with the streaming
kernel's arithmetic, so ids and distance bits must equal the streaming scan's."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _case(seed, n, d, nlist, nq, metric, components=40, sigma=0.3, unit=False):
    rng = np.random.default_rng(seed)
    x, means = gaussian_mixture(rng, n, d, components, sigma)
    q, _ = gaussian_mixture(rng, nq, d, components, sigma, means=means)
    if unit:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    codes = orc.rabitq_encode(x, rot, cen, metric)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    st.set_lists(codes, labels, nlist)
    return x, q, cent, labels, codes, (rot, cen), st


def _both(lib, st, q, buckets, kcand):
    L = lib.load_library()
    capi.check(L.vsag_amd_store_set_scan_contraction(st.handle, -1))
    plain = st.ivf_scan(q, buckets, kcand)
    capi.check(L.vsag_amd_store_set_scan_contraction(st.handle, -2))
    fast = st.ivf_scan(q, buckets, kcand)
    tile = capi.C.c_int()
    L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
    assert tile.value == 256, "the matrix-core pass did not run"
    return plain, fast


def _same(a, b):
    return np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand,unit", [(60000, 128, 64, 2100, 16, 100, False),
                                                            (30000, 100, 37, 4500, 8, 10, True),
                                                            (20000, 768, 16, 5000, 4, 32, True),
                                                            (20000, 33, 16, 9000, 4, 5, False),
                                                            # the other granule counts (a kernel each): 2, 3, 4, 5, 7, 8
                                                            (12000, 256, 16, 5000, 4, 20, True),
                                                            (12000, 384, 16, 5000, 4, 20, False),
                                                            (12000, 500, 16, 5000, 4, 20, True),
                                                            (12000, 640, 16, 5000, 4, 20, True),
                                                            (12000, 800, 16, 5000, 4, 20, False),
                                                            (12000, 1024, 16, 5000, 4, 20, True)])
def test_matrix_core_columns_equal_streaming(lib, metric, n, d, nlist, nq, nprobe, kcand, unit):
    x, q, cent, labels, codes, (rot, cen), st = _case(n + d + metric, n, d, nlist, nq, metric, unit=unit)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1      # three queries without a first list: no bound, served by the direct fallback launch
    buckets[80, 0] = buckets[80, nprobe - 1]  # a far list first (and probed twice): a loose bound
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    # and the checker on a sample
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qcodes = orc.rabitq_process_query(q[:32], rot, cen, metric)
    rids, rds = orc.ivf_scan(orc.RABITQ, metric, d, codes[order], offsets, order, qcodes, buckets[:32], kcand)
    assert_topk_close(fast[0][:32], fast[1][:32], rids, rds, atol=2e-5, label="ivf rabitq on the matrix cores")
    st.destroy()


def test_overflow_missing_buckets_and_equal_vectors(lib):
    """Far lists first (loose bounds: private lists overflow and the queries go back to the streaming kernel), ragged
    bucket rows, and a clump of equal vectors (codes outside the estimator's derivation are candidates of everyone)."""
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 8, 9000, 4, 10
    x, q, cent, labels, codes, _, st = _case(11, n, d, nlist, nq, orc.L2, components=8, sigma=0.1)
    routed, _ = orc.ivf_route(cent, q, nlist)
    buckets = np.ascontiguousarray(routed[:, [nlist - 1, 0, 1, 2]])
    buckets[1::7, 2:] = -1
    buckets[3::11, 0] = -1
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_vectors_equal_to_the_centroid(lib):
    """Rows equal to the trained centroid have zero norm after centring: outside the derivation of the threshold, so
    they are candidates of every query that probes their list."""
    n, d, nlist, nq, nprobe, kcand = 20000, 96, 16, 6000, 6, 20
    rng = np.random.default_rng(4)
    x, means = gaussian_mixture(rng, n, d, 20, 0.3)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.3, means=means)
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    x[5::1000] = cen
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    codes = orc.rabitq_encode(x, rot, cen, orc.L2)
    st = Store(capi.KIND_RABITQ, orc.L2, d, rot=rot, centroid=cen)
    st.set_lists(codes, labels, nlist)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_one_long_list_among_short_and_empty_ones(lib):
    """A list long enough for several chunks of the matrix-core pass (128 tiles each), lists of a single code and lists
    without any."""
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 40, 6000, 6, 20
    rng = np.random.default_rng(12)
    x, means = gaussian_mixture(rng, n, d, 30, 0.3)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.3, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    labels = labels.copy()
    labels[rng.random(n) < 0.45] = 7          # about 18 000 codes: three chunks
    labels[labels == 3] = 7                   # list 3 is empty
    labels[labels == 4] = 7
    labels[11] = 4                            # list 4 holds one code
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    codes = orc.rabitq_encode(x, rot, cen, orc.L2)
    st = Store(capi.KIND_RABITQ, orc.L2, d, rot=rot, centroid=cen)
    st.set_lists(codes, labels, nlist)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[::2, 1] = 7
    buckets[1::2, 2] = 3
    buckets[::5, 3] = 4
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_lists_grown_by_appends_keep_their_matrix_core_copies(lib):
    """The store keeps the code bits and per-code constants of rabitq lists once more for the matrix cores and renews
    them whenever codes are added (lists outgrow their room and move): a store grown in ragged pieces, one of them into
    empty lists, must answer like one built at once, on both paths."""
    from gpu_helpers import dev
    n, d, nlist, nq, nprobe, kcand, metric = 30000, 200, 24, 4000, 6, 40, orc.L2
    x, q, cent, labels, codes, (rot, cen), whole = _case(91, n, d, nlist, nq, metric)
    grown = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    grown.set_lists(codes[:1], labels[:1], nlist)
    L = lib.load_library()
    at = 1
    for step in (63, 1, 500, 7000, 64, 9000, n):
        end = min(n, at + step)
        if end > at:
            cbuf, lbuf = dev(np.ascontiguousarray(codes[at:end])), dev(np.ascontiguousarray(labels[at:end], np.int32))
            capi.check(L.vsag_amd_store_append_lists(grown.handle, cbuf.ptr, lbuf.ptr, None, end - at, None))
            cbuf.free()
            lbuf.free()
        at = end
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    plain_w, fast_w = _both(lib, whole, q, buckets, kcand)
    plain_g, fast_g = _both(lib, grown, q, buckets, kcand)
    assert _same(plain_w, fast_w) and _same(plain_g, fast_g)
    # the two stores hold the same codes under the same ids (lists in another order of arrival: ties aside, the same answers)
    assert np.array_equal(fast_w[1].view(np.uint32), fast_g[1].view(np.uint32))
    whole.destroy()
    grown.destroy()
