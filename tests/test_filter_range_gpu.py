"""Pre-filter (deny mask over inner ids) and range limit of the flat and posting-list scans.

The checker has no filter argument; a filtered scan must equal the checker's scan of the allowed codes alone
(ids mapped back), and a range scan the checker's top-k cut at the radius."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _sq8_store(rng, n, d, metric):
    x, means = gaussian_mixture(rng, n, d, 20, 0.05)
    lb, diff = orc.sq_train(x, 8, metric)
    codes = orc.sq_encode(x, 8, lb, diff, metric)
    st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    st.append(codes)
    return st, codes, lb, diff, means


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("n,d,nq,k,deny_rate", [(30000, 128, 33, 10, 0.5), (5000, 33, 1, 10, 0.99), (700, 16, 5, 100, 0.9),
                                                (64, 8, 2, 10, 1.0)])
def test_flat_scan_with_deny_mask(lib, metric, n, d, nq, k, deny_rate):
    rng = np.random.default_rng(n + d + k)
    st, codes, lb, diff, means = _sq8_store(rng, n, d, metric)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    deny = rng.random(n) < deny_rate
    allowed = np.nonzero(~deny)[0]
    ids, ds = st.flat_scan(q, k, deny=deny)
    assert not np.any(deny[ids[ids != 0xFFFFFFFF]]), "a filtered-out id was returned"
    if allowed.size == 0:
        assert np.all(ids == 0xFFFFFFFF) and np.all(np.isinf(ds))
    else:
        kk = min(k, allowed.size)
        ri, rd = orc.flat_scan_topk(orc.SQ8, metric, d, codes[allowed], q, kk, lb=lb, diff=diff)
        full_i = np.full((nq, k), 0xFFFFFFFF, np.uint32)
        full_d = np.full((nq, k), np.inf, np.float32)
        full_i[:, :kk] = allowed[ri].astype(np.uint32)
        full_d[:, :kk] = rd
        assert_topk_close(ids, ds, full_i, full_d, label="deny %.2f" % deny_rate)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
def test_flat_scan_with_radius(lib, metric):
    rng = np.random.default_rng(91)
    n, d, nq, k = 20000, 64, 16, 50
    st, codes, lb, diff, means = _sq8_store(rng, n, d, metric)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    ri, rd = orc.flat_scan_topk(orc.SQ8, metric, d, codes, q, k, lb=lb, diff=diff)
    # radii that cut every row somewhere in the middle, nowhere, and everywhere
    for radius in (float(np.median(rd[:, k // 3])), float(rd.max()) + 1.0, float(rd.min()) - 1.0):
        ids, ds = st.flat_scan(q, k, radius=radius)
        keep = rd <= radius
        exp_i = np.where(keep, ri, 0xFFFFFFFF).astype(np.uint32)
        exp_d = np.where(keep, rd, np.inf).astype(np.float32)
        # rows whose cut falls within rounding of the radius may differ by that one candidate
        finite = np.isfinite(ds)
        assert np.all(ds[finite] <= radius)
        edge = np.abs(rd - radius) <= 1e-5 * abs(radius)
        rows = ~edge.any(axis=1)
        assert_topk_close(ids[rows], ds[rows], exp_i[rows], exp_d[rows], label="radius %g" % radius)
    # both at once
    deny = rng.random(n) < 0.3
    radius = float(np.median(rd[:, k // 2]))
    ids, ds = st.flat_scan(q, k, deny=deny, radius=radius)
    got = ids[ids != 0xFFFFFFFF]
    assert not np.any(deny[got]) and np.all(ds[np.isfinite(ds)] <= radius)
    st.destroy()


def test_ivf_scan_with_deny_mask_and_radius(lib):
    rng = np.random.default_rng(17)
    n, d, nlist, nq, nprobe, kcand = 20000, 64, 50, 24, 10, 40
    x, means = gaussian_mixture(rng, n, d, 40, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 40, 0.05, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    l, dd = orc.sq_train_uniform(x, 4, orc.L2, mode=3)
    codes = orc.squ_encode(x, 4, l, dd, orc.L2)
    st = Store(capi.KIND_SQ4_UNIFORM, orc.L2, d, bounds=[l, dd])
    st.set_lists(codes, labels, nlist)
    deny = rng.random(n) < 0.6
    ids, ds = st.ivf_scan(q, buckets, kcand, deny=deny)
    assert not np.any(deny[ids[ids != 0xFFFFFFFF]])
    # the checker on lists that hold the allowed vectors only (labels of the others point nowhere)
    allowed = np.nonzero(~deny)[0]
    offsets, order = orc.ivf_build_lists(labels[allowed], nlist)
    qcodes = orc.squ_encode(q, 4, l, dd, orc.L2)
    ri, rd = orc.ivf_scan(orc.SQ4U, orc.L2, d, codes[allowed][order], offsets, order, qcodes, buckets, kcand, lb=l, diff=dd)
    ri = np.where(ri == 0xFFFFFFFF, ri, allowed[np.minimum(ri, allowed.size - 1)].astype(np.uint32))
    assert np.array_equal(ds.view(np.uint32), rd.view(np.uint32))
    assert_topk_close(ids, ds, ri, rd, rtol=0, atol=0, tie_rtol=0, label="ivf deny")
    # range: integer distances, so the cut is exact
    radius = float(np.median(rd[np.isfinite(rd)]))
    ids2, ds2 = st.ivf_scan(q, buckets, kcand, deny=deny, radius=radius)
    exp_d = np.where(rd <= radius, rd, np.inf).astype(np.float32)
    assert np.array_equal(ds2.view(np.uint32), exp_d.view(np.uint32))
    assert np.all((ids2 == 0xFFFFFFFF) == np.isinf(exp_d))
    st.destroy()
