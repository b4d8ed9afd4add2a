"""Seeded random configurations (sizes, dimensions, k, metrics, cluster structure, duplicated queries): the matrix-core
routes of the flat scan (int8 / fp32 pre-selection) and of the posting-list scan (int8 pass) against the streaming
kernels, ids and distance bits."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _same(a, b):
    return np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


@pytest.mark.parametrize("seed", range(12))
def test_random_configuration(lib, seed):
    L = lib.load_library()
    rng = np.random.default_rng(1000 + seed)
    kind = ["sq8", "fp32", "ivf"][seed % 3]
    d = int(rng.choice([16, 24, 32, 48, 64, 96, 100, 128] + ([200, 256] if kind != "ivf" else [])))
    n = int(rng.integers(20000, 200000))
    nq = int(rng.integers(512, 2500))
    k = int(rng.choice([1, 5, 10, 32, 100]))
    metric = int(rng.choice([orc.L2, orc.IP, orc.COSINE]))
    comps = int(rng.choice([1, 5, 50, 500]))
    sigma = float(rng.choice([0.01, 0.05, 0.3]))
    x, means = gaussian_mixture(rng, n, d, comps, sigma)
    q, _ = gaussian_mixture(rng, nq, d, comps, sigma, means=means)
    if rng.random() < 0.4:
        q[: nq // 4] = x[rng.integers(0, n, nq // 4)]  # copies of stored vectors
    buckets = None
    if kind == "sq8":
        lb, diff = orc.sq_train(x, 8, metric)
        st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
        st.append(orc.sq_encode(x, 8, lb, diff, metric))
    elif kind == "fp32":
        st = Store(capi.KIND_FP32, metric, d)
        st.append(x.view(np.uint8).reshape(n, 4 * d))
    else:
        nlist = int(rng.choice([16, 64, 200]))
        nprobe = min(int(rng.choice([4, 8, 16])), nlist)
        nq = max(nq, 8192 * 4 // (nprobe - 1) + 64)  # enough (list, query group) items for the matrix-core pass
        q = np.tile(q, (nq // q.shape[0] + 1, 1))[:nq] + 1e-3 * rng.standard_normal((nq, d)).astype(np.float32)
        cent = x[rng.choice(n, nlist, replace=False)].copy()
        labels, _, _ = orc.kmeans_assign(x, cent)
        l, dd = orc.sq_train_uniform(x, 4, metric, mode=3)
        st = Store(capi.KIND_SQ4_UNIFORM, metric, d, bounds=[l, dd])
        st.set_lists(orc.squ_encode(x, 4, l, dd, metric), labels, nlist)
        buckets, _ = orc.ivf_route(cent, q, nprobe)
    res = {}
    try:
        for mode in ((-1, 0) if kind == "ivf" else (-1, 1, 2)):
            capi.check(L.vsag_amd_set_scan_contraction(mode))
            res[mode] = st.ivf_scan(q, buckets, max(k, 10)) if kind == "ivf" else st.flat_scan(q, k)
            if mode != -1:
                tile = capi.C.c_int()
                L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
                assert tile.value >= 128, "the matrix-core route did not run"
    finally:
        capi.check(L.vsag_amd_set_scan_contraction(0))
    for mode, r in res.items():
        assert _same(res[-1], r), (kind, n, d, nq, k, metric, mode)
    st.destroy()


@pytest.mark.parametrize("seed", range(14))
def test_random_rabitq_configuration(lib, seed):
    """1-bit RaBitQ codes against 4-bit queries: the matrix-core pre-selection against the streaming popcount kernel on
    seeded random sizes, dimensions (padded and unpadded; one to eight granules per code, each of which has a kernel of its
    own), k, metrics, centred and far-off data, duplicated queries."""
    L = lib.load_library()
    rng = np.random.default_rng(2000 + seed)
    d = [32, 100, 128, 200, 384, 512, 600, 640, 768, 800, 896, 960, 64, 256][seed % 14]
    n = int(rng.integers(8000, 60000))
    nq = int(rng.integers(130, 900))
    k = int(rng.choice([1, 10, 50, 100, 200, 256]))
    metric = int(rng.choice([orc.L2, orc.IP]))
    comps = int(rng.choice([1, 5, 50]))
    sigma = float(rng.choice([0.05, 0.3, 1.0]))
    x, means = gaussian_mixture(rng, n, d, comps, sigma)
    q, _ = gaussian_mixture(rng, nq, d, comps, sigma, means=means)
    if seed % 2 == 0:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    if rng.random() < 0.5:
        q[: nq // 4] = x[rng.integers(0, n, nq // 4)]  # copies of stored vectors
    if seed % 3 == 0:
        x[rng.integers(0, n, 40)] = x[0]               # a clump of equal vectors
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    st.append(orc.rabitq_encode(x, rot, cen, metric))
    res = {}
    try:
        for mode in (-1, 1):
            capi.check(L.vsag_amd_set_scan_contraction(mode))
            res[mode] = st.flat_scan(q, k)
            if mode != -1:
                tile = capi.C.c_int()
                L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
                assert tile.value == 128, "the matrix-core route did not run"
    finally:
        capi.check(L.vsag_amd_set_scan_contraction(0))
    assert _same(res[-1], res[1]), (n, d, nq, k, metric)
    st.destroy()


@pytest.mark.parametrize("seed", range(8))
def test_random_uniform_configuration(lib, seed):
    """sq8_uniform and sq4_uniform flat stores: the int8 pre-selection (exact integer products, the l2 form of the test
    for every metric) against the streaming kernel on seeded random configurations."""
    bits = 8 if seed % 2 == 0 else 4
    L = lib.load_library()
    rng = np.random.default_rng(3000 + seed)
    d = int(rng.choice([16, 24, 32, 48, 64, 96, 100, 128]))
    n = int(rng.integers(20000, 200000))
    nq = int(rng.integers(512, 2500))
    k = int(rng.choice([1, 5, 10, 32, 100]))
    metric = int(rng.choice([orc.L2, orc.IP, orc.COSINE]))
    comps = int(rng.choice([1, 5, 50, 500]))
    sigma = float(rng.choice([0.01, 0.05, 0.3]))
    x, means = gaussian_mixture(rng, n, d, comps, sigma)
    q, _ = gaussian_mixture(rng, nq, d, comps, sigma, means=means)
    if rng.random() < 0.4:
        q[: nq // 4] = x[rng.integers(0, n, nq // 4)]
    lb, diff = orc.sq_train_uniform(x, bits, metric, mode=int(rng.choice([1, 3])))
    st = Store(capi.KIND_SQ8_UNIFORM if bits == 8 else capi.KIND_SQ4_UNIFORM, metric, d, bounds=[lb, diff])
    st.append(orc.squ_encode(x, bits, lb, diff, metric))
    res = {}
    try:
        for mode in (-1, 1):
            capi.check(L.vsag_amd_set_scan_contraction(mode))
            res[mode] = st.flat_scan(q, k)
            if mode != -1:
                tile = capi.C.c_int()
                L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
                assert tile.value == 256, "the int8 route did not run"
    finally:
        capi.check(L.vsag_amd_set_scan_contraction(0))
    assert _same(res[-1], res[1]), (bits, n, d, nq, k, metric)
    st.destroy()


@pytest.mark.parametrize("seed", range(12))
def test_random_fp16_configuration(lib, seed):
    """sq8 and sq4 codes of more than 128 dimensions, flat stores and posting lists, on the fp16 matrix cores
    (prefilter_h16.hip): random sizes, dimensions (ragged ones too), k, metric and data spread against the streaming scan."""
    L = lib.load_library()
    rng = np.random.default_rng(7000 + seed)
    bits = [8, 4][seed % 2]
    lists = (seed // 2) % 2 == 1
    d = int(rng.choice([129, 136, 160, 200, 257, 384, 500, 777, 960, 1024]))
    n = int(rng.integers(8000, 60000))
    nq = int(rng.integers(512, 1500))
    k = int(rng.choice([1, 5, 10, 32, 100]))
    metric = int(rng.choice([orc.L2, orc.IP, orc.COSINE]))
    comps = int(rng.choice([1, 5, 50]))
    sigma = float(rng.choice([0.01, 0.05, 0.3]))
    x, means = gaussian_mixture(rng, n, d, comps, sigma)
    q, _ = gaussian_mixture(rng, nq, d, comps, sigma, means=means)
    if rng.random() < 0.4:
        q[: nq // 4] = x[rng.integers(0, n, nq // 4)]
    if rng.random() < 0.5:
        q[nq // 2:] *= np.float32(10.0 ** rng.integers(-4, 5))
    lb, diff = orc.sq_train(x, bits, metric)
    codes = orc.sq_encode(x, bits, lb, diff, metric)
    st = Store(capi.KIND_SQ8 if bits == 8 else capi.KIND_SQ4, metric, d, lb=lb, diff=diff)
    buckets = None
    if lists:
        nlist = int(rng.choice([16, 40]))
        nprobe = int(rng.choice([4, 8]))
        nq = 8192 * 4 // (nprobe - 1) + 64
        q = np.tile(q, (nq // q.shape[0] + 1, 1))[:nq] + 1e-3 * rng.standard_normal((nq, d)).astype(np.float32)
        cent = x[rng.choice(n, nlist, replace=False)].copy()
        labels, _, _ = orc.kmeans_assign(x, cent)
        st.set_lists(codes, labels, nlist)
        buckets, _ = orc.ivf_route(cent, q, nprobe)
    else:
        st.append(codes[: n // 3])
        st.append(codes[n // 3:])
    res = {}
    try:
        for mode in ((-1, 0) if lists else (-1, 1)):
            capi.check(L.vsag_amd_set_scan_contraction(mode))
            res[mode] = st.ivf_scan(q, buckets, max(k, 10)) if lists else st.flat_scan(q, k)
            if mode != -1:
                tile = capi.C.c_int()
                L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
                assert tile.value >= 128, "the matrix-core route did not run"
    finally:
        capi.check(L.vsag_amd_set_scan_contraction(0))
    for mode, r in res.items():
        assert _same(res[-1], r), (bits, lists, n, d, nq, k, metric, mode)
    st.destroy()
