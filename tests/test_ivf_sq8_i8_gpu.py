"""Large batches on sq8 (and sq4) posting lists of at most 128 dimensions: the probe columns behind the first are
pre-selected on the int8 matrix cores (two int8 planes per query, one scale for the batch) and what passes is rescored
with the streaming kernel's arithmetic, so ids and distance bits must equal the streaming scan's."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _case(seed, n, d, nlist, nq, components=40, sigma=0.05, metric=orc.L2, bits=8):
    rng = np.random.default_rng(seed)
    x, means = gaussian_mixture(rng, n, d, components, sigma)
    q, _ = gaussian_mixture(rng, nq, d, components, sigma, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    lb, diff = orc.sq_train(x, bits, metric)
    codes = orc.sq_encode(x, bits, lb, diff, metric)
    st = Store(capi.KIND_SQ8 if bits == 8 else capi.KIND_SQ4, metric, d, lb=lb, diff=diff)
    st.set_lists(codes, labels, nlist)
    return x, q, cent, labels, codes, (lb, diff), st


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


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand", [(60000, 128, 64, 2100, 16, 100), (30000, 100, 37, 4500, 8, 10),
                                                       (20000, 33, 16, 9000, 4, 32), (20000, 7, 16, 9000, 4, 5)])
def test_matrix_core_columns_equal_streaming(lib, bits, metric, n, d, nlist, nq, nprobe, kcand):
    x, q, cent, labels, codes, (lb, diff), st = _case(n + d + metric, n, d, nlist, nq, metric=metric, bits=bits)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1      # three queries without a first list: no bound, served by the direct fallback launch
    buckets[80, 0] = buckets[80, nprobe - 1]  # a far list first (and probed twice): a loose bound
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    # and the checker on a sample
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qs, om = q[:64], metric
    if metric == orc.COSINE:  # inner product of the unit query with the codes of the unit rows
        qs, om = (qs / np.linalg.norm(qs, axis=1, keepdims=True)).astype(np.float32), orc.IP
    rids, rds = orc.ivf_scan(orc.SQ8 if bits == 8 else orc.SQ4, om, d, codes[order], offsets, order, qs, buckets[:64], kcand,
                             lb=lb, diff=diff)
    assert_topk_close(fast[0][:64], fast[1][:64], rids, rds, atol=4e-6, label="ivf sq8 on the matrix cores")
    st.destroy()


def test_overflowing_lists_fall_back_to_streaming(lib):
    """Queries routed to a far list first: the bound the first column leaves is so loose that the other lists hold
    hundreds of better codes, more than a private list takes; those queries go back to the streaming kernel."""
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 8, 9000, 4, 10
    x, q, cent, labels, codes, _, st = _case(11, n, d, nlist, nq, components=8, sigma=0.02)
    routed, _ = orc.ivf_route(cent, q, nlist)
    buckets = np.ascontiguousarray(routed[:, [nlist - 1, 0, 1, 2]])  # farthest list first, then the nearest three
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_missing_buckets_and_ragged_lists(lib):
    n, d, nlist, nq, nprobe, kcand = 30000, 128, 50, 3000, 12, 20
    x, q, cent, labels, codes, _, st = _case(5, n, d, nlist, nq)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[::3, 5:] = -1       # fewer lists than columns
    buckets[1::7, 0] = -1       # no first list at all: no bound, everything overflows
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_queries_of_very_different_sizes_share_one_scale(lib):
    """The batch shares the scale of its largest query: small queries lose resolution (more candidates), never a
    result.  A few queries a thousand times the others, some all zero, one with a NaN."""
    n, d, nlist, nq, nprobe, kcand = 30000, 64, 32, 6000, 8, 10
    x, q, cent, labels, codes, _, st = _case(21, n, d, nlist, nq)
    q = q.copy()
    q[5::500] *= 1000.0
    q[7::900] = 0.0
    q[11, 3] = np.nan
    buckets, _ = orc.ivf_route(cent, np.nan_to_num(q), nprobe)
    plain, fast = _both(lib, st, q, buckets, kcand)
    ok = np.ones(nq, bool)
    ok[11] = False  # NaN distances order as the streaming kernel leaves them; ids are compared for the others
    assert np.array_equal(plain[0][ok], fast[0][ok])
    assert np.array_equal(plain[1][ok].view(np.uint32), fast[1][ok].view(np.uint32))
    st.destroy()


@pytest.mark.parametrize("bits", [8, 4])
def test_lists_that_grew_by_appending(lib, bits):
    """The per-slot terms are renewed when codes are appended (lists move, room behind each list holds no code)."""
    n, d, nlist, nq, nprobe, kcand = 40000, 96, 24, 6000, 6, 20
    rng = np.random.default_rng(2)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    kind = capi.KIND_SQ8 if bits == 8 else capi.KIND_SQ4
    lb, diff = orc.sq_train(x, bits)
    codes = orc.sq_encode(x, bits, lb, diff)
    st = Store(kind, orc.L2, d, lb=lb, diff=diff)
    half = n // 2
    st.set_lists(codes[:half], labels[:half], nlist)
    st.append_lists(codes[half:half + 7000], labels[half:half + 7000])
    st.append_lists(codes[half + 7000:], labels[half + 7000:])
    whole = Store(kind, orc.L2, d, lb=lb, diff=diff)
    whole.set_lists(codes, labels, nlist)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    ref = whole.ivf_scan(q, buckets, kcand)
    assert np.array_equal(ref[1].view(np.uint32), fast[1].view(np.uint32))
    st.destroy()
    whole.destroy()


@pytest.mark.parametrize("bits", [8, 4])
def test_one_long_list_among_short_and_empty_ones(lib, bits):
    """A list long enough for all four chunks of the matrix-core pass, lists of a single code and lists without any."""
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 40, 6000, 6, 20
    rng = np.random.default_rng(12)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    labels = labels.copy()
    labels[rng.random(n) < 0.45] = 7          # about 18 000 codes: four chunks of 70 tiles
    labels[labels == 3] = 7                   # list 3 is empty
    labels[labels == 4] = 7
    labels[11] = 4                            # list 4 holds one code
    lb, diff = orc.sq_train(x, bits)
    codes = orc.sq_encode(x, bits, lb, diff)
    st = Store(capi.KIND_SQ8 if bits == 8 else capi.KIND_SQ4, orc.L2, d, lb=lb, diff=diff)
    st.set_lists(codes, labels, nlist)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[::2, 1] = 7
    buckets[1::2, 2] = 3
    buckets[::5, 3] = 4
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand", [(20000, 200, 20, 7000, 6, 10), (12000, 960, 16, 9000, 4, 32)])
def test_sq4_lists_beyond_128_dimensions_on_the_fp16_matrix_cores(lib, metric, n, d, nlist, nq, nprobe, kcand):
    """sq4 posting lists of more than 128 dimensions: the nibbles and the fp16 value of the scaled query on
    v_mfma_f32_32x32x16_f16 (ivf_h16_kernel), records rescored with the streaming arithmetic: ids and distance bits equal
    the streaming scan's."""
    x, q, cent, labels, codes, (lb, diff), st = _case(n + d + metric, n, d, nlist, nq, metric=metric, bits=4)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1
    buckets[80, 0] = buckets[80, nprobe - 1]
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qs, om = q[:32], metric
    if metric == orc.COSINE:
        qs, om = (qs / np.linalg.norm(qs, axis=1, keepdims=True)).astype(np.float32), orc.IP
    rids, rds = orc.ivf_scan(orc.SQ4, om, d, codes[order], offsets, order, qs, buckets[:32], kcand, lb=lb, diff=diff)
    assert_topk_close(fast[0][:32], fast[1][:32], rids, rds, rtol=2e-5, atol=1e-5, tie_rtol=2e-5,
                      label="ivf sq4 beyond 128 dimensions on the matrix cores")
    st.destroy()
