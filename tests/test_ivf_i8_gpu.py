"""Large batches on sq4_uniform and sq8_uniform posting lists: the probe columns behind the first go through the
int8 matrix cores.  The integer test selects exactly what the streaming kernel would admit and the distances are formed by the
same operations, so ids and distance bits must equal the streaming scan's (and the checker's distances)."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _case(seed, n, d, nlist, nq, components=40, sigma=0.05, metric=orc.L2, bits=4):
    rng = np.random.default_rng(seed)
    x, means = gaussian_mixture(rng, n, d, components, sigma)
    q, _ = gaussian_mixture(rng, nq, d, components, sigma, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    l, dd = orc.sq_train_uniform(x, bits, metric, mode=3)
    codes = orc.squ_encode(x, bits, l, dd, metric)
    st = Store(capi.KIND_SQ4_UNIFORM if bits == 4 else capi.KIND_SQ8_UNIFORM, metric, d, bounds=[l, dd])
    st.set_lists(codes, labels, nlist)
    return x, q, cent, labels, codes, (l, dd), st


def _both(lib, st, q, buckets, kcand):
    L = lib.load_library()
    capi.check(L.vsag_amd_set_scan_contraction(-1))
    try:
        plain = st.ivf_scan(q, buckets, kcand)
    finally:
        capi.check(L.vsag_amd_set_scan_contraction(0))
    fast = st.ivf_scan(q, buckets, kcand)
    tile = capi.C.c_int()
    L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
    assert tile.value == 256, "the matrix-core pass did not run"
    return plain, fast


def _same(a, b):
    return np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand", [(60000, 128, 64, 2100, 16, 100), (30000, 100, 37, 4500, 8, 10),
                                                       (20000, 32, 16, 9000, 4, 32)])
def test_matrix_core_columns_equal_streaming(lib, n, d, nlist, nq, nprobe, kcand):
    x, q, cent, labels, codes, (l, dd), st = _case(n + d, n, d, nlist, nq)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1      # three queries without a first list: no bound, served by the direct fallback launch
    buckets[80, 0] = buckets[80, nprobe - 1]  # a far list first (and probed twice): a loose bound
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    # and the checker's distances, bit for bit, on a sample
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qproc = orc.squ_encode(q[:64], 4, l, dd, orc.L2)
    _, rds = orc.ivf_scan(orc.SQ4U, orc.L2, d, codes[order], offsets, order, qproc, buckets[:64], kcand, lb=l, diff=dd)
    assert np.array_equal(fast[1][:64].view(np.uint32), rds.view(np.uint32))
    st.destroy()


def test_overflowing_lists_fall_back_to_streaming(lib):
    """Queries routed to a far list first: the bound the first column leaves is so loose that the other lists hold
    hundreds of better codes, more than a private list takes; those queries go back to the streaming kernel."""
    # 12 000 queries x 3 columns: more gated pairs than the direct fallback launch takes (32 768), so the streaming
    # kernel serves them over the per-list grouping
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 8, 12000, 4, 10
    x, q, cent, labels, codes, (l, dd), st = _case(11, n, d, nlist, nq, components=8, sigma=0.02)
    routed, _ = orc.ivf_route(cent, q, nlist)
    buckets = np.ascontiguousarray(routed[:, [nlist - 1, 0, 1, 2]])  # farthest list first, then the nearest three
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_missing_buckets_and_ragged_lists(lib):
    n, d, nlist, nq, nprobe, kcand = 30000, 128, 50, 3000, 12, 20
    x, q, cent, labels, codes, (l, dd), st = _case(5, n, d, nlist, nq)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[::3, 5:] = -1       # fewer lists than columns
    buckets[1::7, 0] = -1       # no first list at all: no bound, everything overflows
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("metric", [orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand", [(60000, 128, 64, 2100, 16, 100), (30000, 100, 37, 4500, 8, 10),
                                                       (20000, 7, 16, 9000, 4, 5)])
def test_inner_product_and_cosine_columns_equal_streaming(lib, bits, metric, n, d, nlist, nq, nprobe, kcand):
    """No integer form for these metrics: a float threshold with every rounding charged against it, then the
    streaming kernel's own operations on what passes.  Byte codes (sq8_uniform): the same test on the product of the
    centred operands."""
    x, q, cent, labels, codes, (l, dd), st = _case(n + d + metric, n, d, nlist, nq, metric=metric, bits=bits)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qproc = orc.squ_encode(q[:64], bits, l, dd, metric)
    _, rds = orc.ivf_scan(orc.SQ4U if bits == 4 else orc.SQ8U, metric, d, codes[order], offsets, order, qproc, buckets[:64],
                          kcand, lb=l, diff=dd)
    assert np.array_equal(fast[1][:64].view(np.uint32), rds.view(np.uint32))
    st.destroy()


@pytest.mark.parametrize("n,d,nlist,nq,nprobe,kcand", [(60000, 128, 64, 2100, 16, 100), (30000, 100, 37, 4500, 8, 10),
                                                       (20000, 33, 16, 9000, 4, 32), (20000, 7, 16, 9000, 4, 5)])
def test_sq8_uniform_l2_columns_equal_streaming(lib, n, d, nlist, nq, nprobe, kcand):
    """sq8_uniform under l2 (sq8_uniform_quantizer.cpp:204-250): byte values on both sides, centred by 128 for the
    signed matrix instruction; the product is put right with the sums of the code and of the query, so ids and distance
    bits equal the streaming scan's and the checker's.  Dimensions that fill neither a dword nor a granule included."""
    x, q, cent, labels, codes, (l, dd), st = _case(n + d + 8, n, d, nlist, nq, bits=8)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1
    buckets[80, 0] = buckets[80, nprobe - 1]
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    qproc = orc.squ_encode(q[:64], 8, l, dd, orc.L2)
    _, rds = orc.ivf_scan(orc.SQ8U, orc.L2, d, codes[order], offsets, order, qproc, buckets[:64], kcand, lb=l, diff=dd)
    assert np.array_equal(fast[1][:64].view(np.uint32), rds.view(np.uint32))
    st.destroy()


def test_sq8_uniform_l2_extreme_codes(lib):
    """Codes and queries at the ends of the byte range (all 0, all 255, alternating): the centred product and the
    terms that put it right reach their largest magnitudes."""
    n, d, nlist, nq, nprobe, kcand = 16384, 128, 8, 8192, 4, 10
    rng = np.random.default_rng(3)
    x = rng.random((n, d), dtype=np.float32)
    x[::5] = 0.0
    x[1::5] = 1.0
    x[2::5, ::2] = 0.0
    x[2::5, 1::2] = 1.0
    q = rng.random((nq, d), dtype=np.float32)
    q[::4] = 1.0
    q[1::4] = 0.0
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels = (np.arange(n) % nlist).astype(np.int32)
    l, dd = np.float32(0.0), np.float32(1.0)
    codes = orc.squ_encode(x, 8, l, dd, orc.L2)
    st = Store(capi.KIND_SQ8_UNIFORM, orc.L2, d, bounds=[l, dd])
    st.set_lists(codes, labels, nlist)
    buckets = np.tile(np.arange(nprobe, dtype=np.int32), (nq, 1))
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_sq8_uniform_l2_appended_lists(lib):
    """Codes appended to the lists afterwards carry their sums like the first batch (and through a move of the lists)."""
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 16, 6000, 8, 10
    x, q, cent, labels, codes, (l, dd), st = _case(77, n, d, nlist, nq, bits=8)
    st.destroy()
    st = Store(capi.KIND_SQ8_UNIFORM, orc.L2, d, bounds=[l, dd])
    st.set_lists(codes[:10000], labels[:10000], nlist)
    st.append_lists(codes[10000:], labels[10000:])
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    whole = Store(capi.KIND_SQ8_UNIFORM, orc.L2, d, bounds=[l, dd])
    whole.set_lists(codes, labels, nlist)
    ref = whole.ivf_scan(q, buckets, kcand)
    assert _same(ref, fast)
    whole.destroy()
    st.destroy()
