"""Parity of the HIP flat scan + fused top-k against the CPU checker, through the C ABI.

Tolerances (stated by the task): float distances within 1e-4 relative; top-k ids identical where distance
gaps exceed the tie band; integer paths (uniform codes) produce bit-identical distances."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, gaussian_mixture

pytestmark = pytest.mark.gpu

METRICS = [(orc.L2, "l2"), (orc.IP, "ip")]


def _sq_case(rng, n, d, nq, bits):
    x, means = gaussian_mixture(rng, n, d, 20, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    lb, diff = orc.sq_train(x, bits)
    codes = orc.sq_encode(x, bits, lb, diff)
    return x, q, lb, diff, codes


@pytest.mark.parametrize("metric,mname", METRICS)
@pytest.mark.parametrize("n,d,nq,k", [(20000, 128, 37, 10), (1000, 33, 5, 10), (63, 7, 3, 4), (1, 16, 2, 3),
                                      (5000, 960, 9, 100)])
def test_sq8_flat_scan(lib, metric, mname, n, d, nq, k):
    rng = np.random.default_rng(47 + n + d)
    x, q, lb, diff, codes = _sq_case(rng, n, d, nq, 8)
    st = Store(lib.KIND_SQ8, metric, d, lb=lb, diff=diff)
    st.append(codes)
    assert st.size() == n
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(orc.SQ8, metric, d, codes, q, k, lb=lb, diff=diff)
    assert_topk_close(ids, ds, rids, rds, label="sq8 %s n=%d d=%d" % (mname, n, d))
    st.destroy()


@pytest.mark.parametrize("metric,mname", METRICS)
@pytest.mark.parametrize("n,d,nq,k", [(8000, 128, 17, 10), (500, 65, 4, 7)])
def test_sq4_flat_scan(lib, metric, mname, n, d, nq, k):
    rng = np.random.default_rng(48 + n + d)
    x, q, lb, diff, codes = _sq_case(rng, n, d, nq, 4)
    st = Store(lib.KIND_SQ4, metric, d, lb=lb, diff=diff)
    st.append(codes)
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(orc.SQ4, metric, d, codes, q, k, lb=lb, diff=diff)
    assert_topk_close(ids, ds, rids, rds, label="sq4 %s n=%d d=%d" % (mname, n, d))
    st.destroy()


@pytest.mark.parametrize("metric,mname", METRICS + [(orc.COSINE, "cosine")])
@pytest.mark.parametrize("n,d,nq,k", [(10000, 128, 21, 10), (300, 9, 3, 5), (4000, 960, 6, 64)])
def test_fp32_flat_scan(lib, metric, mname, n, d, nq, k):
    rng = np.random.default_rng(49 + n + d)
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((nq, d), dtype=np.float32)
    st = Store(lib.KIND_FP32, metric, d)
    st.append(x.view(np.uint8).reshape(n, 4 * d))
    ids, ds = st.flat_scan(q, k)
    if metric == orc.COSINE:
        xn = x / np.sqrt((x.astype(np.float64) ** 2).sum(1, keepdims=True)).astype(np.float32)
        qn = q / np.sqrt((q.astype(np.float64) ** 2).sum(1, keepdims=True)).astype(np.float32)
        rids, rds = orc.flat_scan_topk(orc.FP32, orc.IP, d, xn.view(np.uint8).reshape(n, 4 * d), qn, k)
        assert_topk_close(ids, ds, rids, rds, atol=2e-6, label="fp32 cosine")
    else:
        rids, rds = orc.flat_scan_topk(orc.FP32, metric, d, x.view(np.uint8).reshape(n, 4 * d), q, k)
        assert_topk_close(ids, ds, rids, rds, atol=2e-6, label="fp32 %s n=%d d=%d" % (mname, n, d))
    st.destroy()


@pytest.mark.parametrize("metric,mname", METRICS)
@pytest.mark.parametrize("bits,kind", [(4, "sq4u"), (8, "sq8u")])
@pytest.mark.parametrize("n,d,nq,k", [(12000, 128, 19, 10), (700, 33, 4, 100)])
def test_uniform_flat_scan_bit_exact(lib, metric, mname, bits, kind, n, d, nq, k):
    rng = np.random.default_rng(50 + n + d + bits)
    x, means = gaussian_mixture(rng, n, d, 20, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    okind = orc.SQ4U if bits == 4 else orc.SQ8U
    lkind = lib.KIND_SQ4_UNIFORM if bits == 4 else lib.KIND_SQ8_UNIFORM
    lb, diff = orc.sq_train_uniform(x, bits, metric, mode=3 if bits == 4 else 1)
    codes = orc.squ_encode(x, bits, lb, diff, metric)
    qcodes = orc.squ_encode(q, bits, lb, diff, metric)
    st = Store(lkind, metric, d, bounds=[lb, diff])
    st.append(codes)
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(okind, metric, d, codes, qcodes, k, lb=lb, diff=diff)
    # integer inner products: the distance multiset must be identical bit for bit for L2; the IP form has
    # three float operations whose order is kept, so it is bit-exact as well.
    assert np.array_equal(ds.view(np.uint32), rds.view(np.uint32)), "%s %s distances differ" % (kind, mname)
    assert_topk_close(ids, ds, rids, rds, rtol=0, atol=0, tie_rtol=0, label=kind)
    st.destroy()


def test_append_in_pieces_equals_one_append(lib):
    rng = np.random.default_rng(7)
    n, d = 3000, 48
    x, q, lb, diff, codes = _sq_case(rng, n, d, 6, 8)
    a = Store(lib.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    a.append(codes)
    b = Store(lib.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    for s, e in [(0, 1), (1, 64), (64, 1000), (1000, 1001), (1001, 3000)]:
        b.append(codes[s:e])
    ia, da = a.flat_scan(q, 10)
    ib, db = b.flat_scan(q, 10)
    assert np.array_equal(ia, ib) and np.array_equal(da, db)
    a.destroy()
    b.destroy()


@pytest.mark.parametrize("kind,d", [("sq8", 128), ("sq8", 16), ("fp32", 128), ("sq4u", 128), ("fp32", 4)])
@pytest.mark.parametrize("n", [1024, 2048, 16384])
def test_store_filled_to_the_last_tile_of_its_buffer(lib, kind, d, n):
    """A store grows by doubling from 16 tiles, so these sizes fill the tile buffer to its last byte.  The scan fetches
    tile rows in groups with fixed offsets and no branch around a load, which reads past the last tile by design: the
    buffer ends with slack for that, and nothing read there may reach a result.  One query per call (eight rows per
    group) and a small batch."""
    rng = np.random.default_rng(n + d)
    x, means = gaussian_mixture(rng, n, d, 10, 0.05)
    q, _ = gaussian_mixture(rng, 9, d, 10, 0.05, means=means)
    if kind == "sq8":
        lb, diff = orc.sq_train(x, 8)
        codes = orc.sq_encode(x, 8, lb, diff)
        st = Store(lib.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
        ref = lambda qq, k: orc.flat_scan_topk(orc.SQ8, orc.L2, d, codes, qq, k, lb=lb, diff=diff)
    elif kind == "sq4u":
        lb, diff = orc.sq_train_uniform(x, 4, orc.L2, mode=3)
        codes = orc.squ_encode(x, 4, lb, diff, orc.L2)
        st = Store(lib.KIND_SQ4_UNIFORM, orc.L2, d, bounds=[lb, diff])
        ref = lambda qq, k: orc.flat_scan_topk(orc.SQ4U, orc.L2, d, codes, orc.squ_encode(qq, 4, lb, diff, orc.L2), k,
                                               lb=lb, diff=diff)
    else:
        codes = x.view(np.uint8).reshape(n, 4 * d)
        st = Store(lib.KIND_FP32, orc.L2, d)
        ref = lambda qq, k: orc.flat_scan_topk(orc.FP32, orc.L2, d, codes, qq, k)
    # in pieces, so that the buffer has grown (and been copied) several times on the way
    st.append(codes[:1000])
    st.append(codes[1000:n - 1])
    st.append(codes[n - 1:])
    assert st.size() == n
    for qq in (q[:1], q):
        ids, ds = st.flat_scan(qq, 10)
        rids, rds = ref(qq, 10)
        assert_topk_close(ids, ds, rids, rds, atol=2e-6, label="%s filled to capacity" % kind)
        assert ids.max() < n
    st.destroy()


def test_empty_store_and_bad_arguments(lib):
    st = Store(lib.KIND_FP32, orc.L2, 8)
    ids, ds = st.flat_scan(np.zeros((2, 8), np.float32), 3)
    assert np.all(ids == 0xFFFFFFFF) and np.all(np.isinf(ds))
    import ctypes as C
    rc = lib.load_library().vsag_amd_flat_scan_topk(st.handle, None, 1, 0, None, None, None, 0, None)
    assert rc == lib.INVALID_ARGUMENT
    assert b"k must be" in lib.load_library().vsag_amd_last_error()
    st.destroy()


def _unit_rows(a):
    """Rows divided by their norm; a zero row divides by 1 (DivScalarImpl, simd/kernels/scalar_op.h:40-42)."""
    norm = np.sqrt((a.astype(np.float64) ** 2).sum(1, keepdims=True)).astype(np.float32)
    norm[norm == 0] = 1.0
    return (a / norm).astype(np.float32)


@pytest.mark.parametrize("kind", ["fp32", "sq8"])
@pytest.mark.parametrize("contraction", [0, 1])
def test_cosine_with_zero_rows_and_a_zero_query(lib, kind, contraction):
    """A zero base row and a zero query under cosine: the reference divides by 1 instead of by the zero norm, so the
    distance is 1 - 0 = 1 and nothing turns into NaN; the other queries' results do not change."""
    rng = np.random.default_rng(91)
    n, d, nq, k = 70000 if contraction else 3000, 64, 6, 10
    x = (rng.random((n, d), dtype=np.float32) - 0.3).astype(np.float32)
    x[17] = 0.0
    x[n - 5] = 0.0
    q = (rng.random((nq, d), dtype=np.float32) - 0.3).astype(np.float32)
    q[2] = 0.0
    l = lib.load_library()
    if kind == "fp32":
        st = Store(lib.KIND_FP32, orc.COSINE, d)
        st.append(x.view(np.uint8).reshape(n, 4 * d))
        ref = lambda qq: orc.flat_scan_topk(orc.FP32, orc.IP, d, _unit_rows(x).view(np.uint8).reshape(n, 4 * d), qq, k)
    else:
        lb, diff = orc.sq_train(x, 8, orc.COSINE)
        codes = orc.sq_encode(x, 8, lb, diff, orc.COSINE)
        st = Store(lib.KIND_SQ8, orc.COSINE, d, lb=lb, diff=diff)
        st.append(codes)
        ref = lambda qq: orc.flat_scan_topk(orc.SQ8, orc.IP, d, codes, qq, k, lb=lb, diff=diff)
    lib.check(l.vsag_amd_set_scan_contraction(contraction))
    try:
        ids, ds = st.flat_scan(q, k)
    finally:
        lib.check(l.vsag_amd_set_scan_contraction(0))
    assert not np.isnan(ds).any(), "a zero norm must not produce NaN distances"
    rids, rds = ref(_unit_rows(q))
    assert_topk_close(ids, ds, rids, rds, atol=2e-6, label="%s cosine with zero rows" % kind)
    if kind == "fp32":
        assert np.all(ds[2] == 1.0), "a zero query is at distance 1 from everything"
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(4096, 128, 1500, 64), (5000, 100, 1030, 10), (8192, 32, 2000, 1), (1024, 16, 1100, 256),
                                      (3000, 30, 1024, 100), (2047, 7, 1300, 5)])
def test_many_queries_against_a_small_fp32_store(lib, metric, n, d, nq, k):
    """A few thousand fp32 codes against a thousand queries and more (the routing of an ivf search): the fp32 matrix
    cores fill a table of approximate distances, every query takes the codes within reach of its k-th table value and
    scores them with the streaming arithmetic.  Ids and distance bits equal the streaming scan's."""
    rng = np.random.default_rng(n + d + k)
    x, means = gaussian_mixture(rng, n, d, 20, 0.1)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.1, means=means)
    q[3] *= 1e4
    q[4] *= 1e-4
    q[5] = x[17]
    if metric != orc.COSINE:
        q[6] = 0.0
    st = Store(lib.KIND_FP32, metric, d)
    st.append(x.view(np.uint8).reshape(n, 4 * d))
    L = lib.load_library()
    lib.check(L.vsag_amd_set_scan_contraction(-1))
    try:
        plain = st.flat_scan(q, k)
    finally:
        lib.check(L.vsag_amd_set_scan_contraction(0))
    fast = st.flat_scan(q, k)
    tile = lib.C.c_int()
    L.vsag_amd_last_scan_info(lib.C.byref(tile), None, None)
    assert tile.value == 64, "the table route did not run"
    assert np.array_equal(plain[0], fast[0]) and np.array_equal(plain[1].view(np.uint32), fast[1].view(np.uint32))
    st.destroy()


def test_small_fp32_store_with_thousands_of_equal_rows(lib):
    """More codes at the k-th distance than a query's candidate pool takes (and a query with a NaN): those queries are
    redone by a full scan of their own."""
    n, d, nq, k = 8192, 32, 1200, 40
    rng = np.random.default_rng(9)
    x = (rng.random((n, d), dtype=np.float32) * 10 + 20).astype(np.float32)
    x[5::4] = x[5]  # 2047 copies of one row: the same distance, ids apart
    q = (x[5] + rng.random((nq, d), dtype=np.float32) * 0.1).astype(np.float32)
    q[100:] = (rng.random((nq - 100, d), dtype=np.float32) * 10 + 20).astype(np.float32)
    q[7, 3] = np.nan
    st = Store(lib.KIND_FP32, orc.L2, d)
    st.append(x.view(np.uint8).reshape(n, 4 * d))
    L = lib.load_library()
    lib.check(L.vsag_amd_set_scan_contraction(-1))
    try:
        plain = st.flat_scan(q, k)
    finally:
        lib.check(L.vsag_amd_set_scan_contraction(0))
    fast = st.flat_scan(q, k)
    ok = np.ones(nq, bool)
    ok[7] = False
    assert np.array_equal(plain[0][ok], fast[0][ok])
    assert np.array_equal(plain[1][ok].view(np.uint32), fast[1][ok].view(np.uint32))
    assert np.all(fast[0][:100][ok[:100]] % 4 == 1)
    st.destroy()
