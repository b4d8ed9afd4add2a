"""Large batches on flat fp32 / sq8 stores: the matrix-core contraction pre-selects, the streaming arithmetic
decides.  Its results must equal the streaming scan's bit for bit (and therefore the checker's within the usual
tolerance), including when candidates overflow and the streaming kernel takes over."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture()
def modes(lib):
    L = capi.load_library()

    def both(store, q, k, mode=1):
        capi.check(L.vsag_amd_set_scan_contraction(-1))
        plain = store.flat_scan(q, k)
        capi.check(L.vsag_amd_set_scan_contraction(mode))
        fast = store.flat_scan(q, k)
        tile = capi.C.c_int()
        L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
        capi.check(L.vsag_amd_set_scan_contraction(0))
        return plain, fast, tile.value
    yield both
    capi.check(L.vsag_amd_set_scan_contraction(0))


def same(a, b):
    return np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("n,d,nq,k", [(40000, 128, 300, 10), (20001, 100, 129, 100), (9000, 960, 64, 10),
                                      (5000, 33, 1000, 7)])
def test_sq8_contraction_equals_streaming(lib, modes, metric, n, d, nq, k):
    rng = np.random.default_rng(n + d + k)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    lb, diff = orc.sq_train(x, 8, metric)
    codes = orc.sq_encode(x, 8, lb, diff, metric)
    st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    st.append(codes[:n // 3])
    st.append(codes[n // 3:])  # the per-code terms follow appends
    # mode 1: the int8 matrix cores up to 128 dimensions (256 queries per pass); mode 2: always the fp32 ones
    for mode, tile_expected in ((1, 256 if d <= 128 else 128), (2, 128)):
        plain, fast, tile = modes(st, q, k, mode)
        assert tile == tile_expected, "the contraction path did not run"
        assert same(plain, fast)
    ri, rd = orc.flat_scan_topk(orc.SQ8, metric, d, codes, q[:16], k, lb=lb, diff=diff)
    assert_topk_close(fast[0][:16], fast[1][:16], ri, rd, label="sq8 contraction")
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(30000, 129, 600, 10), (20000, 200, 520, 100), (12000, 960, 512, 10),
                                      (9000, 1000, 130, 7)])
def test_sq8_beyond_128_dimensions_on_the_fp16_matrix_cores(lib, modes, metric, n, d, nq, k):
    """sq8 stores of more than 128 dimensions: the code bytes and the two fp16 parts of the scaled query on
    v_mfma_f32_32x32x16_f16 (prefilter_h16.hip), rescored exactly.  Awkward queries as for the int8 planes: zeros,
    tiny and huge magnitudes, one dominant dimension, copies of stored vectors, far outside the trained range, NaN."""
    rng = np.random.default_rng(n + d + k + metric)
    x, means = gaussian_mixture(rng, n, d, 20, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    if metric != orc.COSINE:  # no direction to normalise
        q[0] = 0.0
        q[1] = 1e-20
        q[6] = np.nan
        q[7, 3] = np.inf
    q[2] *= 1e6
    q[3] *= 1e-6
    q[4] = 0.0
    q[4, d // 2] = 1e4
    q[5] = 1e-30
    q[5, 1] = 3e37 if metric != orc.COSINE else 3.0
    q[8:40] = x[8:40]
    q[40:60] = -q[40:60]
    q[60:80] += 100.0
    lb, diff = orc.sq_train(x, 8, metric)
    codes = orc.sq_encode(x, 8, lb, diff, metric)
    st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    st.append(codes[:n // 2])
    st.append(codes[n // 2:])
    plain, fast, tile = modes(st, q, k, 1)
    assert tile == 128, "the contraction path did not run"
    assert same(plain, fast)
    plain, fp32, tile = modes(st, q, k, 2)  # the fp32 matrix cores: the same again
    assert tile == 128 and same(plain, fp32)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(30000, 160, 600, 10), (12000, 960, 512, 10), (9000, 1000, 130, 100)])
def test_sq4_beyond_128_dimensions_on_the_fp16_matrix_cores(lib, modes, metric, n, d, nq, k):
    """sq4 stores of more than 128 dimensions take the fp16 pass as well (the nibbles are exact in fp16), in mode 2 too:
    sq4 has no route on the fp32 matrix cores."""
    rng = np.random.default_rng(n + d + k + metric)
    x, means = gaussian_mixture(rng, n, d, 20, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    if metric != orc.COSINE:
        q[0] = 0.0
        q[1] = 1e-20
        q[6] = np.nan
    q[2] *= 1e6
    q[3] *= 1e-6
    q[4] = 0.0
    q[4, d // 2] = 1e4
    q[8:40] = x[8:40]
    q[60:80] += 100.0
    lb, diff = orc.sq_train(x, 4, metric)
    codes = orc.sq_encode(x, 4, lb, diff, metric)
    st = Store(capi.KIND_SQ4, metric, d, lb=lb, diff=diff)
    st.append(codes[:n // 2])
    st.append(codes[n // 2:])
    for mode in (1, 2):
        plain, fast, tile = modes(st, q, k, mode)
        assert tile == 128, "the contraction path did not run"
        assert same(plain, fast)
    qs, om = q[8:24], metric
    if metric == orc.COSINE:  # inner product of the unit query with the codes of the unit rows
        qs, om = (qs / np.linalg.norm(qs, axis=1, keepdims=True)).astype(np.float32), orc.IP
    ri, rd = orc.flat_scan_topk(orc.SQ4, om, d, codes, qs, k, lb=lb, diff=diff)
    assert_topk_close(fast[0][8:24], fast[1][8:24], ri, rd, label="sq4 beyond 128 dimensions")
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("d", [16, 100, 128])
def test_sq8_int8_planes_hold_for_awkward_queries(lib, modes, metric, d):
    """Queries the two int8 planes represent badly or trivially: one dominant dimension, tiny and huge magnitudes,
    all zeros, copies of stored vectors, far outside the trained range."""
    rng = np.random.default_rng(1000 + d + metric)
    n, nq, k = 30000, 320, 10
    x, means = gaussian_mixture(rng, n, d, 20, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 20, 0.05, means=means)
    if metric != orc.COSINE:  # no direction to normalise
        q[0] = 0.0
        q[1] = 1e-20
    q[2] *= 1e6
    q[3] *= 1e-6
    q[4] = 0.0
    q[4, d // 2] = 1e4
    q[5:40] = x[5:40]          # duplicates of stored vectors
    q[40:60] = -q[40:60]
    q[60:80] += 100.0          # far outside [lb, lb + diff]
    q[80, :] = np.where(np.arange(d) % 2 == 0, 1e-3, 1e3)
    lb, diff = orc.sq_train(x, 8, metric)
    codes = orc.sq_encode(x, 8, lb, diff, metric)
    st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    st.append(codes)
    plain, fast, tile = modes(st, q, k)
    assert tile == 256
    assert same(plain, fast)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(40000, 128, 300, 10), (20001, 100, 129, 100), (9000, 31, 640, 7),
                                      (30000, 16, 320, 10)])
def test_sq4_contraction_equals_streaming(lib, modes, metric, n, d, nq, k):
    """sq4 (a range per dimension, two 4-bit values per byte): the two int8 planes of a query against the nibbles as
    they are; awkward queries among the ordinary ones."""
    rng = np.random.default_rng(n + d + k + metric)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    if metric != orc.COSINE:
        q[0] = 0.0
        q[1] = 1e-20
    q[2] *= 1e6
    q[3] *= 1e-6
    q[5:40] = x[5:40]
    q[60:80] += 100.0
    lb, diff = orc.sq_train(x, 4, metric)
    codes = orc.sq_encode(x, 4, lb, diff, metric)
    st = Store(capi.KIND_SQ4, metric, d, lb=lb, diff=diff)
    st.append(codes[:n // 3])
    st.append(codes[n // 3:])  # the per-code terms follow appends
    plain, fast, tile = modes(st, q, k)
    assert tile == 256, "the contraction path did not run"
    assert same(plain, fast)
    # asking for the fp32 matrix cores finds no route for this kind and the int8 one serves
    plain, fast, tile = modes(st, q, k, 2)
    assert tile == 256 and same(plain, fast)
    om, oq = (orc.IP, (q[100:116] / np.linalg.norm(q[100:116], axis=1, keepdims=True)).astype(np.float32)) \
        if metric == orc.COSINE else (metric, q[100:116])
    ri, rd = orc.flat_scan_topk(orc.SQ4, om, d, codes, oq, k, lb=lb, diff=diff)
    assert_topk_close(fast[0][100:116], fast[1][100:116], ri, rd, atol=4e-6, label="sq4 contraction")
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(30000, 128, 200, 10), (7000, 65, 77, 32)])
def test_fp32_contraction_equals_streaming(lib, modes, metric, n, d, nq, k):
    rng = np.random.default_rng(n + d + k + metric)
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((nq, d), dtype=np.float32)
    x[5] = q[3]  # an exact duplicate of a query: distance 0 must come out as 0
    st = Store(capi.KIND_FP32, metric, d)
    st.append(x.view(np.uint8).reshape(n, 4 * d))
    plain, fast, tile = modes(st, q, k)
    assert tile == 128
    assert same(plain, fast)
    if metric == orc.L2:
        assert fast[0][3, 0] == 5 and fast[1][3, 0] == 0.0
    st.destroy()


@pytest.mark.parametrize("kind", ["fp32", "sq8"])
def test_many_short_tiles_per_workgroup(lib, modes, kind):
    """100000 x 128 against 1000 queries: every workgroup walks many code tiles with a short contraction each, so
    the epilogue of one tile runs next to the start of the following one."""
    rng = np.random.default_rng(77)
    n, d, nq, k = 100000, 128, 1000, 10
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    if kind == "fp32":
        st = Store(capi.KIND_FP32, orc.L2, d)
        st.append(x.view(np.uint8).reshape(n, 4 * d))
    else:
        lb, diff = orc.sq_train(x, 8, orc.L2)
        st = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
        st.append(orc.sq_encode(x, 8, lb, diff, orc.L2))
    for _ in range(3):
        plain, fast, tile = modes(st, q, k)
        assert tile == (128 if kind == "fp32" else 256)
        assert same(plain, fast)
    st.destroy()


def test_contraction_overflow_falls_back_to_streaming(lib, modes):
    """Thousands of equal distances per query: the candidate buffers overflow, the streaming kernel serves the query."""
    rng = np.random.default_rng(8)
    n, d, nq, k = 30000, 32, 150, 10
    base = rng.integers(0, 256, (40, d), dtype=np.uint8)
    codes = base[rng.integers(0, 40, n)]  # 40 distinct codes, 750 copies each
    lb, diff = np.zeros(d, np.float32), np.ones(d, np.float32)
    q = rng.random((nq, d), dtype=np.float32)
    st = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    st.append(codes)
    for mode, tile_expected in ((1, 256), (2, 128)):
        plain, fast, tile = modes(st, q, k, mode)
        assert tile == tile_expected
        assert same(plain, fast)
    ri, rd = orc.flat_scan_topk(orc.SQ8, orc.L2, d, codes, q[:8], k, lb=lb, diff=diff)
    # which of the equal distances the checker keeps is its heap's business; the distances must agree
    np.testing.assert_allclose(fast[1][:8], rd, rtol=1e-5)
    assert np.all(np.diff(fast[0], axis=1)[np.diff(fast[1], axis=1) == 0] > 0), "ties are ordered by id"
    st.destroy()


def _rabitq_store(rng, n, d, metric, centered=True):
    x = rng.standard_normal((n, d)).astype(np.float32)
    if centered:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    else:
        x = x * 0.1 + 1.0  # far from the origin: large raw norms, small residuals
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    st.append(orc.rabitq_encode(x, rot, cen, metric))
    return x, st


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("n,d,nq,k,centered", [(30000, 128, 300, 10, True), (20000, 768, 260, 200, True),
                                               (9000, 100, 129, 50, False), (70000, 256, 700, 100, True),
                                               (12000, 1024, 150, 20, True)])
def test_rabitq_contraction_equals_streaming(lib, modes, metric, n, d, nq, k, centered):
    """1-bit codes against 4-bit queries on the int8 matrix cores: the estimator is affine in the integer inner
    product, so the pre-selection is a threshold on it; the rescored result must equal the streaming scan's bits."""
    rng = np.random.default_rng(n + d + k + metric)
    x, st = _rabitq_store(rng, n, d, metric, centered)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    if centered:
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    else:
        q = q * 0.1 + 1.0
    q[3] = x[17]                 # a stored vector
    q[4] = 0.0                   # no direction at all
    q[5] = 1.0                   # constant coordinates before the rotation
    plain, fast, tile = modes(st, q, k)
    assert tile == 128, "the contraction path did not run"
    assert same(plain, fast)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
def test_rabitq_store_of_many_appends_and_codes_outside_the_pass(lib, modes, metric):
    """The store keeps its code bits and per-code constants once more for the matrix cores, renewed by every append
    (also of the tile an earlier append left part full).  Codes the pre-selection's derivation does not cover -- a zero
    norm, a non-positive error factor, a sum field that is not the number of set bits -- must still come out as the
    streaming scan has them."""
    n, d, nq, k = 21000, 200, 200, 30
    rng = np.random.default_rng(77 + metric)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    g = rng.standard_normal((d, d))
    rot, r = np.linalg.qr(g)
    rot = (rot * np.sign(np.diag(r))).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    x[5] = cen @ rot                    # the centroid itself (rotated back): a zero norm after centring
    codes = orc.rabitq_encode(x, rot, cen, metric)
    tail = codes[:, -(12 if metric == orc.L2 else 16):].view(np.float32)  # norm, error factor, sum[, raw norm]
    tail[70, 1] = -0.5                  # a negative error factor
    tail[131, 2] += 3.0                 # a sum field that is not the set bits
    tail[4000, 0] = 0.0                 # a zero norm
    tail[20999, 2] = 0.0
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    at = 0
    for step in (1, 63, 64, 65, 1000, 37, 12000, 3, n):   # ragged: tiles left part full and filled later
        end = min(n, at + step)
        if end > at:
            st.append(codes[at:end])
        at = end
    assert at == n
    q = rng.standard_normal((nq, d)).astype(np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    plain, fast, tile = modes(st, q, k)
    assert tile == 128, "the contraction path did not run"
    assert same(plain, fast)
    whole = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    whole.append(codes)
    assert same(plain, whole.flat_scan(q, k))
    whole.destroy()
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(40000, 128, 300, 10), (20001, 100, 129, 100), (5000, 33, 1000, 7),
                                      (70000, 64, 600, 1)])
def test_sq8_uniform_contraction_equals_streaming(lib, modes, metric, n, d, nq, k):
    """sq8_uniform: code and query are both rows of bytes, the product is an integer the int8 matrix cores deliver
    exactly; distances are integers scaled once, so ties abound and must come out in id order on both routes."""
    rng = np.random.default_rng(n + d + k + 3 * metric)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    q[3] = x[17]          # a stored vector
    q[4] = 0.0            # clamps to the lower bound everywhere
    q[5] = 10.0           # clamps to the upper bound everywhere
    lb, diff = orc.sq_train_uniform(x, 8, metric, mode=1)
    codes = orc.squ_encode(x, 8, lb, diff, metric)
    st = Store(capi.KIND_SQ8_UNIFORM, metric, d, bounds=[lb, diff])
    st.append(codes[:n // 3])
    st.append(codes[n // 3:])
    plain, fast, tile = modes(st, q, k)
    assert tile == 256, "the int8 route did not run"
    assert same(plain, fast)
    plain, fast, tile = modes(st, q, k, mode=2)  # no fp32 route for this kind: still the int8 matrix cores
    assert tile == 256 and same(plain, fast)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d,nq,k", [(40000, 128, 300, 10), (20001, 100, 129, 100), (5000, 33, 1000, 7),
                                      (70000, 64, 600, 1)])
def test_sq4_uniform_contraction_equals_streaming(lib, modes, metric, n, d, nq, k):
    """sq4_uniform: two 4-bit values per byte, split into low- and high-nibble granules when staged."""
    rng = np.random.default_rng(n + d + k + 5 * metric)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    q[3] = x[17]
    q[4] = 0.0
    q[5] = 10.0
    lb, diff = orc.sq_train_uniform(x, 4, metric, mode=3)
    codes = orc.squ_encode(x, 4, lb, diff, metric)
    st = Store(capi.KIND_SQ4_UNIFORM, metric, d, bounds=[lb, diff])
    st.append(codes[:n // 3])
    st.append(codes[n // 3:])
    plain, fast, tile = modes(st, q, k)
    assert tile == 256, "the int8 route did not run"
    assert same(plain, fast)
    st.destroy()


def test_settings_of_one_store_leave_the_others_alone(lib):
    """vsag_amd_store_set_scan_contraction / _set_scan_tuning: a store's own settings go before the process-wide ones
    and do not touch searches on another store."""
    L = capi.load_library()
    n, d, nq, k = 70000, 64, 600, 10
    rng = np.random.default_rng(21)
    x, means = gaussian_mixture(rng, n, d, 30, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 30, 0.05, means=means)
    lb, diff = orc.sq_train(x, 8, orc.L2)
    codes = orc.sq_encode(x, 8, lb, diff, orc.L2)
    a = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    b = Store(capi.KIND_SQ8, orc.L2, d, lb=lb, diff=diff)
    a.append(codes)
    b.append(codes)
    tile = capi.C.c_int()

    def last_tile():
        L.vsag_amd_last_scan_info(capi.C.byref(tile), None, None)
        return tile.value
    capi.check(L.vsag_amd_store_set_scan_contraction(a.handle, -1))
    ws_a, ws_b = (int(L.vsag_amd_flat_scan_workspace_bytes(s.handle, nq, k)) for s in (a, b))
    assert ws_a < ws_b, "the streaming scan needs no candidate buffers"
    ra = a.flat_scan(q, k)
    assert last_tile() == 4, "store a was told to stream"
    rb = b.flat_scan(q, k)
    assert last_tile() == 256, "store b follows the process-wide default"
    assert same(ra, rb)
    capi.check(L.vsag_amd_store_set_scan_tuning(a.handle, 2, -1))
    ra2 = a.flat_scan(q, k)
    assert last_tile() == 2
    assert same(ra, ra2)
    b.flat_scan(q[:8], k)
    assert last_tile() == 4, "store b keeps the default tile"
    # back to the process-wide settings; a bad mode is refused
    capi.check(L.vsag_amd_store_set_scan_contraction(a.handle, -2))
    capi.check(L.vsag_amd_store_set_scan_tuning(a.handle, -1, -1))
    a.flat_scan(q, k)
    assert last_tile() == 256
    assert L.vsag_amd_store_set_scan_contraction(a.handle, 3) == capi.INVALID_ARGUMENT
    assert L.vsag_amd_store_set_scan_tuning(a.handle, 3, 0) == capi.INVALID_ARGUMENT
    a.destroy()
    b.destroy()
