"""Parity of quantizer training / encoding on the device against the CPU checker: codes are compared bit
for bit, trained bounds exactly (they are order statistics of the same deterministic sample)."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from gpu_helpers import dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _train(lib, x, bits, metric, mode, trunc_rate=0.05, max_sample=0):
    L = lib.load_library()
    n, d = x.shape
    xb = dev(x)
    lb, diff = capi.DeviceBuffer(d * 4), capi.DeviceBuffer(d * 4)
    wsb = L.vsag_amd_sq_train_workspace_bytes(n, d, max_sample)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_sq_train(xb.ptr, n, d, bits, metric, mode, trunc_rate, max_sample, lb.ptr, diff.ptr,
                                   ws.ptr, wsb, None))
    return lb.to_numpy(np.float32, (d,)), diff.to_numpy(np.float32, (d,))


def _train_uniform(lib, x, bits, metric, mode, trunc_rate=0.05):
    L = lib.load_library()
    n, d = x.shape
    xb = dev(x)
    out = capi.DeviceBuffer(8)
    wsb = L.vsag_amd_sq_train_workspace_bytes(n, d, 0)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_sq_train_uniform(xb.ptr, n, d, bits, metric, mode, trunc_rate, 0, out.ptr, ws.ptr, wsb,
                                           None))
    r = out.to_numpy(np.float32, (2,))
    return r[0], r[1]


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("metric", [orc.L2, orc.COSINE])
@pytest.mark.parametrize("n,d,max_sample", [(5000, 33, 0), (120000, 16, 0), (3000, 8, 1000), (1, 5, 0), (2, 3, 0)])
def test_sq_train_matches_oracle(lib, bits, metric, n, d, max_sample):
    rng = np.random.default_rng(n + d + bits)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x[:, 0] = np.round(x[:, 0] * 4) / 4  # duplicates around the order statistic
    for mode in (capi.SQ_TRAIN_TRUNC_BOUND, capi.SQ_TRAIN_CLASSIC):
        lb, diff = _train(lib, x, bits, metric, mode, max_sample=max_sample)
        rlb, rdiff = orc.sq_train(x, bits, metric, mode=mode, max_sample=max_sample)
        assert np.array_equal(lb, rlb), (mode, lb[:4], rlb[:4])
        assert np.array_equal(diff, rdiff), (mode, diff[:4], rdiff[:4])


@pytest.mark.parametrize("bits,mode", [(4, 3), (8, 1), (4, 1), (8, 3)])
def test_sq_train_uniform_matches_oracle(lib, bits, mode):
    rng = np.random.default_rng(bits + mode)
    x = rng.random((20000, 24), dtype=np.float32)
    lb, diff = _train_uniform(lib, x, bits, orc.L2, mode)
    rlb, rdiff = orc.sq_train_uniform(x, bits, orc.L2, mode=mode)
    assert lb == rlb and diff == rdiff


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d", [(4000, 128), (300, 7), (65, 33)])
def test_sq_encode_bit_exact(lib, bits, metric, n, d):
    L = lib.load_library()
    rng = np.random.default_rng(n + d)
    x = (rng.standard_normal((n, d)) * 0.3 + 0.5).astype(np.float32)
    x[0, 0] = np.nan  # NaN -> code 0 (scalar_quantizer_test.cpp:101-135)
    lb, diff = orc.sq_train(x[1:], bits, metric)
    diff[d - 1] = 0.0  # zero range -> delta = 1
    codes_ref = orc.sq_encode(x, bits, lb, diff, metric)
    cs = codes_ref.shape[1]
    xb, lbb, dfb = dev(x), dev(lb), dev(diff)
    out = capi.DeviceBuffer(n * cs)
    capi.check(L.vsag_amd_sq_encode(xb.ptr, n, d, bits, metric, lbb.ptr, dfb.ptr, out.ptr, None))
    codes = out.to_numpy(np.uint8, (n, cs))
    if metric == orc.COSINE:
        ok = ~np.isnan(x).any(1)  # a NaN row has a NaN norm on both sides; its codes are all-zero anyway
        assert np.array_equal(codes[ok], codes_ref[ok])
    else:
        assert np.array_equal(codes, codes_ref)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("n,d", [(3000, 128), (100, 15), (64, 6)])
def test_squ_encode_bit_exact(lib, bits, metric, n, d):
    L = lib.load_library()
    rng = np.random.default_rng(n + d + bits)
    x = rng.random((n, d), dtype=np.float32)
    lb, diff = orc.sq_train_uniform(x, bits, metric, mode=3 if bits == 4 else 1)
    ref = orc.squ_encode(x, bits, lb, diff, metric)
    cs = ref.shape[1]
    kind = capi.KIND_SQ4_UNIFORM if bits == 4 else capi.KIND_SQ8_UNIFORM
    assert cs == L.vsag_amd_code_size(kind, metric, d, 0)
    xb, bb = dev(x), dev(np.array([lb, diff], np.float32))
    out = capi.DeviceBuffer(n * cs)
    capi.check(L.vsag_amd_squ_encode(xb.ptr, n, d, bits, metric, bb.ptr, out.ptr, None))
    codes = out.to_numpy(np.uint8, (n, cs))
    assert np.array_equal(codes, ref)


def _rotation(rng, d):
    q, r = np.linalg.qr(rng.standard_normal((d, d)))
    q = q * np.sign(np.diag(r))
    return q.astype(np.float32)


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("n,d", [(500, 128), (200, 15), (64, 768)])
def test_rabitq_train_encode_query_bit_exact(lib, metric, n, d):
    """The device keeps every running sum in element order and does not fuse multiply-adds, so the codes,
    the trailing floats and the processed queries equal the checker's bit for bit."""
    L = lib.load_library()
    rng = np.random.default_rng(n + d)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    q = rng.standard_normal((9, d)).astype(np.float32)
    rot = _rotation(rng, d)
    cen_ref = orc.rabitq_train(x, rot)
    xb, rb = dev(x), dev(rot)
    cen = capi.DeviceBuffer(d * 4)
    capi.check(L.vsag_amd_rabitq_train(xb.ptr, n, d, rb.ptr, cen.ptr, None))
    cen_gpu = cen.to_numpy(np.float32, (d,))
    assert np.array_equal(cen_gpu, cen_ref)

    ref = orc.rabitq_encode(x, rot, cen_ref, metric)
    cs = ref.shape[1]
    assert cs == L.vsag_amd_code_size(capi.KIND_RABITQ, metric, d, 4)
    out = capi.DeviceBuffer(n * cs)
    capi.check(L.vsag_amd_rabitq_encode(xb.ptr, n, d, rb.ptr, cen.ptr, metric, 4, out.ptr, None))
    codes = out.to_numpy(np.uint8, (n, cs))
    assert np.array_equal(codes, ref)

    qref = orc.rabitq_process_query(q, rot, cen_ref, metric)
    qs = qref.shape[1]
    assert qs == L.vsag_amd_rabitq_query_code_size(d, metric, 4)
    qb = dev(q)
    qout = capi.DeviceBuffer(q.shape[0] * qs)
    capi.check(L.vsag_amd_rabitq_process_query(qb.ptr, q.shape[0], d, rb.ptr, cen.ptr, metric, 4, qout.ptr, None))
    qcodes = qout.to_numpy(np.uint8, (q.shape[0], qs))
    assert np.array_equal(qcodes, qref)


@pytest.mark.parametrize("metric,mname", [(orc.L2, "l2"), (orc.IP, "ip")])
@pytest.mark.parametrize("n,d,nq,k", [(6000, 128, 11, 10), (900, 768, 5, 200), (300, 15, 3, 7)])
def test_rabitq_flat_scan(lib, metric, mname, n, d, nq, k):
    from gpu_helpers import Store, assert_topk_close
    rng = np.random.default_rng(n + d + 5)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    codes = orc.rabitq_encode(x, rot, cen, metric)
    qcodes = orc.rabitq_process_query(q, rot, cen, metric)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen)
    st.append(codes)
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(orc.RABITQ, metric, d, codes, qcodes, k)
    # Integer inner products are exact and the float estimator keeps the checker's operation order.
    assert_topk_close(ids, ds, rids, rds, rtol=1e-5, atol=1e-6, label="rabitq " + mname)
    st.destroy()


@pytest.mark.parametrize("metric,mname", [(orc.L2, "l2"), (orc.IP, "ip"), (orc.COSINE, "cosine")])
@pytest.mark.parametrize("n,d,nq,k", [(6000, 128, 11, 10), (900, 768, 5, 100), (300, 15, 3, 7), (2000, 200, 1, 10)])
def test_rabitq_flat_scan_fp32_queries(lib, metric, mname, n, d, nq, k):
    """rabitq_bits_per_dim_query = 32: the query stays fp32 (RaBitQFloatBinaryIP, src/simd/generic.cpp:447-471)."""
    from gpu_helpers import Store, assert_topk_close
    rng = np.random.default_rng(n + d + 32)
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    codes = orc.rabitq_encode(x, rot, cen, metric, 32)
    qcodes = orc.rabitq_process_query(q, rot, cen, metric, 32)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen, qbits=32)
    assert st.code_size() == codes.shape[1]
    st.append(codes)
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(orc.RABITQ, metric, d, codes, qcodes, k, qbits=32)
    # the sum over set bits is taken in another order than the checker's running sum
    assert_topk_close(ids, ds, rids, rds, rtol=1e-4, atol=2e-5, tie_rtol=2e-4, label="rabitq fp32 query " + mname)
    st.destroy()


# ------------------------------------------------------------------ multi-bit RaBitQ base codes
@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("bits,n,d", [(2, 700, 128), (4, 500, 128), (8, 300, 128), (3, 200, 15), (4, 150, 200),
                                      (5, 120, 768), (8, 130, 64)])
def test_rabitq_multibit_encode_and_query(lib, metric, fast, bits, n, d):
    """rabitq_bits_per_dim_base 2..8 (rabitq_quantizer.cpp:774-809): FastEncodeRaBitQ / EncodeExtendRaBitQ, bit planes,
    norm of the code, norm, error -- byte for byte the checker's codes; the processed query carries its sum."""
    rng = np.random.default_rng(bits * 1000 + d + int(fast))
    L = lib.load_library()
    x = rng.standard_normal((n, d)).astype(np.float32)
    x[3] = 0.0  # a zero row: the centred vector still is not zero, a plain case
    q = rng.standard_normal((7, d)).astype(np.float32)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    word = orc.rabitq_bits(32, bits)
    ref = orc.rabitq_encode_multibit(x, rot, cen, metric, bits, fast=fast, rounds=6)
    cs = ref.shape[1]
    assert cs == L.vsag_amd_code_size(capi.KIND_RABITQ, metric, d, word)
    xb, rb, cb = dev(x), dev(rot), dev(cen)
    out = capi.DeviceBuffer(n * cs)
    capi.check(L.vsag_amd_rabitq_encode_multibit(xb.ptr, n, d, rb.ptr, cb.ptr, metric, word, 1 if fast else 0, 6,
                                                 out.ptr, None))
    codes = out.to_numpy(np.uint8, (n, cs))
    bad = np.flatnonzero((codes != ref).any(axis=1))
    assert bad.size == 0, (bad[:5], codes[bad[0]], ref[bad[0]])

    qref = orc.rabitq_process_query(q, rot, cen, metric, word)
    qs = qref.shape[1]
    assert qs == L.vsag_amd_rabitq_query_code_size(d, metric, word)
    qb = dev(q)
    qout = capi.DeviceBuffer(q.shape[0] * qs)
    capi.check(L.vsag_amd_rabitq_process_query(qb.ptr, q.shape[0], d, rb.ptr, cb.ptr, metric, word, qout.ptr, None))
    assert np.array_equal(qout.to_numpy(np.uint8, (q.shape[0], qs)), qref)


def test_rabitq_multibit_rounds_and_arguments(lib):
    lib = lib.load_library()
    rng = np.random.default_rng(77)
    n, d, bits = 300, 96, 4
    x = rng.standard_normal((n, d)).astype(np.float32)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    word = orc.rabitq_bits(32, bits)
    xb, rb, cb = dev(x), dev(rot), dev(cen)
    cs = orc.rabitq_code_size(d, orc.L2, word)
    out = capi.DeviceBuffer(n * cs)
    for rounds in (1, 2, 32):
        capi.check(lib.vsag_amd_rabitq_encode_multibit(xb.ptr, n, d, rb.ptr, cb.ptr, orc.L2, word, 1, rounds, out.ptr, None))
        assert np.array_equal(out.to_numpy(np.uint8, (n, cs)),
                              orc.rabitq_encode_multibit(x, rot, cen, orc.L2, bits, fast=True, rounds=rounds))
    for bad_word, fast, rounds in ((orc.rabitq_bits(4, 4), 1, 6), (32 | (9 << 8), 1, 6), (32 | (1 << 8), 1, 6),
                                   (word, 1, 0), (word, 1, 33)):
        assert lib.vsag_amd_rabitq_encode_multibit(xb.ptr, n, d, rb.ptr, cb.ptr, orc.L2, bad_word, fast, rounds, out.ptr,
                                                   None) == capi.INVALID_ARGUMENT


@pytest.mark.parametrize("metric,mname", [(orc.L2, "l2"), (orc.IP, "ip"), (orc.COSINE, "cosine")])
@pytest.mark.parametrize("bits,n,d,nq,k", [(2, 6000, 128, 11, 10), (4, 3000, 128, 70, 10), (8, 2000, 128, 5, 100),
                                           (4, 900, 768, 5, 50), (3, 300, 15, 3, 7), (5, 1500, 200, 1, 10),
                                           (8, 500, 960, 9, 20)])
def test_rabitq_multibit_flat_scan(lib, metric, mname, bits, n, d, nq, k):
    """Multi-bit codes against fp32 queries (rabitq_quantizer.cpp:1799-1808 over RaBitQFloatSplitCodeIP,
    generic.cpp:743-771).  Floating point: the device adds the query values plane by plane, the checker dimension by
    dimension, so distances agree to 1e-4 relative (2e-5 absolute) and ids up to ties of that width."""
    from gpu_helpers import Store, assert_topk_close
    lib = lib.load_library()
    rng = np.random.default_rng(n + d + bits)
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    word = orc.rabitq_bits(32, bits)
    codes = orc.rabitq_encode_multibit(x, rot, cen, metric, bits)
    qcodes = orc.rabitq_process_query(q, rot, cen, metric, word)
    st = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen, qbits=word)
    assert st.code_size() == codes.shape[1]
    st.append(codes)
    # the codes come back out of the tiles as they went in
    back = capi.DeviceBuffer(codes.size)
    capi.check(lib.vsag_amd_store_export_codes(st.handle, 0, n, back.ptr, None))
    assert np.array_equal(back.to_numpy(np.uint8, codes.shape), codes)
    ids, ds = st.flat_scan(q, k)
    rids, rds = orc.flat_scan_topk(orc.RABITQ, metric, d, codes, qcodes, k, qbits=word)
    assert_topk_close(ids, ds, rids, rds, rtol=1e-4, atol=2e-5, tie_rtol=2e-4, label="rabitq %d-bit %s" % (bits, mname))
    st.destroy()
