"""The flat scan that allocates nothing (vsag_amd_flat_scan_topk_noalloc): same ids and distance bits as
vsag_amd_flat_scan_topk_ex with a caller's workspace, on two calls in a row that share the library's scratch
array (the second smaller), under a filter and a radius, a clear refusal beyond the array's size, and -- for every
call -- no device memory taken from hipMalloc or from the stream-ordered allocator, also on the stores whose
queries are encoded with temporaries (rabitq: rotated rows; uniform kinds under cosine: a norm per query)."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def memory_marks(lib, reset):
    """(free device bytes, high-water mark of the stream-ordered allocator's pool since its last reset)."""
    free, high = C.c_uint64(), C.c_uint64()
    capi.check(lib.vsag_amd_memory_info(C.byref(free), None, C.byref(high), 1 if reset else 0))
    return free.value, high.value


def noalloc_scan(lib, store, queries, k, opt=None, count_memory=True):
    q = np.ascontiguousarray(queries, np.float32)
    nq = q.shape[0]
    qb = dev(q)
    ids, ds = capi.DeviceBuffer(nq * k * 4), capi.DeviceBuffer(nq * k * 4)
    # poison the outputs: whatever the call leaves untouched would show
    capi.check(lib.vsag_amd_memset(ids.ptr, 0x5A, nq * k * 4, None))
    capi.check(lib.vsag_amd_memset(ds.ptr, 0x5A, nq * k * 4, None))
    capi.synchronize()
    # The call must take no device memory: neither hipMalloc (free bytes unchanged while it is in flight and after)
    # nor the stream-ordered allocator (its pool's high-water mark, reset to zero here, stays zero).
    free0, _ = memory_marks(lib, True)
    capi.check(lib.vsag_amd_flat_scan_topk_noalloc(store.handle, qb.ptr, nq, k, C.byref(opt) if opt is not None else None,
                                                   ids.ptr, ds.ptr, None))
    free1, high1 = memory_marks(lib, False)
    capi.synchronize()
    free2, high2 = memory_marks(lib, False)
    assert (high1, high2) == (0, 0), "the stream-ordered allocator was used: %d / %d bytes" % (high1, high2)
    if count_memory:
        assert free1 >= free0 and free2 >= free0, "device memory was taken: %d -> %d -> %d" % (free0, free1, free2)
    out = ids.to_numpy(np.uint32, (nq, k)), ds.to_numpy(np.float32, (nq, k))
    for b in (qb, ids, ds):
        b.free()
    return out


def same(a, b):
    return np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


def test_noalloc_flat_scan_equals_workspace_scan(lib):
    l = capi.load_library()
    assert l.vsag_amd_flat_scan_noalloc_max_bytes() == 32 << 20
    rng = np.random.default_rng(2024)
    n, d, k = 40000, 128, 10
    x, means = gaussian_mixture(rng, n, d, 50, 0.05)
    lb, diff = orc.sq_train(x, 8)
    codes = orc.sq_encode(x, 8, lb, diff)
    store = Store(capi.KIND_SQ8, capi.METRIC_L2, d, lb=lb, diff=diff)
    store.append(codes)
    q1, _ = gaussian_mixture(rng, 96, d, 50, 0.05, means=means)
    q2, _ = gaussian_mixture(rng, 5, d, 50, 0.05, means=means)
    # The first scan of a process lets the HIP runtime take memory of its own (2 MiB here: what it sets up on first use
    # of kernels and pools, whichever entry point launches them): one call before the free bytes are counted, as a
    # caller that cannot allocate makes one before it starts capturing or serving.  (The stream-ordered allocator is watched even here.)
    a0 = noalloc_scan(l, store, q1, k, count_memory=False)
    # two calls in a row on the shared array, the second with a smaller input (and another k)
    a1 = noalloc_scan(l, store, q1, k)
    assert same(a0, a1)
    a2 = noalloc_scan(l, store, q2, 7)
    assert same(a1, store.flat_scan(q1, k))
    assert same(a2, store.flat_scan(q2, 7))
    oi, od = orc.flat_scan_topk(orc.SQ8, orc.L2, d, codes, q2, 7, lb=lb, diff=diff)
    assert_topk_close(a2[0], a2[1], oi, od, label="noalloc sq8")
    # one query per call, the serving pattern, again after the larger calls
    for i in range(4):
        assert same(noalloc_scan(l, store, q1[i:i + 1], k), (a1[0][i:i + 1], a1[1][i:i + 1]))
    # options travel as in the _ex entry point
    deny = rng.random(n) < 0.5
    radius = float(np.median(a1[1][:, -1]))
    opt, keep = store._options(deny, radius)
    b1 = noalloc_scan(l, store, q1[:16], k, opt)
    assert same(b1, store.flat_scan(q1[:16], k, deny=deny, radius=radius))
    for b in keep:
        b.free()
    # beyond the array: refused, and says why
    big = np.zeros((4096, d), np.float32)
    assert l.vsag_amd_flat_scan_workspace_bytes(store.handle, 4096, 1000) > (32 << 20)
    qb = dev(big)
    ids, ds = capi.DeviceBuffer(4096 * 1000 * 4), capi.DeviceBuffer(4096 * 1000 * 4)
    rc = l.vsag_amd_flat_scan_topk_noalloc(store.handle, qb.ptr, 4096, 1000, None, ids.ptr, ds.ptr, None)
    assert rc == capi.INVALID_ARGUMENT and b"scratch" in l.vsag_amd_last_error()
    for b in (qb, ids, ds):
        b.free()
    # and the array still serves the next call
    assert same(noalloc_scan(l, store, q2, 7), a2)
    store.destroy()


def _rotation(rng, d):
    g = rng.standard_normal((d, d))
    q, r = np.linalg.qr(g)
    return (q * np.sign(np.diag(r))).astype(np.float32)


@pytest.mark.parametrize("qbits", [4, 32])
@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
def test_noalloc_rabitq_store(lib, metric, qbits):
    """RaBitQ queries are rotated before they are quantised; the rotated rows live in the scratch array too."""
    l = capi.load_library()
    rng = np.random.default_rng(100 + qbits + metric)
    n, d, k = 9000, 200, 10
    x = rng.standard_normal((n, d)).astype(np.float32)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    codes = orc.rabitq_encode(x, rot, cen, metric, qbits)
    store = Store(capi.KIND_RABITQ, metric, d, rot=rot, centroid=cen, qbits=qbits)
    store.append(codes)
    q1 = rng.standard_normal((40, d)).astype(np.float32)
    q2 = rng.standard_normal((3, d)).astype(np.float32)
    noalloc_scan(l, store, q1, k, count_memory=False)  # first launches of these kernels in the process: see above
    a1 = noalloc_scan(l, store, q1, k)
    a2 = noalloc_scan(l, store, q2, 5)
    assert same(a1, store.flat_scan(q1, k))
    assert same(a2, store.flat_scan(q2, 5))
    oi, od = orc.flat_scan_topk(orc.RABITQ, metric, d, codes, orc.rabitq_process_query(q2, rot, cen, metric, qbits), 5,
                                qbits=qbits)
    assert_topk_close(a2[0], a2[1], oi, od, rtol=1e-4, atol=2e-5, tie_rtol=2e-4, label="noalloc rabitq")
    store.destroy()


@pytest.mark.parametrize("bits", [4, 8])
def test_noalloc_uniform_store_under_cosine(lib, bits):
    """The uniform kinds encode the query with the base encoder, which wants a norm per row under cosine."""
    l = capi.load_library()
    rng = np.random.default_rng(7 + bits)
    n, d, k = 5000, 96, 10
    x = rng.random((n, d), dtype=np.float32)
    lb, diff = orc.sq_train_uniform(x, bits, orc.COSINE, mode=3 if bits == 4 else 1)
    codes = orc.squ_encode(x, bits, lb, diff, orc.COSINE)
    kind = capi.KIND_SQ4_UNIFORM if bits == 4 else capi.KIND_SQ8_UNIFORM
    store = Store(kind, orc.COSINE, d, bounds=(lb, diff))
    store.append(codes)
    q1 = rng.random((33, d), dtype=np.float32)
    q2 = rng.random((2, d), dtype=np.float32)
    noalloc_scan(l, store, q1, k, count_memory=False)  # first launches of these kernels in the process: see above
    a1 = noalloc_scan(l, store, q1, k)
    a2 = noalloc_scan(l, store, q2, 4)
    assert same(a1, store.flat_scan(q1, k))
    assert same(a2, store.flat_scan(q2, 4))
    okind = orc.SQ4U if bits == 4 else orc.SQ8U
    oi, od = orc.flat_scan_topk(okind, orc.COSINE, d, codes, orc.squ_encode(q2, bits, lb, diff, orc.COSINE), 4,
                                lb=lb, diff=diff)
    assert_topk_close(a2[0], a2[1], oi, od, label="noalloc uniform cosine")
    store.destroy()
