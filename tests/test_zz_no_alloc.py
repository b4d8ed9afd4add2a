"""The flat scan that allocates nothing (vsag_amd_flat_scan_topk_noalloc): same ids and distance bits as
vsag_amd_flat_scan_topk_ex with a caller's workspace, on two calls in a row that share the library's scratch
array (the second smaller), under a filter and a radius, and a clear refusal beyond the array's size."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def noalloc_scan(lib, store, queries, k, opt=None):
    q = np.ascontiguousarray(queries, np.float32)
    nq = q.shape[0]
    qb = dev(q)
    ids, ds = capi.DeviceBuffer(nq * k * 4), capi.DeviceBuffer(nq * k * 4)
    # poison the outputs: whatever the call leaves untouched would show
    capi.check(lib.vsag_amd_memset(ids.ptr, 0x5A, nq * k * 4, None))
    capi.check(lib.vsag_amd_memset(ds.ptr, 0x5A, nq * k * 4, None))
    capi.check(lib.vsag_amd_flat_scan_topk_noalloc(store.handle, qb.ptr, nq, k, C.byref(opt) if opt is not None else None,
                                                   ids.ptr, ds.ptr, None))
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
    # two calls in a row on the shared array, the second with a smaller input (and another k)
    a1 = noalloc_scan(l, store, q1, k)
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
