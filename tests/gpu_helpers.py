"""Helpers for the GPU parity tests: numpy <-> device through the C ABI, and top-k comparison."""
import ctypes as C

import numpy as np

from vsag_amd import capi


def dev(arr):
    return capi.DeviceBuffer.from_numpy(np.ascontiguousarray(arr))


class Store:
    """A vsag_amd store handle plus the device buffers that must outlive it."""

    def __init__(self, kind, metric, dim, lb=None, diff=None, bounds=None, rot=None, centroid=None, qbits=4,
                 pq_dim=0, codebooks=None):
        self.lib = capi.load_library()
        self.kind, self.metric, self.dim, self.qbits, self.pq_dim = kind, metric, dim, qbits, pq_dim
        self._keep = []
        p = capi.StoreParams()
        p.kind, p.metric, p.dim, p.rabitq_query_bits = kind, metric, dim, qbits
        if kind in (capi.KIND_SQ8, capi.KIND_SQ4):
            a, b = dev(np.asarray(lb, np.float32)), dev(np.asarray(diff, np.float32))
            self._keep += [a, b]
            p.lower_bound_dev, p.diff_dev = a.ptr, b.ptr
        elif kind in (capi.KIND_SQ4_UNIFORM, capi.KIND_SQ8_UNIFORM):
            a = dev(np.asarray(bounds, np.float32))
            self._keep.append(a)
            p.lower_bound_dev = a.ptr
        elif kind == capi.KIND_RABITQ:
            a, b = dev(np.asarray(rot, np.float32)), dev(np.asarray(centroid, np.float32))
            self._keep += [a, b]
            p.rotation_dev, p.centroid_dev = a.ptr, b.ptr
        elif kind == capi.KIND_PQFS:
            a = dev(np.asarray(codebooks, np.float32))
            self._keep.append(a)
            p.pq_dim, p.codebooks_dev = pq_dim, a.ptr
        h = C.c_void_p()
        capi.check(self.lib.vsag_amd_store_create(C.byref(p), C.byref(h)))
        self.handle = h

    def code_size(self):
        dim = self.pq_dim if self.kind == capi.KIND_PQFS else self.dim  # a pqfs code depends on pq_dim alone
        return int(self.lib.vsag_amd_code_size(self.kind, self.metric, dim, self.qbits))

    def append(self, codes):
        codes = np.ascontiguousarray(codes)
        n = codes.shape[0]
        assert codes.nbytes == n * self.code_size(), (codes.nbytes, n, self.code_size())
        buf = dev(codes)
        capi.check(self.lib.vsag_amd_store_append(self.handle, buf.ptr, n, None))
        capi.synchronize()
        buf.free()

    def set_lists(self, codes, labels, nlist):
        codes = np.ascontiguousarray(codes)
        n = codes.shape[0]
        cbuf, lbuf = dev(codes), dev(np.ascontiguousarray(labels, np.int32))
        capi.check(self.lib.vsag_amd_store_set_lists(self.handle, cbuf.ptr, lbuf.ptr, n, nlist, None))
        capi.synchronize()
        cbuf.free()
        lbuf.free()

    def append_lists(self, codes, labels, bias=None):
        codes = np.ascontiguousarray(codes)
        cbuf, lbuf = dev(codes), dev(np.ascontiguousarray(labels, np.int32))
        bbuf = dev(np.ascontiguousarray(bias, np.float32)) if bias is not None else None
        capi.check(self.lib.vsag_amd_store_append_lists(self.handle, cbuf.ptr, lbuf.ptr,
                                                        bbuf.ptr if bbuf is not None else None, codes.shape[0], None))
        capi.synchronize()
        for b in (cbuf, lbuf, bbuf):
            if b is not None:
                b.free()

    def size(self):
        return int(self.lib.vsag_amd_store_size(self.handle))

    def _options(self, deny, radius):
        """(options pointer or None, buffers to free).  deny: boolean array over inner ids (True = filtered out)."""
        if deny is None and radius is None:
            return None, []
        opt = capi.SearchOptions()
        keep = []
        if deny is not None:
            bits = np.packbits(np.asarray(deny, bool), bitorder="little")
            words = np.zeros((bits.size + 3) // 4 * 4, np.uint8)
            words[:bits.size] = bits
            buf = dev(words.view(np.uint32))
            keep.append(buf)
            opt.deny_bits_dev = buf.ptr
        if radius is not None:
            opt.use_radius, opt.radius = 1, float(radius)
        return opt, keep

    def flat_scan(self, queries, k, deny=None, radius=None):
        q = np.ascontiguousarray(queries, np.float32)
        nq = q.shape[0]
        qb = dev(q)
        opt, keep = self._options(deny, radius)
        if opt is not None:
            ids = capi.DeviceBuffer(nq * k * 4)
            ds = capi.DeviceBuffer(nq * k * 4)
            wsb = self.lib.vsag_amd_flat_scan_workspace_bytes(self.handle, nq, k)
            ws = capi.DeviceBuffer(wsb)
            capi.check(self.lib.vsag_amd_flat_scan_topk_ex(self.handle, qb.ptr, nq, k, C.byref(opt), ids.ptr, ds.ptr,
                                                          ws.ptr, wsb, None))
            out = ids.to_numpy(np.uint32, (nq, k)), ds.to_numpy(np.float32, (nq, k))
            for b in [qb, ids, ds, ws] + keep:
                b.free()
            return out
        ids = capi.DeviceBuffer(nq * k * 4)
        ds = capi.DeviceBuffer(nq * k * 4)
        wsb = self.lib.vsag_amd_flat_scan_workspace_bytes(self.handle, nq, k)
        ws = capi.DeviceBuffer(wsb)
        capi.check(self.lib.vsag_amd_flat_scan_topk(self.handle, qb.ptr, nq, k, ids.ptr, ds.ptr, ws.ptr, wsb, None))
        out = ids.to_numpy(np.uint32, (nq, k)), ds.to_numpy(np.float32, (nq, k))
        for b in (qb, ids, ds, ws):
            b.free()
        return out

    def ivf_scan(self, queries, buckets, kcand, deny=None, radius=None):
        q = np.ascontiguousarray(queries, np.float32)
        b = np.ascontiguousarray(buckets, np.int32)
        nq, nprobe = b.shape
        qb, bb = dev(q), dev(b)
        opt, keep = self._options(deny, radius)
        if opt is not None:
            ids = capi.DeviceBuffer(nq * kcand * 4)
            ds = capi.DeviceBuffer(nq * kcand * 4)
            wsb = self.lib.vsag_amd_ivf_scan_workspace_bytes(self.handle, nq, nprobe, kcand)
            ws = capi.DeviceBuffer(wsb)
            capi.check(self.lib.vsag_amd_ivf_scan_topk_ex(self.handle, qb.ptr, nq, bb.ptr, nprobe, kcand, C.byref(opt),
                                                         ids.ptr, ds.ptr, ws.ptr, wsb, None))
            out = ids.to_numpy(np.uint32, (nq, kcand)), ds.to_numpy(np.float32, (nq, kcand))
            for x in [qb, bb, ids, ds, ws] + keep:
                x.free()
            return out
        ids = capi.DeviceBuffer(nq * kcand * 4)
        ds = capi.DeviceBuffer(nq * kcand * 4)
        wsb = self.lib.vsag_amd_ivf_scan_workspace_bytes(self.handle, nq, nprobe, kcand)
        ws = capi.DeviceBuffer(wsb)
        capi.check(self.lib.vsag_amd_ivf_scan_topk(self.handle, qb.ptr, nq, bb.ptr, nprobe, kcand, ids.ptr, ds.ptr,
                                                   ws.ptr, wsb, None))
        out = ids.to_numpy(np.uint32, (nq, kcand)), ds.to_numpy(np.float32, (nq, kcand))
        for x in (qb, bb, ids, ds, ws):
            x.free()
        return out

    def destroy(self):
        if self.handle is not None:
            self.lib.vsag_amd_store_destroy(self.handle)
            self.handle = None
            for b in self._keep:
                b.free()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def assert_topk_close(gpu_ids, gpu_d, ref_ids, ref_d, rtol=1e-4, atol=1e-6, tie_rtol=1e-4, label=""):
    """Distances agree within rtol position by position; ids agree as sets except for candidates that sit
    in the tie band of the k-th distance (the reference leaves the order of equal distances open)."""
    gpu_ids, ref_ids = np.asarray(gpu_ids), np.asarray(ref_ids)
    gpu_d, ref_d = np.asarray(gpu_d, np.float64), np.asarray(ref_d, np.float64)
    assert gpu_ids.shape == ref_ids.shape, (gpu_ids.shape, ref_ids.shape)
    finite = np.isfinite(ref_d)
    assert np.array_equal(finite, np.isfinite(gpu_d)), label + ": different number of results"
    err = np.abs(gpu_d[finite] - ref_d[finite])
    bound = atol + rtol * np.abs(ref_d[finite])
    assert np.all(err <= bound), "%s: distance mismatch, worst %.3e (allowed %.3e)" % (
        label, float((err - bound).max() + bound[np.argmax(err - bound)]), float(bound[np.argmax(err - bound)]))
    bad = 0
    for q in range(gpu_ids.shape[0]):
        g = {int(i): d for i, d in zip(gpu_ids[q], gpu_d[q]) if np.isfinite(d)}
        r = {int(i): d for i, d in zip(ref_ids[q], ref_d[q]) if np.isfinite(d)}
        if set(g) == set(r):
            continue
        kth = max(r.values())
        band = atol + tie_rtol * abs(kth)
        for i in set(g) - set(r):
            if abs(g[i] - kth) > band:
                bad += 1
        for i in set(r) - set(g):
            if abs(r[i] - kth) > band:
                bad += 1
    assert bad == 0, "%s: %d ids differ outside the tie band" % (label, bad)
    assert np.all(gpu_ids[~finite] == 0xFFFFFFFF), label + ": padding ids must be INVALID"


def gaussian_mixture(rng, n, d, components, sigma, means=None, uniform_means=True):
    if means is None:
        means = rng.random((components, d), dtype=np.float32) if uniform_means else \
            rng.standard_normal((components, d)).astype(np.float32)
    which = rng.integers(0, components, n)
    x = means[which] + sigma * rng.standard_normal((n, d)).astype(np.float32)
    return x.astype(np.float32), means
