"""Large batches on fp32 posting lists (the reference's default ivf codec, src/algorithm/ivf/ivf.cpp:60-130) and on sq8
lists of more than 128 dimensions: the probe columns behind the first are pre-selected on the fp32 matrix cores and
what passes is rescored with the streaming kernel's arithmetic, so ids and distance bits equal the streaming scan's."""
import numpy as np
import pytest

import oracle as orc
from gpu_helpers import Store, assert_topk_close, dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def _case(seed, n, d, nlist, nq, kind, components=40, sigma=0.05, metric=orc.L2):
    rng = np.random.default_rng(seed)
    x, means = gaussian_mixture(rng, n, d, components, sigma)
    q, _ = gaussian_mixture(rng, nq, d, components, sigma, means=means)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    if kind == "fp32":
        codes = x.view(np.uint8).reshape(n, 4 * d)
        st = Store(capi.KIND_FP32, metric, d)
        params = (None, None)
    else:
        lb, diff = orc.sq_train(x, 8, metric)
        codes = orc.sq_encode(x, 8, lb, diff, metric)
        st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
        params = (lb, diff)
    st.set_lists(codes, labels, nlist)
    return x, q, cent, labels, codes, params, st


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


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
@pytest.mark.parametrize("kind,n,d,nlist,nq,nprobe,kcand", [
    ("fp32", 60000, 128, 64, 2100, 16, 100), ("fp32", 30000, 100, 37, 4500, 8, 10), ("fp32", 20000, 33, 16, 9000, 4, 32),
    ("fp32", 20000, 7, 16, 9000, 4, 5), ("fp32", 12000, 960, 16, 9000, 4, 10),
    ("sq8", 20000, 200, 20, 7000, 6, 10), ("sq8", 12000, 960, 16, 9000, 4, 10)])
def test_fp32_matrix_core_columns_equal_streaming(lib, metric, kind, n, d, nlist, nq, nprobe, kcand):
    x, q, cent, labels, codes, (lb, diff), st = _case(n + d + metric, n, d, nlist, nq, kind, metric=metric)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1      # three queries without a first list: no bound, served by the direct fallback launch
    buckets[80, 0] = buckets[80, nprobe - 1]  # a far list first (and probed twice): a loose bound
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    if kind == "sq8":
        offsets, order = orc.ivf_build_lists(labels, nlist)
        qs, om = q[:32], metric
        if metric == orc.COSINE:
            qs, om = (qs / np.linalg.norm(qs, axis=1, keepdims=True)).astype(np.float32), orc.IP
        rids, rds = orc.ivf_scan(orc.SQ8, om, d, codes[order], offsets, order, qs, buckets[:32], kcand, lb=lb, diff=diff)
        assert_topk_close(fast[0][:32], fast[1][:32], rids, rds, rtol=2e-5, atol=1e-5, tie_rtol=2e-5,
                          label="ivf sq8 beyond 128 dimensions on the matrix cores")
    st.destroy()


def test_fp32_overflowing_lists_fall_back_to_streaming(lib):
    n, d, nlist, nq, nprobe, kcand = 40000, 64, 8, 9000, 4, 10
    x, q, cent, labels, codes, _, st = _case(11, n, d, nlist, nq, "fp32", components=8, sigma=0.02)
    routed, _ = orc.ivf_route(cent, q, nlist)
    buckets = np.ascontiguousarray(routed[:, [nlist - 1, 0, 1, 2]])  # farthest list first, then the nearest three
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


def test_fp32_duplicates_and_ragged_lists(lib):
    """Many equal vectors (equal distances: the candidates of a pair overflow its private lists and the query streams)
    and lists of very different lengths, some empty."""
    n, d, nlist, nq, nprobe, kcand = 30000, 48, 40, 4000, 10, 20
    rng = np.random.default_rng(3)
    x, q, cent, labels, codes, _, st0 = _case(5, n, d, nlist, nq, "fp32")
    st0.destroy()
    x[:4000] = x[0]
    labels = labels.copy()
    labels[labels == 3] = 4      # an empty list
    labels[:4000] = 7            # a long list of duplicates
    st = Store(capi.KIND_FP32, orc.L2, d)
    st.set_lists(x.view(np.uint8).reshape(n, 4 * d), labels, nlist)
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    st.destroy()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP])
@pytest.mark.parametrize("kind,n,d,nlist,nq,nprobe,kcand", [
    ("fp32", 30000, 96, 40, 4500, 8, 10), ("fp32", 20000, 33, 16, 9000, 4, 32), ("fp32", 12000, 960, 16, 9000, 4, 10),
    ("sq8", 20000, 64, 20, 7000, 6, 10), ("sq8", 20000, 200, 20, 7000, 6, 100)])
def test_residual_lists_on_the_matrix_cores_equal_streaming(lib, metric, kind, n, d, nlist, nq, nprobe, kcand):
    """use_residual (bucket_datacell.h:527-572,594-639): codes of x - c.  The slot's bias joins the code's term and the
    pair's <q, c> the threshold of the fp32 matrix-core test, and the rescoring takes both off in the streaming kernel's
    order, so ids and distance bits equal the streaming scan's; with fp32 codes the result is the plain scan of x again."""
    L = lib.load_library()
    rng = np.random.default_rng(n + d + metric)
    x, means = gaussian_mixture(rng, n, d, 40, 0.05)
    q, _ = gaussian_mixture(rng, nq, d, 40, 0.05, means=means)
    x, q = (x - 0.3).astype(np.float32), (q - 0.3).astype(np.float32)
    cent = x[rng.choice(n, nlist, replace=False)].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    res = orc.residual_rows(x, labels, cent, metric)
    if kind == "fp32":
        codes, dec = res.view(np.uint8).reshape(n, 4 * d), res
        st = Store(capi.KIND_FP32, metric, d)
    else:
        lb, diff = orc.sq_train(res, 8, metric)
        codes = orc.sq_encode(res, 8, lb, diff, metric)
        dec = orc.sq_decode(codes, d, 8, lb, diff)
        st = Store(capi.KIND_SQ8, metric, d, lb=lb, diff=diff)
    bias = orc.residual_bias(dec, labels, cent) if metric == orc.L2 else None
    cb = dev(cent)
    capi.check(L.vsag_amd_store_set_residual(st.handle, cb.ptr, nlist, None))
    st.set_lists(codes[:0], labels[:0], nlist)
    half = n // 3
    st.append_lists(codes[:half], labels[:half], None if bias is None else bias[:half])
    st.append_lists(codes[half:], labels[half:], None if bias is None else bias[half:])
    buckets, _ = orc.ivf_route(cent, q, nprobe)
    buckets = buckets.copy()
    buckets[70:73, 0] = -1
    buckets[80, 0] = buckets[80, nprobe - 1]
    plain, fast = _both(lib, st, q, buckets, kcand)
    assert _same(plain, fast)
    if kind == "fp32":
        direct = Store(capi.KIND_FP32, metric, d)
        direct.set_lists(x.view(np.uint8).reshape(n, 4 * d), labels, nlist)
        pi, pd = direct.ivf_scan(q[:256], buckets[:256], kcand)
        assert_topk_close(fast[0][:256], fast[1][:256], pi, pd, rtol=2e-4, atol=5e-4 if d > 500 else 5e-5, tie_rtol=5e-4,
                          label="residual fp32 lists against the plain scan")
        direct.destroy()
    cb.free()
    st.destroy()
