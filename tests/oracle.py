"""ctypes access to the CPU checker (oracle/liboracle.so) and, when built, to the reference's own scalar
kernels compiled from its sources (oracle/_ref/libvsag_simd.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "liboracle.so")
REF_SIMD = os.path.join(ORACLE_DIR, "_ref", "libvsag_simd.so")

L2, IP, COSINE = 0, 1, 2
FP32, SQ8, SQ4, SQ4U, SQ8U, RABITQ, PQFS = range(7)
KIND_BITS = {SQ8: 8, SQ4: 4, SQ4U: 4, SQ8U: 8}

_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_lib = None


def build():
    subprocess.run(["make", "-C", ORACLE_DIR, "liboracle.so"], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
        _lib.orc_kmeans_assign.restype = C.c_double
        _lib.orc_kmeans_run.restype = C.c_double
        _lib.orc_kmeans_run_with.restype = C.c_double
        for name in ("orc_fp32_l2sqr", "orc_fp32_ip", "orc_sq8_ip", "orc_sq8_l2sqr", "orc_sq4_ip", "orc_sq4_l2sqr",
                     "orc_squ_dist", "orc_rabitq_dist", "orc_normalize", "orc_normalize_with_centroid",
                     "orc_rabitq_float_binary_ip", "orc_rabitq_float_planes_ip", "orc_rabitq_float_sq_ip"):
            getattr(_lib, name).restype = C.c_float
        for name in ("orc_squ_code_size", "orc_rabitq_code_size", "orc_rabitq_query_code_size"):
            getattr(_lib, name).restype = C.c_uint64
        _lib.orc_rabitq_sq4u_binary_ip.restype = C.c_uint32
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def u64(v):
    return C.c_uint64(int(v))


def set_threads(threads):
    """OpenMP threads of the checker's parallel loops from now on."""
    lib().orc_set_threads(int(threads))


def sq_train(x, bits, metric=L2, mode=3, trunc_rate=0.05, max_sample=0):
    x = f32(x)
    n, d = x.shape
    lb = np.empty(d, np.float32)
    diff = np.empty(d, np.float32)
    lib().orc_sq_train(_p(x), u64(n), u64(d), bits, metric, mode, C.c_float(trunc_rate), u64(max_sample), _p(lb),
                       _p(diff))
    return lb, diff


def sq_train_uniform(x, bits, metric=L2, mode=3, trunc_rate=0.05, max_sample=0):
    x = f32(x)
    n, d = x.shape
    lb = C.c_float()
    diff = C.c_float()
    lib().orc_sq_train_uniform(_p(x), u64(n), u64(d), bits, metric, mode, C.c_float(trunc_rate), u64(max_sample),
                               C.byref(lb), C.byref(diff))
    return np.float32(lb.value), np.float32(diff.value)


def sq_encode(x, bits, lb, diff, metric=L2):
    x = f32(x)
    n, d = x.shape
    cs = (d * bits + 7) // 8
    codes = np.zeros((n, cs), np.uint8)
    lib().orc_sq_encode(_p(x), u64(n), u64(d), bits, metric, _p(f32(lb)), _p(f32(diff)), _p(codes))
    return codes


def sq_decode(codes, d, bits, lb, diff):
    n = codes.shape[0]
    out = np.empty((n, d), np.float32)
    lib().orc_sq_decode(_p(np.ascontiguousarray(codes)), u64(n), u64(d), bits, _p(f32(lb)), _p(f32(diff)), _p(out))
    return out


def squ_code_size(d, bits, metric):
    return int(lib().orc_squ_code_size(u64(d), bits, metric))


def squ_encode(x, bits, lb, diff, metric=L2):
    x = f32(x)
    n, d = x.shape
    cs = squ_code_size(d, bits, metric)
    codes = np.zeros((n, cs), np.uint8)
    lib().orc_squ_encode(_p(x), u64(n), u64(d), bits, metric, C.c_float(lb), C.c_float(diff), _p(codes))
    return codes


def rabitq_code_size(d, metric, qbits=4):
    return int(lib().orc_rabitq_code_size(u64(d), metric, qbits))


def rabitq_query_code_size(d, metric, qbits=4):
    return int(lib().orc_rabitq_query_code_size(u64(d), metric, qbits))


def rabitq_train(x, rot):
    x = f32(x)
    n, d = x.shape
    c = np.empty(d, np.float32)
    lib().orc_rabitq_train(_p(x), u64(n), u64(d), _p(f32(rot)), _p(c))
    return c


def rabitq_encode(x, rot, centroid, metric, qbits=4):
    x = f32(x)
    n, d = x.shape
    codes = np.zeros((n, rabitq_code_size(d, metric, qbits)), np.uint8)
    lib().orc_rabitq_encode(_p(x), u64(n), u64(d), _p(f32(rot)), _p(f32(centroid)), metric, qbits, _p(codes))
    return codes


def rabitq_decode(codes, d, rot, centroid, metric, qbits=4):
    """RaBitQuantizer::DecodeOneImpl; None where the reference returns false (multi-bit codes)."""
    codes = np.ascontiguousarray(codes, np.uint8)
    out = np.zeros((codes.shape[0], d), np.float32)
    ok = lib().orc_rabitq_decode(_p(codes), u64(codes.shape[0]), u64(d), _p(f32(rot)), _p(f32(centroid)), metric, qbits,
                                 _p(out))
    return out if ok else None


def fht_primitive(which, data, flip=None, val=0.0):
    """0 FlipSign, 1 VecRescale, 2 FHTRotate, 3 KacsWalk of the reference's generic kernels, on a copy."""
    out = f32(data).copy()
    fp = _p(np.ascontiguousarray(flip, np.uint8)) if flip is not None else None
    lib().orc_fht_primitive(which, fp, _p(out), u64(out.shape[0]), C.c_float(val))
    return out


def fht_kac_transform(flip, x, inverse=False):
    """FhtKacRotator::Transform / InverseTransform of every row of x with the sign bits `flip` (4 x ceil(d / 8) bytes)."""
    x = f32(np.atleast_2d(x))
    flip = np.ascontiguousarray(flip, np.uint8)
    out = np.empty_like(x)
    for i in range(x.shape[0]):
        lib().orc_fht_kac_transform(_p(flip), u64(x.shape[1]), 1 if inverse else 0, _p(x[i]), _p(out[i]))
    return out


def rabitq_bits(qbits, base_bits=1):
    """The `qbits` argument of every rabitq function here: query bits (4 | 32) plus 256 * base bits for multi-bit base
    codes (rabitq_bits_per_dim_base 2..8, fp32 queries only)."""
    return qbits if base_bits == 1 else (qbits | (base_bits << 8))


def rabitq_encode_multibit(x, rot, centroid, metric, base_bits, fast=True, rounds=6):
    """RaBitQuantizer::EncodeOneInternal with rabitq_bits_per_dim_base = base_bits (2..8) and fp32 queries."""
    x = f32(x)
    n, d = x.shape
    qbits = rabitq_bits(32, base_bits)
    codes = np.zeros((n, rabitq_code_size(d, metric, qbits)), np.uint8)
    lib().orc_rabitq_encode_multibit(_p(x), u64(n), u64(d), _p(f32(rot)), _p(f32(centroid)), metric, qbits,
                                     1 if fast else 0, u64(rounds), _p(codes))
    return codes


def rabitq_fast_encode(o, bits, rounds=6):
    o = f32(o)
    code = np.zeros(o.shape[0], np.uint8)
    norm = C.c_float()
    lib().orc_rabitq_fast_encode(_p(o), u64(o.shape[0]), bits, u64(rounds), _p(code), C.byref(norm))
    return code, norm.value


def rabitq_extend_encode(o, bits):
    o = f32(o)
    code = np.zeros(o.shape[0], np.uint8)
    norm = C.c_float()
    lib().orc_rabitq_extend_encode(_p(o), u64(o.shape[0]), bits, _p(code), C.byref(norm))
    return code, norm.value


def rabitq_pack_planes(scalar, bits):
    scalar = np.ascontiguousarray(scalar, np.uint8)
    d = scalar.shape[0]
    planes = np.zeros((d + 7) // 8 * bits, np.uint8)
    lib().orc_rabitq_pack_planes(_p(scalar), u64(d), bits, _p(planes))
    return planes


def rabitq_float_planes_ip(v, planes, bits):
    v = f32(v)
    return float(lib().orc_rabitq_float_planes_ip(_p(v), _p(np.ascontiguousarray(planes, np.uint8)), u64(v.shape[0]),
                                                  bits))


def rabitq_float_sq_ip(v, codes):
    v = f32(v)
    return float(lib().orc_rabitq_float_sq_ip(_p(v), _p(np.ascontiguousarray(codes, np.uint8)), u64(v.shape[0])))


def rabitq_process_query(q, rot, centroid, metric, qbits=4):
    q = f32(q)
    nq, d = q.shape
    qs = rabitq_query_code_size(d, metric, qbits)
    out = np.zeros((nq, qs), np.uint8)
    rot = f32(rot)
    centroid = f32(centroid)
    for i in range(nq):
        lib().orc_rabitq_process_query(_p(q[i]), u64(d), _p(rot), _p(centroid), metric, qbits,
                                       C.c_void_p(out.ctypes.data + i * qs))
    return out


# ---- pqfs (for the scans below a PQFS store's `d` is its number of subspaces, pq_dim) ----
def pq_train(x, pq_dim, metric=L2, seed=11):
    x = f32(x)
    n, d = x.shape
    cb = np.empty((pq_dim, 16, d // pq_dim), np.float32)
    lib().orc_pq_train(_p(x), u64(n), u64(d), u64(pq_dim), metric, u64(seed), _p(cb))
    return cb


def pq_encode(x, pq_dim, codebooks, metric=L2):
    x = f32(x)
    n, d = x.shape
    codes = np.zeros((n, (pq_dim + 1) // 2), np.uint8)
    lib().orc_pq_encode(_p(x), u64(n), u64(d), u64(pq_dim), _p(f32(codebooks)), metric, _p(codes))
    return codes


def pq_decode(codes, d, pq_dim, codebooks):
    codes = np.ascontiguousarray(codes)
    out = np.empty((codes.shape[0], d), np.float32)
    lib().orc_pq_decode(_p(codes), u64(codes.shape[0]), u64(d), u64(pq_dim), _p(f32(codebooks)), _p(out))
    return out


def pqfs_process_query(q, pq_dim, codebooks, metric=L2):
    """nq x (pq_dim * 16 + 8) bytes: the byte table, then diff and lower as floats."""
    q = f32(np.atleast_2d(q))
    nq, d = q.shape
    out = np.zeros((nq, pq_dim * 16 + 8), np.uint8)
    lib().orc_pqfs_process_query(_p(q), u64(nq), u64(d), u64(pq_dim), _p(f32(codebooks)), metric, _p(out))
    return out


def pqfs_package32(codes, pq_dim, valid=-1):
    codes = np.ascontiguousarray(codes)
    cs = (pq_dim + 1) // 2
    assert codes.shape == (32, cs)
    out = np.zeros(32 * cs, np.uint8)
    lib().orc_pqfs_package32(_p(codes), u64(pq_dim), C.c_int64(valid), _p(out))
    return out


def pqfs_unpack32(packaged, pq_dim):
    packaged = np.ascontiguousarray(packaged)
    cs = (pq_dim + 1) // 2
    out = np.zeros((32, cs), np.uint8)
    lib().orc_pqfs_unpack32(_p(packaged), u64(pq_dim), _p(out))
    return out


def pqfs_lookup32(lut, packaged, pq_dim):
    out = np.zeros(32, np.int32)
    lib().orc_pqfs_lookup32(_p(np.ascontiguousarray(lut)), _p(np.ascontiguousarray(packaged)), u64(pq_dim), _p(out))
    return out


def pqfs_scan_batch(qcode, packaged, count, pq_dim, metric):
    out = np.empty(count, np.float32)
    lib().orc_pqfs_scan_batch(_p(np.ascontiguousarray(qcode)), _p(np.ascontiguousarray(packaged)), u64(count),
                              u64(pq_dim), metric, _p(out))
    return out


def ref_pqfs_lookup32(isa):
    """vsag::<isa>::PQFastScanLookUp32 of oracle/_ref as a ctypes function, or None."""
    if not os.path.exists(REF_SIMD):
        return None
    name = "PQFastScanLookUp32"
    try:
        return getattr(C.CDLL(REF_SIMD), "_ZN4vsag%d%s%d%sEPKhS2_mPi" % (len(isa), isa, len(name), name))
    except AttributeError:
        return None


def flat_scan_topk(kind, metric, d, codes, queries, k, lb=None, diff=None, qbits=4, strict=False, threads=0):
    """codes: (n, code_size) uint8 (fp32 rows viewed as bytes); queries: processed queries, 2-D."""
    codes = np.ascontiguousarray(codes)
    queries = np.ascontiguousarray(queries)
    n = codes.shape[0]
    cs = codes.shape[1] * codes.itemsize
    nq = queries.shape[0]
    qstride = queries.shape[1] * queries.itemsize
    ids = np.empty((nq, k), np.uint32)
    dists = np.empty((nq, k), np.float32)
    lbp = _p(f32(np.atleast_1d(lb))) if lb is not None else None
    dfp = _p(f32(np.atleast_1d(diff))) if diff is not None else None
    lib().orc_flat_scan_topk(kind, metric, u64(d), _p(codes), u64(n), u64(cs), lbp, dfp, qbits, _p(queries), u64(nq),
                             u64(qstride), u64(k), int(strict), _p(ids), _p(dists), threads)
    return ids, dists


def flat_dists(kind, metric, d, codes, queries, lb=None, diff=None, qbits=4):
    codes = np.ascontiguousarray(codes)
    queries = np.ascontiguousarray(queries)
    n = codes.shape[0]
    cs = codes.shape[1] * codes.itemsize
    nq = queries.shape[0]
    qstride = queries.shape[1] * queries.itemsize
    out = np.empty((nq, n), np.float32)
    lbp = _p(f32(np.atleast_1d(lb))) if lb is not None else None
    dfp = _p(f32(np.atleast_1d(diff))) if diff is not None else None
    lib().orc_flat_dists(kind, metric, u64(d), _p(codes), u64(n), u64(cs), lbp, dfp, qbits, _p(queries), u64(nq),
                         u64(qstride), _p(out))
    return out


def kmeans_assign(x, cent):
    x = f32(x)
    cent = f32(cent)
    n, d = x.shape
    k = cent.shape[0]
    labels = np.empty(n, np.int32)
    mind = np.empty(n, np.float32)
    loss = lib().orc_kmeans_assign(_p(x), u64(n), u64(d), _p(cent), u64(k), _p(labels), _p(mind))
    return labels, mind, loss


def kmeans_update(x, labels, cent):
    x = f32(x)
    cent = f32(cent).copy()
    n, d = x.shape
    k = cent.shape[0]
    counts = np.empty(k, np.int32)
    lib().orc_kmeans_update(_p(x), _p(np.ascontiguousarray(labels, np.int32)), u64(n), u64(d), u64(k), _p(cent),
                            _p(counts))
    return cent, counts


def kmeans_init_pp(x, k, first, draws):
    """k-means++ seeding with the random draws given: (centroids, picked rows)."""
    x = f32(x)
    n, d = x.shape
    draws = np.ascontiguousarray(draws, np.float64)
    assert draws.shape[0] >= k - 1
    cent = np.empty((k, d), np.float32)
    picks = np.empty(k, np.uint64)
    lib().orc_kmeans_init_pp(_p(x), u64(n), u64(d), u64(k), u64(first), _p(draws), _p(cent), _p(picks))
    return cent, picks


def kmeans_run(x, cent0, iters, seed):
    x = f32(x)
    cent = f32(cent0).copy()
    n, d = x.shape
    k = cent.shape[0]
    labels = np.empty(n, np.int32)
    loss = lib().orc_kmeans_run(_p(x), u64(n), u64(d), _p(cent), u64(k), iters, u64(seed), _p(labels))
    return cent, labels, loss


def kmeans_run_with(x, cent0, iters, seed, assign):
    """kmeans_run with the assignment step done by `assign(cent[k, d]) -> (labels[n], err / n)` (the update and the
    re-seeding of empty clusters stay the checker's)."""
    x = f32(x)
    cent = f32(cent0).copy()
    n, d = x.shape
    k = cent.shape[0]
    labels = np.empty(n, np.int32)

    @C.CFUNCTYPE(C.c_double, C.POINTER(C.c_float), C.POINTER(C.c_int32), C.c_void_p)
    def step(cent_p, labels_p, _user):
        c = np.ctypeslib.as_array(cent_p, shape=(k, d))
        out, err = assign(c)
        np.ctypeslib.as_array(labels_p, shape=(n,))[:] = out
        return float(err)

    loss = lib().orc_kmeans_run_with(_p(x), u64(n), u64(d), _p(cent), u64(k), iters, u64(seed), _p(labels), step, None)
    return cent, labels, loss


def ivf_route(cent, queries, nprobe, metric=L2):
    cent = f32(cent)
    queries = f32(queries)
    nlist, d = cent.shape
    nq = queries.shape[0]
    b = np.empty((nq, nprobe), np.int32)
    ds = np.empty((nq, nprobe), np.float32)
    lib().orc_ivf_route(_p(cent), u64(nlist), u64(d), metric, _p(queries), u64(nq), u64(nprobe), _p(b), _p(ds))
    return b, ds


def ivf_build_lists(labels, nlist):
    labels = np.ascontiguousarray(labels, np.int32)
    n = labels.shape[0]
    offsets = np.empty(nlist + 1, np.uint64)
    order = np.empty(n, np.uint32)
    lib().orc_ivf_build_lists(_p(labels), u64(n), u64(nlist), _p(offsets), _p(order))
    return offsets, order


def ivf_scan(kind, metric, d, codes_posting, offsets, order, queries, buckets, kcand, lb=None, diff=None, qbits=4,
             threads=0):
    codes = np.ascontiguousarray(codes_posting)
    queries = np.ascontiguousarray(queries)
    buckets = np.ascontiguousarray(buckets, np.int32)
    cs = codes.shape[1] * codes.itemsize
    nq, nprobe = buckets.shape
    qstride = queries.shape[1] * queries.itemsize
    ids = np.empty((nq, kcand), np.uint32)
    dists = np.empty((nq, kcand), np.float32)
    lbp = _p(f32(np.atleast_1d(lb))) if lb is not None else None
    dfp = _p(f32(np.atleast_1d(diff))) if diff is not None else None
    lib().orc_ivf_scan(kind, metric, u64(d), _p(codes), u64(cs), lbp, dfp, qbits,
                       _p(np.ascontiguousarray(offsets, np.uint64)), _p(np.ascontiguousarray(order, np.uint32)),
                       _p(queries), u64(nq), u64(qstride), _p(buckets), u64(nprobe), u64(kcand), _p(ids), _p(dists),
                       threads)
    return ids, dists


def residual_rows(x, labels, cent, metric=L2):
    x = f32(x)
    n, d = x.shape
    out = np.empty((n, d), np.float32)
    lib().orc_residual_rows(_p(x), u64(n), u64(d), metric, _p(np.ascontiguousarray(labels, np.int32)), _p(f32(cent)),
                            _p(out))
    return out


def squ_decode(codes, d, bits, lb, diff, metric=L2):
    codes = np.ascontiguousarray(codes)
    n = codes.shape[0]
    out = np.empty((n, d), np.float32)
    lib().orc_squ_decode(_p(codes), u64(n), u64(d), bits, metric, C.c_float(lb), C.c_float(diff), _p(out))
    return out


def residual_bias(decoded, labels, cent):
    decoded = f32(decoded)
    n, d = decoded.shape
    out = np.empty(n, np.float32)
    lib().orc_residual_bias(_p(decoded), u64(n), u64(d), _p(np.ascontiguousarray(labels, np.int32)), _p(f32(cent)), _p(out))
    return out


def ivf_scan_residual(kind, metric, d, codes_posting, offsets, order, queries, raw_queries, cent, bias_posting, buckets,
                      kcand, lb=None, diff=None, qbits=4):
    codes = np.ascontiguousarray(codes_posting)
    queries = np.ascontiguousarray(queries)
    buckets = np.ascontiguousarray(buckets, np.int32)
    cs = codes.shape[1] * codes.itemsize
    nq, nprobe = buckets.shape
    qstride = queries.shape[1] * queries.itemsize
    ids = np.empty((nq, kcand), np.uint32)
    dists = np.empty((nq, kcand), np.float32)
    lbp = _p(f32(np.atleast_1d(lb))) if lb is not None else None
    dfp = _p(f32(np.atleast_1d(diff))) if diff is not None else None
    bp = _p(f32(bias_posting)) if bias_posting is not None else None
    lib().orc_ivf_scan_residual(kind, metric, u64(d), _p(codes), u64(cs), lbp, dfp, qbits,
                                _p(np.ascontiguousarray(offsets, np.uint64)), _p(np.ascontiguousarray(order, np.uint32)),
                                _p(queries), u64(nq), u64(qstride), _p(f32(raw_queries)), _p(f32(cent)), bp, _p(buckets),
                                u64(nprobe), u64(kcand), _p(ids), _p(dists))
    return ids, dists


def rerank_fp32(raw, queries, cand, k, metric=L2):
    raw = f32(raw)
    queries = f32(queries)
    cand = np.ascontiguousarray(cand, np.uint32)
    nq, kcand = cand.shape
    d = raw.shape[1]
    ids = np.empty((nq, k), np.uint32)
    dists = np.empty((nq, k), np.float32)
    lib().orc_rerank_fp32(_p(raw), u64(d), metric, _p(queries), u64(nq), _p(cand), u64(kcand), u64(k), _p(ids),
                          _p(dists))
    return ids, dists


# ---- the reference's own scalar kernels, compiled from its sources (when oracle/_ref was built) ----------
_ref = None
_REF_SYMBOLS = {
    "FP32ComputeIP": "_ZN4vsag7generic13FP32ComputeIPEPKfS2_m",
    "FP32ComputeL2Sqr": "_ZN4vsag7generic16FP32ComputeL2SqrEPKfS2_m",
    "SQ8ComputeIP": "_ZN4vsag7generic12SQ8ComputeIPEPKfPKhS2_S2_m",
    "SQ8ComputeL2Sqr": "_ZN4vsag7generic15SQ8ComputeL2SqrEPKfPKhS2_S2_m",
    "SQ4ComputeIP": "_ZN4vsag7generic12SQ4ComputeIPEPKfPKhS2_S2_m",
    "SQ4ComputeL2Sqr": "_ZN4vsag7generic15SQ4ComputeL2SqrEPKfPKhS2_S2_m",
    "SQ4UniformComputeCodesIP": "_ZN4vsag7generic24SQ4UniformComputeCodesIPEPKhS2_m",
    "SQ8UniformComputeCodesIP": "_ZN4vsag7generic24SQ8UniformComputeCodesIPEPKhS2_m",
    "RaBitQSQ4UBinaryIP": "_ZN4vsag7generic18RaBitQSQ4UBinaryIPEPKhS2_m",
    "RaBitQFloatBinaryIP": "_ZN4vsag7generic19RaBitQFloatBinaryIPEPKfPKhmf",
    "RaBitQFloatSQIP": "_ZN4vsag7generic15RaBitQFloatSQIPEPKfPKhm",
    "RaBitQFloatSplitCodeIP": "_ZN4vsag7generic22RaBitQFloatSplitCodeIPEPKfPKhS4_mj",
    "NormalizeWithCentroid": "_ZN4vsag7generic21NormalizeWithCentroidEPKfS2_Pfm",
    "InverseNormalizeWithCentroid": "_ZN4vsag7generic28InverseNormalizeWithCentroidEPKfS2_Pfmf",
    "FlipSign": "_ZN4vsag7generic8FlipSignEPKhPfm",
    "VecRescale": "_ZN4vsag7generic10VecRescaleEPfmf",
    "FHTRotate": "_ZN4vsag7generic9FHTRotateEPfm",
    "KacsWalk": "_ZN4vsag7generic8KacsWalkEPfm",
    "Normalize": "_ZN4vsag7generic9NormalizeEPKfPfm",
}


def ref():
    """dict name -> ctypes function of vsag::generic, or None when oracle/_ref is not built."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SIMD):
            return None
        dll = C.CDLL(REF_SIMD)
        fns = {}
        for name, sym in _REF_SYMBOLS.items():
            fn = getattr(dll, sym)
            fn.restype = C.c_uint32 if name == "RaBitQSQ4UBinaryIP" else C.c_float
            fns[name] = fn
        _ref = fns
    return _ref


def ref_best_isa():
    """Highest ISA tier of the reference's kernels this host can execute: 'avx512', 'avx2' or 'generic'."""
    if lib().orc_cpu_has_avx512():
        return "avx512"
    if lib().orc_cpu_has_avx2():
        return "avx2"
    return "generic"


def ref_sq8_fn(metric, isa):
    """Address of vsag::<isa>::SQ8ComputeL2Sqr / SQ8ComputeIP in oracle/_ref, or None."""
    if not os.path.exists(REF_SIMD):
        return None
    dll = C.CDLL(REF_SIMD)
    name = "SQ8ComputeL2Sqr" if metric == L2 else "SQ8ComputeIP"
    sym = "_ZN4vsag%d%s%d%sEPKfPKhS2_S2_m" % (len(isa), isa, len(name), name)
    return C.cast(getattr(dll, sym), C.c_void_p)


def use_reference_kernels(isa):
    """Puts the reference's compiled kernels of tier `isa` (oracle/_ref) under the checker's scan loops, for timing
    a CPU baseline; None restores the scalar restatements.  Returns the names that were found, or None when
    oracle/_ref is not built."""
    if isa is None or not os.path.exists(REF_SIMD):
        lib().orc_set_reference_kernels(None, None, None, None, None)
        return None
    dll = C.CDLL(REF_SIMD)
    found = {}

    def sym(name, args, tiers):
        for t in tiers:
            s = "_ZN4vsag%d%s%d%sE%s" % (len(t), t, len(name), name, args)
            try:
                found[name] = "vsag::%s::%s" % (t, name)
                return C.cast(getattr(dll, s), C.c_void_p)
            except AttributeError:
                found.pop(name, None)
        return None

    tiers = {"avx512": ["avx512", "avx2", "avx", "sse", "generic"], "avx2": ["avx2", "avx", "sse", "generic"],
             "generic": ["generic"]}[isa]
    pop = (["avx512vpopcntdq"] if isa == "avx512" and lib().orc_cpu_has_avx512vpopcntdq() else []) + tiers
    lib().orc_set_reference_kernels(sym("FP32ComputeL2Sqr", "PKfS2_m", tiers), sym("FP32ComputeIP", "PKfS2_m", tiers),
                                    sym("SQ4UniformComputeCodesIP", "PKhS2_m", tiers),
                                    sym("SQ8UniformComputeCodesIP", "PKhS2_m", tiers),
                                    sym("RaBitQSQ4UBinaryIP", "PKhS2_m", pop))
    return found


def flat_scan_topk_fn(fn, metric, d, codes, queries, k, lb, diff, threads=0):
    codes = np.ascontiguousarray(codes)
    queries = f32(queries)
    n, cs = codes.shape
    nq = queries.shape[0]
    ids = np.empty((nq, k), np.uint32)
    dists = np.empty((nq, k), np.float32)
    lib().orc_flat_scan_topk_fn(fn, metric, u64(d), _p(codes), u64(n), u64(cs), _p(f32(lb)), _p(f32(diff)),
                                _p(queries), u64(nq), u64(k), _p(ids), _p(dists), threads)
    return ids, dists


def rabitq_encode_sq(normed):
    normed = f32(normed)
    d = normed.shape[0]
    quant = np.zeros(d, np.uint8)
    ub, lb, delta, qsum = C.c_float(), C.c_float(), C.c_float(), C.c_float()
    lib().orc_rabitq_encode_sq(_p(normed), u64(d), _p(quant), C.byref(ub), C.byref(lb), C.byref(delta),
                               C.byref(qsum))
    return quant, ub.value, lb.value, delta.value, qsum.value


def rabitq_reorder_sq(quant):
    quant = np.ascontiguousarray(quant, np.uint8)
    d = quant.shape[0]
    plane_bytes = (d + 511) // 512 * 512 // 8
    planes = np.zeros(4 * plane_bytes, np.uint8)
    lib().orc_rabitq_reorder_sq(_p(quant), u64(d), _p(planes))
    return planes, plane_bytes
