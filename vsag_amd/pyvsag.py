"""Python view of the GPU-backed index classes with the call shapes of the reference's pyvsag.Index
(python_bindings/index_binding.cpp:641-716): Index(name, parameters), build(vectors, ids, num_elements, dim),
add(...), knn_search(vector, k, parameters) -> (ids, dists), range_search(point, threshold, parameters),
get_num_elements(), train(...), cal_distance_by_id(query, ids, ...), serialize(path) / deserialize(path) (the file forms of
the binding's save / load).  Additions: knn_search_batch (many queries per
call, optionally with the buckets every query scans), the `filter` / `limit` keywords (the C API's *_with_filter entry
points: filter(label) == True filters the vector out) and `statistics=True` (the search's statistics JSON as a third
result).  Everything goes through libvsag_amd_host.so's C API; errors raise
VsagError with the reference's error code."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libvsag_amd_host.so")

ERROR_NAMES = {0: "SUCCESS", -1: "UNKNOWN_ERROR", -2: "INTERNAL_ERROR", -3: "INVALID_ARGUMENT", -4: "WRONG_STATUS",
               -5: "BUILD_TWICE", -6: "INDEX_NOT_EMPTY", -7: "UNSUPPORTED_INDEX", -8: "UNSUPPORTED_INDEX_OPERATION",
               -9: "DIMENSION_NOT_EQUAL", -10: "INDEX_EMPTY", -11: "NO_ENOUGH_MEMORY", -12: "READ_ERROR",
               -13: "MISSING_FILE", -14: "INVALID_BINARY"}


class ErrorT(C.Structure):
    _fields_ = [("code", C.c_int), ("message", C.c_char * 1024)]


class SearchResult(C.Structure):
    _fields_ = [("dists", C.POINTER(C.c_float)), ("ids", C.POINTER(C.c_int64)), ("count", C.c_int64),
                ("other_result", C.c_void_p)]


FILTER_FUNC = C.CFUNCTYPE(C.c_bool, C.c_int64)


class VsagError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s: %s" % (ERROR_NAMES.get(code, str(code)), message))
        self.code = code
        self.message = message


_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise FileNotFoundError("%s is not built: run `python -m vsag_amd.build`" % HOST_LIB_PATH)
        # the kernels' library first, so that the host library's dependency resolves to the in-tree build
        C.CDLL(os.path.join(_HERE, "lib", "libvsag_amd.so"), mode=C.RTLD_GLOBAL)
        lib = C.CDLL(HOST_LIB_PATH)
        lib.vsag_index_factory.restype = C.c_void_p
        lib.vsag_index_factory.argtypes = [C.c_char_p, C.c_char_p]
        lib.vsag_last_factory_error.restype = ErrorT
        lib.vsag_index_destroy.restype = ErrorT
        lib.vsag_index_destroy.argtypes = [C.c_void_p]
        for name in ("vsag_index_build", "vsag_index_add", "vsag_index_train"):
            fn = getattr(lib, name)
            fn.restype = ErrorT
            fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64]
        lib.vsag_index_knn_search.restype = ErrorT
        lib.vsag_index_knn_search.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64, C.c_char_p,
                                              C.POINTER(SearchResult)]
        lib.vsag_index_knn_search_with_filter.restype = ErrorT
        lib.vsag_index_knn_search_with_filter.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64, C.c_char_p,
                                                          FILTER_FUNC, C.POINTER(SearchResult)]
        lib.vsag_index_range_search.restype = ErrorT
        lib.vsag_index_range_search.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_float, C.c_int64, C.c_char_p,
                                                C.POINTER(SearchResult)]
        lib.vsag_index_range_search_with_filter.restype = ErrorT
        lib.vsag_index_range_search_with_filter.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_float, C.c_int64,
                                                            C.c_char_p, FILTER_FUNC, C.POINTER(SearchResult)]
        lib.vsag_index_knn_search_batch.restype = ErrorT
        lib.vsag_index_knn_search_batch.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_int64,
                                                    C.c_char_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int64)]
        lib.vsag_index_eval_knn_search.restype = ErrorT
        lib.vsag_index_eval_knn_search.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_int64, C.c_char_p,
                                                   C.c_int, C.c_void_p, C.c_void_p, C.POINTER(C.c_double)]
        lib.vsag_index_search_buckets.restype = ErrorT
        lib.vsag_index_search_buckets.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_int64, C.c_char_p,
                                                  C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int64)]
        lib.vsag_index_calculate_distances.restype = ErrorT
        lib.vsag_index_calculate_distances.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_void_p,
                                                       C.c_uint64, C.c_bool, C.c_int64, C.c_void_p, C.c_void_p]
        lib.vsag_index_calculate_distance_by_ids.restype = ErrorT
        lib.vsag_index_calculate_distance_by_ids.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64,
                                                             C.c_void_p]
        lib.vsag_search_result_enable_statistics.restype = ErrorT
        lib.vsag_search_result_enable_statistics.argtypes = [C.POINTER(SearchResult)]
        lib.vsag_search_result_get_statistics.restype = C.c_char_p
        lib.vsag_search_result_get_statistics.argtypes = [C.POINTER(SearchResult)]
        lib.vsag_search_result_destroy_statistics.restype = None
        lib.vsag_search_result_destroy_statistics.argtypes = [C.POINTER(SearchResult)]
        for name in ("vsag_serialize_file", "vsag_deserialize_file"):
            fn = getattr(lib, name)
            fn.restype = ErrorT
            fn.argtypes = [C.c_void_p, C.c_char_p]
        lib.vsag_index_get_num_elements.restype = C.c_int64
        lib.vsag_index_get_num_elements.argtypes = [C.c_void_p]
        lib.vsag_last_failed_id_count.restype = C.c_int64
        _lib = lib
    return _lib


def _check(err):
    if err.code != 0:
        raise VsagError(err.code, err.message.decode("utf-8", "replace"))


class Index:
    def __init__(self, name, parameters):
        lib = _load()
        self._h = lib.vsag_index_factory(name.encode(), parameters.encode())
        if not self._h:
            _check(lib.vsag_last_factory_error())
            raise VsagError(-1, "index creation failed")

    def _insert(self, fn, vectors, ids, num_elements, dim):
        v = np.ascontiguousarray(vectors, np.float32).reshape(-1)
        i = np.ascontiguousarray(ids, np.int64).reshape(-1)
        assert v.size >= num_elements * dim and i.size >= num_elements
        _check(fn(self._h, v.ctypes.data, i.ctypes.data, dim, num_elements))
        return int(_load().vsag_last_failed_id_count())

    def build(self, vectors, ids, num_elements, dim):
        """Returns the number of ids that could not be inserted."""
        return self._insert(_load().vsag_index_build, vectors, ids, num_elements, dim)

    def add(self, vectors, ids, num_elements, dim):
        return self._insert(_load().vsag_index_add, vectors, ids, num_elements, dim)

    def train(self, vectors, ids, num_elements, dim):
        """Trains centroids and quantizers; adds nothing."""
        self._insert(_load().vsag_index_train, vectors, ids, num_elements, dim)

    def knn_search(self, vector, k, parameters, filter=None, statistics=False):
        q = np.ascontiguousarray(vector, np.float32).reshape(-1)
        kk = max(int(k), 1)
        ids = np.empty(kk, np.int64)
        dists = np.empty(kk, np.float32)
        res = SearchResult(dists.ctypes.data_as(C.POINTER(C.c_float)), ids.ctypes.data_as(C.POINTER(C.c_int64)), 0,
                           None)
        lib = _load()
        if statistics:
            _check(lib.vsag_search_result_enable_statistics(C.byref(res)))
        try:
            if filter is None:
                _check(lib.vsag_index_knn_search(self._h, q.ctypes.data, q.size, k, parameters.encode(), C.byref(res)))
            else:
                cb = FILTER_FUNC(lambda label: bool(filter(label)))
                _check(lib.vsag_index_knn_search_with_filter(self._h, q.ctypes.data, q.size, k, parameters.encode(), cb,
                                                             C.byref(res)))
            if statistics:
                text = lib.vsag_search_result_get_statistics(C.byref(res))
                return ids[:res.count].copy(), dists[:res.count].copy(), (text or b"").decode()
        finally:
            if statistics:
                lib.vsag_search_result_destroy_statistics(C.byref(res))
        return ids[:res.count].copy(), dists[:res.count].copy()

    def cal_distance_by_id(self, query, ids, precise=True, topk=-1):
        """Index::CalDistanceById: query (dim,) or (nq, dim); ids (count,) or (nq, count).  topk == -1: the distances
        in the order of ids (-1 for unknown labels); topk > 0: (labels, distances) of the smallest per row."""
        q = np.ascontiguousarray(query, np.float32)
        one = q.ndim == 1
        q = q.reshape(1, -1) if one else q
        i = np.ascontiguousarray(ids, np.int64).reshape(q.shape[0], -1)
        count = i.shape[1]
        cols = count if topk == -1 else min(int(topk), count)
        out_d = np.empty((q.shape[0], max(cols, 0)), np.float32)
        out_i = np.empty((q.shape[0], max(cols, 0)), np.int64)
        _check(_load().vsag_index_calculate_distances(self._h, q.ctypes.data, q.shape[0], q.shape[1], i.ctypes.data,
                                                      count, bool(precise), int(topk), out_i.ctypes.data,
                                                      out_d.ctypes.data))
        if topk == -1:
            return out_d[0] if one else out_d
        return (out_i[0], out_d[0]) if one else (out_i, out_d)

    def range_search(self, point, threshold, parameters, limit=None, filter=None):
        """Everything within `threshold`, nearest first; at most `limit` results (default: every vector)."""
        q = np.ascontiguousarray(point, np.float32).reshape(-1)
        kk = max(int(limit) if limit is not None else self.get_num_elements(), 1)
        ids = np.empty(kk, np.int64)
        dists = np.empty(kk, np.float32)
        res = SearchResult(dists.ctypes.data_as(C.POINTER(C.c_float)), ids.ctypes.data_as(C.POINTER(C.c_int64)), 0,
                           None)
        lim = int(limit) if limit is not None else kk
        if filter is None:
            _check(_load().vsag_index_range_search(self._h, q.ctypes.data, q.size, threshold, lim, parameters.encode(),
                                                   C.byref(res)))
        else:
            cb = FILTER_FUNC(lambda label: bool(filter(label)))
            _check(_load().vsag_index_range_search_with_filter(self._h, q.ctypes.data, q.size, threshold, lim,
                                                               parameters.encode(), cb, C.byref(res)))
        return ids[:res.count].copy(), dists[:res.count].copy()

    def knn_search_batch(self, vectors, k, parameters, bucket_ids=None):
        """bucket_ids: one sequence of list numbers per query (SearchRequest::bucket_ids_): the lists that query scans
        instead of the routed ones."""
        q = np.ascontiguousarray(vectors, np.float32)
        nq, dim = q.shape
        ids = np.empty((nq, k), np.int64)
        dists = np.empty((nq, k), np.float32)
        rdim = C.c_int64()
        if bucket_ids is None:
            _check(_load().vsag_index_knn_search_batch(self._h, q.ctypes.data, nq, dim, k, parameters.encode(),
                                                       ids.ctypes.data, dists.ctypes.data, C.byref(rdim)))
            return ids, dists
        offsets = np.zeros(len(bucket_ids) + 1, np.uint64)
        offsets[1:] = np.cumsum([len(b) for b in bucket_ids])
        if len(bucket_ids) != nq:
            raise VsagError(-3, "bucket_ids_ size must match the number of query vectors")
        flat = np.zeros(max(int(offsets[-1]), 1), np.int64)  # never a null pointer: an empty row is an error to report
        flat[:int(offsets[-1])] = np.concatenate([np.asarray(b, np.int64).reshape(-1) for b in bucket_ids])
        _check(_load().vsag_index_search_buckets(self._h, q.ctypes.data, nq, dim, k, parameters.encode(),
                                                 flat.ctypes.data, offsets.ctypes.data,
                                                 ids.ctypes.data, dists.ctypes.data, C.byref(rdim)))
        return ids, dists

    def eval_knn_search(self, vectors, k, parameters, threads):
        """The reference evaluator's loop (tools/eval/case/search_eval_case.cpp:233-277): one query per KnnSearch call
        from `threads` caller threads on this index.  Returns (ids, distances, wall seconds of the loop)."""
        q = np.ascontiguousarray(vectors, np.float32)
        nq, dim = q.shape
        ids = np.empty((nq, k), np.int64)
        dists = np.empty((nq, k), np.float32)
        seconds = C.c_double()
        _check(_load().vsag_index_eval_knn_search(self._h, q.ctypes.data, nq, dim, k, parameters.encode(), int(threads),
                                                  ids.ctypes.data, dists.ctypes.data, C.byref(seconds)))
        return ids, dists, seconds.value

    def serialize(self, path):
        """The index as one file in the reference's stream layout (cells of codes, quantizer state, labels, footer)."""
        _check(_load().vsag_serialize_file(self._h, str(path).encode()))

    def deserialize(self, path):
        """Loads a file written by serialize() (or by the reference) into this empty index."""
        _check(_load().vsag_deserialize_file(self._h, str(path).encode()))

    def get_num_elements(self):
        return int(_load().vsag_index_get_num_elements(self._h))

    def close(self):
        if self._h:
            _load().vsag_index_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
