"""ctypes binding of the C ABI declared in include/vsag_amd.h (libvsag_amd.so).

Only plumbing lives here: loading the library, argument types, a device-buffer helper built on the
library's own malloc / memcpy entry points.  There is no computation and no fallback: if the library is
missing or no gfx950 device is usable, calls raise.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libvsag_amd.so")

SUCCESS = 0
INVALID_ARGUMENT = -3
METRIC_L2, METRIC_IP, METRIC_COSINE = 0, 1, 2
KIND_FP32, KIND_SQ8, KIND_SQ4, KIND_SQ4_UNIFORM, KIND_SQ8_UNIFORM, KIND_RABITQ, KIND_PQFS = range(7)
SQ_TRAIN_CLASSIC, SQ_TRAIN_TRUNC_BOUND = 1, 3
INVALID_ID = 0xFFFFFFFF

METRICS = {"l2": METRIC_L2, "ip": METRIC_IP, "cosine": METRIC_COSINE}
KINDS = {"fp32": KIND_FP32, "sq8": KIND_SQ8, "sq4": KIND_SQ4, "sq4_uniform": KIND_SQ4_UNIFORM,
         "sq8_uniform": KIND_SQ8_UNIFORM, "rabitq": KIND_RABITQ, "pqfs": KIND_PQFS}


class VsagAmdError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("vsag_amd error %d: %s" % (code, message))
        self.code = code


class StoreParams(C.Structure):
    _fields_ = [("kind", C.c_int), ("metric", C.c_int), ("dim", C.c_uint32),
                ("lower_bound_dev", C.c_void_p), ("diff_dev", C.c_void_p), ("rotation_dev", C.c_void_p),
                ("centroid_dev", C.c_void_p), ("rabitq_query_bits", C.c_int), ("pq_dim", C.c_uint32),
                ("codebooks_dev", C.c_void_p)]


class SearchOptions(C.Structure):
    _fields_ = [("deny_bits_dev", C.c_void_p), ("use_radius", C.c_int), ("radius", C.c_float)]


_u64, _u32, _i32, _sz, _vp, _f32 = C.c_uint64, C.c_uint32, C.c_int, C.c_size_t, C.c_void_p, C.c_float

# name -> (restype, argtypes); the list is also what the export test checks against the header.
PROTOTYPES = {
    "vsag_amd_init": (C.c_int, [C.c_int]),
    "vsag_amd_last_error": (C.c_char_p, []),
    "vsag_amd_device_info": (C.c_int, [C.c_char_p, _sz, C.POINTER(C.c_int), C.POINTER(_u64)]),
    "vsag_amd_malloc": (C.c_int, [C.POINTER(_vp), _sz]),
    "vsag_amd_free": (C.c_int, [_vp]),
    "vsag_amd_memcpy_h2d": (C.c_int, [_vp, _vp, _sz, _vp]),
    "vsag_amd_memcpy_d2h": (C.c_int, [_vp, _vp, _sz, _vp]),
    "vsag_amd_memcpy_d2d": (C.c_int, [_vp, _vp, _sz, _vp]),
    "vsag_amd_host_malloc": (C.c_int, [C.POINTER(_vp), _sz]),
    "vsag_amd_host_free": (C.c_int, [_vp]),
    "vsag_amd_memcpy_h2d_async": (C.c_int, [_vp, _vp, _sz, _vp]),
    "vsag_amd_memcpy_d2h_async": (C.c_int, [_vp, _vp, _sz, _vp]),
    "vsag_amd_memset": (C.c_int, [_vp, C.c_int, _sz, _vp]),
    "vsag_amd_memory_info": (C.c_int, [_vp, _vp, _vp, C.c_int]),
    "vsag_amd_stream_synchronize": (C.c_int, [_vp]),
    "vsag_amd_stream_create": (C.c_int, [C.POINTER(_vp)]),
    "vsag_amd_stream_destroy": (C.c_int, [_vp]),
    "vsag_amd_sq_train_workspace_bytes": (_sz, [_u64, _u32, _u64]),
    "vsag_amd_sq_train": (C.c_int, [_vp, _u64, _u32, _i32, _i32, _i32, _f32, _u64, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_sq_train_uniform": (C.c_int, [_vp, _u64, _u32, _i32, _i32, _i32, _f32, _u64, _vp, _vp, _sz, _vp]),
    "vsag_amd_code_size": (_u64, [_i32, _i32, _u32, _i32]),
    "vsag_amd_sq_encode": (C.c_int, [_vp, _u64, _u32, _i32, _i32, _vp, _vp, _vp, _vp]),
    "vsag_amd_squ_encode": (C.c_int, [_vp, _u64, _u32, _i32, _i32, _vp, _vp, _vp]),
    "vsag_amd_rabitq_train": (C.c_int, [_vp, _u64, _u32, _vp, _vp, _vp]),
    "vsag_amd_rabitq_encode": (C.c_int, [_vp, _u64, _u32, _vp, _vp, _i32, _i32, _vp, _vp]),
    "vsag_amd_fht_kac_matrix": (C.c_int, [_vp, _u32, _vp]),
    "vsag_amd_rabitq_decode": (C.c_int, [_vp, _u64, _u32, _vp, _vp, _i32, _i32, _vp, _vp]),
    "vsag_amd_rabitq_encode_multibit": (C.c_int, [_vp, _u64, _u32, _vp, _vp, _i32, _i32, _i32, _u32, _vp, _vp]),
    "vsag_amd_rabitq_query_code_size": (_u64, [_u32, _i32, _i32]),
    "vsag_amd_rabitq_process_query": (C.c_int, [_vp, _u64, _u32, _vp, _vp, _i32, _i32, _vp, _vp]),
    "vsag_amd_pq_train_workspace_bytes": (_sz, [_u64, _u32, _u32]),
    "vsag_amd_pq_train": (C.c_int, [_vp, _u64, _u32, _u32, _i32, _u64, _vp, _vp, _sz, _vp]),
    "vsag_amd_pq_encode": (C.c_int, [_vp, _u64, _u32, _u32, _vp, _i32, _vp, _vp, _vp]),
    "vsag_amd_pq_decode": (C.c_int, [_vp, _u64, _u32, _u32, _vp, _vp, _vp]),
    "vsag_amd_pqfs_process_query": (C.c_int, [_vp, _u64, _u32, _u32, _vp, _i32, _vp, _vp]),
    "vsag_amd_pqfs_package": (C.c_int, [_vp, _u64, _u32, _vp, _vp]),
    "vsag_amd_pqfs_unpack": (C.c_int, [_vp, _u64, _u32, _vp, _vp]),
    "vsag_amd_store_create": (C.c_int, [C.POINTER(StoreParams), C.POINTER(_vp)]),
    "vsag_amd_store_destroy": (C.c_int, [_vp]),
    "vsag_amd_store_size": (_u64, [_vp]),
    "vsag_amd_store_append": (C.c_int, [_vp, _vp, _u64, _vp]),
    "vsag_amd_store_set_lists": (C.c_int, [_vp, _vp, _vp, _u64, _u32, _vp]),
    "vsag_amd_store_append_lists": (C.c_int, [_vp, _vp, _vp, _vp, _u64, _vp]),
    "vsag_amd_store_set_residual": (C.c_int, [_vp, _vp, _u32, _vp]),
    "vsag_amd_residual_rows": (C.c_int, [_vp, _u64, _u32, _i32, _vp, _vp, _vp, _vp]),
    "vsag_amd_residual_bias": (C.c_int, [_vp, _vp, _u64, _vp, _vp, _vp, _vp, _vp]),
    "vsag_amd_store_list_sizes": (C.c_int, [_vp, _vp, _u32]),
    "vsag_amd_store_distances_workspace_bytes": (_sz, [_vp, _u64]),
    "vsag_amd_store_distances": (C.c_int, [_vp, _vp, _u64, _vp, _u32, _vp, _vp, _sz, _vp]),
    "vsag_amd_flat_scan_workspace_bytes": (_sz, [_vp, _u64, _u32]),
    "vsag_amd_flat_scan_topk": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_flat_scan_topk_ex": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_flat_scan_noalloc_max_bytes": (_sz, []),
    "vsag_amd_flat_scan_topk_noalloc": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _vp, _vp, _vp]),
    "vsag_amd_set_scan_tuning": (C.c_int, [_i32, _i32]),
    "vsag_amd_set_scan_contraction": (C.c_int, [_i32]),
    "vsag_amd_store_set_scan_contraction": (C.c_int, [_vp, _i32]),
    "vsag_amd_store_set_scan_tuning": (C.c_int, [_vp, _i32, _i32]),
    "vsag_amd_last_scan_info": (C.c_int, [C.POINTER(C.c_int), C.POINTER(_u64), C.POINTER(_u64)]),
    "vsag_amd_set_kernel_timing": (C.c_int, [_i32]),
    "vsag_amd_last_kernel_ms": (C.c_int, [C.POINTER(_f32)]),
    "vsag_amd_kmeans_assign_workspace_bytes": (_sz, [_u64, _u32, _u32]),
    "vsag_amd_kmeans_assign": (C.c_int, [_vp, _u64, _u32, _vp, _u32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_kmeans_update_workspace_bytes": (_sz, [_u64, _u32, _u32]),
    "vsag_amd_kmeans_update": (C.c_int, [_vp, _vp, _u64, _u32, _u32, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_kmeans_init_plus_plus_workspace_bytes": (_sz, [_u64]),
    "vsag_amd_kmeans_init_plus_plus": (C.c_int, [_vp, _u64, _u32, _u32, _u64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_kmeans_run_workspace_bytes": (_sz, [_u64, _u32, _u32]),
    "vsag_amd_kmeans_run": (C.c_int, [_vp, _u64, _u32, _vp, _u32, _i32, _u64, _vp, C.POINTER(C.c_double), _vp, _sz,
                                      _vp]),
    "vsag_amd_ivf_route_workspace_bytes": (_sz, [_vp, _u64, _u32]),
    "vsag_amd_ivf_route": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_ivf_scan_workspace_bytes": (_sz, [_vp, _u64, _u32, _u32]),
    "vsag_amd_ivf_scan_topk": (C.c_int, [_vp, _vp, _u64, _vp, _u32, _u32, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_ivf_scan_topk_ex": (C.c_int, [_vp, _vp, _u64, _vp, _u32, _u32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "vsag_amd_ivf_probed_codes": (C.c_int, [_vp, _vp, _u64, _u32, _vp, _vp]),
    "vsag_amd_rerank_fp32": (C.c_int, [_vp, _u64, _u32, _i32, _vp, _u64, _vp, _u32, _u32, _vp, _vp, _vp]),
    "vsag_amd_store_expect_stored_codes": (C.c_int, [_vp, C.c_int]),
    "vsag_amd_store_export_codes": (C.c_int, [_vp, _u64, _u64, _vp, _vp]),
    "vsag_amd_store_export_lists": (C.c_int, [_vp, _vp, _vp, _vp, _vp]),
    "vsag_amd_rows_distances_fp32": (C.c_int, [_vp, _u64, _u32, _i32, _vp, _u64, _vp, _u32, _vp, _vp]),
}

_lib = None


def load_library():
    """Loads libvsag_amd.so (no device is touched yet) and sets the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s is not built: run `python -m vsag_amd.build` (there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise VsagAmdError(rc, load_library().vsag_amd_last_error().decode("utf-8", "replace"))


def init(device=0):
    check(load_library().vsag_amd_init(device))


def device_info():
    name = C.create_string_buffer(256)
    cus = C.c_int()
    mem = C.c_uint64()
    check(load_library().vsag_amd_device_info(name, 256, C.byref(cus), C.byref(mem)))
    return name.value.decode(), cus.value, mem.value


class DeviceBuffer:
    """Device allocation owned through vsag_amd_malloc / vsag_amd_free."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(load_library().vsag_amd_malloc(C.byref(p), max(self.nbytes, 1)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr, stream=None):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        if arr.nbytes:
            check(load_library().vsag_amd_memcpy_h2d(buf.ptr, arr.ctypes.data, arr.nbytes, stream))
        return buf

    def to_numpy(self, dtype, shape, stream=None, offset=0):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes:
            check(load_library().vsag_amd_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes, stream))
        return out

    def free(self):
        if self.ptr is not None:
            load_library().vsag_amd_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def synchronize(stream=None):
    check(load_library().vsag_amd_stream_synchronize(stream))
