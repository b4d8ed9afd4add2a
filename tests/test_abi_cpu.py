"""The C-ABI library loads without a GPU, exports every symbol include/vsag_amd.h declares (and nothing the
binding does not know), and fails loudly instead of falling back when no device is usable."""
import os
import re
import subprocess

import pytest

from vsag_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "vsag_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(vsag_amd_[a-z0-9_]+)\s*\(", text))


def exported_functions():
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], check=True, stdout=subprocess.PIPE,
                         text=True).stdout
    return set(line.split()[-1] for line in out.splitlines() if " T " in line and "vsag_amd_" in line)


def test_header_symbols_are_exported_and_bound():
    declared = declared_functions()
    assert len(declared) > 30
    exported = exported_functions()
    assert declared <= exported, "declared but not exported: %s" % sorted(declared - exported)
    assert exported <= declared, "exported but not declared: %s" % sorted(exported - declared)
    assert set(capi.PROTOTYPES) == declared, sorted(set(capi.PROTOTYPES) ^ declared)


def test_library_loads_and_every_declared_symbol_resolves():
    lib = capi.load_library()
    for name in declared_functions():
        assert getattr(lib, name) is not None


def test_error_codes_match_the_reference_c_api():
    # include/vsag/vsag_c_api.h:20-34 of the reference
    text = open(HEADER).read()
    for name, value in [("SUCCESS", 0), ("UNKNOWN_ERROR", -1), ("INTERNAL_ERROR", -2), ("INVALID_ARGUMENT", -3),
                        ("WRONG_STATUS", -4), ("UNSUPPORTED_INDEX_OPERATION", -8), ("DIMENSION_NOT_EQUAL", -9),
                        ("INDEX_EMPTY", -10), ("NO_ENOUGH_MEMORY", -11)]:
        m = re.search(r"#define VSAG_AMD_%s \(?(-?\d+)\)?" % name, text)
        assert m and int(m.group(1)) == value, name


def test_code_sizes_need_no_device():
    lib = capi.load_library()
    assert lib.vsag_amd_code_size(capi.KIND_SQ8, capi.METRIC_L2, 128, 0) == 128
    assert lib.vsag_amd_code_size(capi.KIND_SQ4, capi.METRIC_L2, 33, 0) == 17
    assert lib.vsag_amd_code_size(capi.KIND_FP32, capi.METRIC_IP, 960, 0) == 3840
    assert lib.vsag_amd_code_size(capi.KIND_SQ4_UNIFORM, capi.METRIC_L2, 128, 0) == 72
    assert lib.vsag_amd_code_size(capi.KIND_SQ4_UNIFORM, capi.METRIC_IP, 6, 0) == 12
    assert lib.vsag_amd_code_size(capi.KIND_SQ8_UNIFORM, capi.METRIC_L2, 128, 0) == 136
    assert lib.vsag_amd_code_size(capi.KIND_RABITQ, capi.METRIC_IP, 768, 4) == 112
    assert lib.vsag_amd_rabitq_query_code_size(768, capi.METRIC_IP, 4) == 532


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present: the no-device path cannot be shown")
def test_no_device_is_a_loud_error_not_a_fallback():
    lib = capi.load_library()
    assert lib.vsag_amd_init(0) == -2
    assert b"no CPU fallback" in lib.vsag_amd_last_error()
    with pytest.raises(capi.VsagAmdError):
        capi.init(0)
    # compute entry points refuse as well
    assert lib.vsag_amd_kmeans_assign(None, 1, 1, None, 1, None, None, None, None, 0, None) == -2


@pytest.mark.parametrize("d", [1, 2, 7, 8, 33, 64, 100, 128, 200, 256])
def test_fht_rotator_matrix_is_the_rotator(d):
    """vsag_amd_fht_kac_matrix (host work only): the matrix times a vector equals FhtKacRotator::Transform
    (fht_kac_rotate_transformer.cpp:64-96) of that vector as the checker restates it, and R^T undoes it
    (InverseTransform, :97-120)."""
    import ctypes as C

    import numpy as np

    import oracle as orc
    lib = capi.load_library()
    rng = np.random.default_rng(500 + d)
    flip = rng.integers(0, 256, 4 * ((d + 7) // 8)).astype(np.uint8)
    rot = np.empty((d, d), np.float32)
    capi.check(lib.vsag_amd_fht_kac_matrix(flip.ctypes.data_as(C.c_void_p), d, rot.ctypes.data_as(C.c_void_p)))
    x = rng.standard_normal((5, d)).astype(np.float32)
    want = orc.fht_kac_transform(flip, x)
    tol = 4e-6 * np.sqrt(d) * (1 + np.abs(x).max())
    np.testing.assert_allclose(x.astype(np.float64) @ rot.astype(np.float64).T, want, rtol=0, atol=tol)
    np.testing.assert_allclose(want.astype(np.float64) @ rot.astype(np.float64), orc.fht_kac_transform(flip, want, inverse=True),
                               rtol=0, atol=tol)
    # the images of the basis vectors, entry for entry
    cols = orc.fht_kac_transform(flip, np.eye(d, dtype=np.float32))
    np.testing.assert_allclose(rot.T, cols, rtol=0, atol=1e-6)
