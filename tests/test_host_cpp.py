"""The host layer driven from C++ (tests/cpp/host_api.cpp, built by `python -m vsag_amd.build` into
vsag_amd/lib/host_api_test): Factory::CreateIndex with an Allocator (include/vsag/factory.h:47-50), Build, KnnSearch,
CalDistanceById, Serialize / Deserialize through std::iostream, error types."""
import os
import subprocess

import pytest

EXE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "vsag_amd", "lib", "host_api_test")


def _run():
    assert os.path.exists(EXE), "build first: python -m vsag_amd.build"
    return subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)


def test_without_a_gpu_the_factory_fails_loudly():
    import ctypes
    try:
        hip = ctypes.CDLL("libamdhip64.so")
        count = ctypes.c_int(0)
        if hip.hipGetDeviceCount(ctypes.byref(count)) == 0 and count.value > 0:
            pytest.skip("a GPU is present")
    except OSError:
        pass
    proc = _run()
    assert proc.returncode == 100, proc.stdout
    assert "no CPU fallback" in proc.stdout


@pytest.mark.gpu
def test_cpp_consumer_of_the_host_api():
    proc = _run()
    assert proc.returncode == 0 and "all checks passed" in proc.stdout, proc.stdout
    assert "FAIL" not in proc.stdout
