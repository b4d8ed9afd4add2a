"""Parameter contract and error conventions of Factory::CreateIndex, checked without a GPU (the constructors
validate before the device is touched).  Mirrors the reference's parameter tests: unknown index_param keys are
"invalid config param: <key>" (src/utils/util_functions.cpp:45-66), missing dtype / metric_type / dim are
INVALID_ARGUMENT (src/index_common_param.cpp:117-174), unknown index names are UNSUPPORTED_INDEX."""
import json
import os

import pytest

from vsag_amd import pyvsag

BASE = {"dtype": "float32", "metric_type": "l2", "dim": 16}


def create(name, params):
    return pyvsag.Index(name, params if isinstance(params, str) else json.dumps(params))


@pytest.mark.parametrize("name", ["brute_force", "ivf"])
def test_invalid_json_and_missing_common_keys(name):
    with pytest.raises(pyvsag.VsagError) as e:
        create(name, "{not json")
    assert e.value.code == -3
    for missing in ("dtype", "metric_type", "dim"):
        p = dict(BASE)
        del p[missing]
        with pytest.raises(pyvsag.VsagError) as e:
            create(name, p)
        assert e.value.code == -3 and missing in e.value.message
    with pytest.raises(pyvsag.VsagError) as e:
        create(name, dict(BASE, metric_type="hamming"))
    assert e.value.code == -3 and "metric_type" in e.value.message
    with pytest.raises(pyvsag.VsagError) as e:
        create(name, dict(BASE, dtype="int8"))
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        create(name, dict(BASE, dim=0))
    assert e.value.code == -3


@pytest.mark.parametrize("name", ["brute_force", "ivf"])
def test_unknown_index_param_key_is_rejected(name):
    with pytest.raises(pyvsag.VsagError) as e:
        create(name, dict(BASE, index_param={"no_such_key": 1}))
    assert e.value.code == -3 and e.value.message == "invalid config param: no_such_key"


def test_unsupported_index_and_quantizer():
    with pytest.raises(pyvsag.VsagError) as e:
        create("hnsw_on_gpu", BASE)
    assert e.value.code == -7
    with pytest.raises(pyvsag.VsagError) as e:
        create("brute_force", dict(BASE, index_param={"base_quantization_type": "pq"}))
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        create("ivf", dict(BASE, index_param={"buckets_count": 0}))
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        create("ivf", dict(BASE, index_param={"train_sample_count": 100}))
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        create("ivf", dict(BASE, index_param={"ivf_train_type": "spectral"}))
    assert e.value.code == -3


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_valid_parameters_without_a_gpu_fail_loudly():
    with pytest.raises(pyvsag.VsagError) as e:
        create("brute_force", dict(BASE, index_param={"base_quantization_type": "sq8"}))
    assert e.value.code == -2 and "no CPU fallback" in e.value.message
