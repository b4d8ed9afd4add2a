"""brute_force / ivf through the kept API (CreateIndex -> Build -> KnnSearch with the reference's JSON), modelled on
the reference's functional tests: recall floors (tests/test_ivf.cpp:94-102 with RECALL_THRESHOLD 0.85,
tests/test_index.h:373), result shape (tests/test_index/test_index_search.cpp:60-99), batch == serial
(tests/test_ivf.cpp:3283-3341), exact self-distance after fp32 reorder (tests/test_ivf.cpp:340-367), error paths."""
import ctypes as C
import json

import numpy as np
import pytest

import oracle as orc
from vsag_amd import capi, pyvsag

pytestmark = pytest.mark.gpu
RECALL_THRESHOLD = 0.85


def vectors(count, dim, seed=47, normalize=True):
    """generate_vectors of the reference fixtures (tests/fixtures/data/vector_generator.cpp:121-124)."""
    rng = np.random.Generator(np.random.MT19937(seed))
    x = rng.uniform(0.1, 0.9, (count, dim)).astype(np.float32)
    if normalize:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    return x


def ground_truth(x, q, k, metric):
    x64, q64 = x.astype(np.float64), q.astype(np.float64)
    if metric == "l2":
        d = ((q64[:, None, :] - x64[None]) ** 2).sum(2)
    elif metric == "ip":
        d = 1 - q64 @ x64.T
    else:
        d = 1 - (q64 / np.linalg.norm(q64, axis=1, keepdims=True)) @ (x64 / np.linalg.norm(x64, axis=1, keepdims=True)).T
    idx = np.argsort(d, 1, kind="stable")[:, :k]
    return idx, np.take_along_axis(d, idx, 1)


def recall(ids, gt_ids, labels):
    hit = sum(len(set(a.tolist()) & set(labels[b].tolist())) for a, b in zip(ids, gt_ids))
    return hit / float(gt_ids.size)


def make(name, dim, metric, **index_param):
    return pyvsag.Index(name, json.dumps({"dtype": "float32", "metric_type": metric, "dim": dim,
                                         "index_param": index_param}))


@pytest.mark.parametrize("name,d", [("ivf", 128), ("ivf", 100), ("brute_force", 96)])
def test_rabitq_with_the_fht_rotator(lib, tmp_path, name, d):
    """rabitq_use_fht (rabitq_quantizer.cpp:81-86): FhtKacRotator's rotation instead of the random orthogonal matrix,
    for a power-of-two dimension and for others (the Kac walk branch).  An orthogonal map either way: the recall floor of
    tests/test_ivf.cpp:1212-1230 holds; the file carries the rotator's sign bits (FhtKacRotator::Serialize) and
    use_fht in its parameters, loads to the same answers, and is refused by an index built without the flag."""
    n, nq, k = 3000, 50, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64)
    params = dict(base_quantization_type="rabitq")
    if name == "ivf":
        params.update(buckets_count=10, train_sample_count=3000, use_reorder=True, precise_quantization_type="fp32")
    search = json.dumps({"ivf": {"scan_buckets_count": 10, "factor": 20.0}}) if name == "ivf" else "{}"
    idx = make(name, d, "l2", rabitq_use_fht=True, **params)
    idx.build(x, labels, n, d)
    gt, _ = ground_truth(x, q, k, "l2")
    ids, dists = idx.knn_search_batch(q, k, search)
    path = tmp_path / "fht.index"
    idx.serialize(path)
    plain = make(name, d, "l2", **params)
    plain.build(x, labels, n, d)
    if name == "ivf":
        assert recall(ids, gt, labels) >= 0.85
    else:
        # no rerank here: the 1-bit estimate alone, as good with one rotation as with the other
        assert abs(recall(ids, gt, labels) - recall(plain.knn_search_batch(q, k, search)[0], gt, labels)) <= 0.08
    plain_path = tmp_path / "plain.index"
    plain.serialize(plain_path)
    rot_bytes = d * d * 4 - 4 * ((d + 7) // 8)
    assert plain_path.stat().st_size - path.stat().st_size >= rot_bytes - 64  # sign bits instead of the matrix
    assert b'\\"use_fht\\":true' in path.read_bytes() or b'"use_fht":true' in path.read_bytes()
    again = make(name, d, "l2", rabitq_use_fht=True, **params)
    again.deserialize(path)
    ids2, dists2 = again.knn_search_batch(q, k, search)
    assert np.array_equal(ids, ids2) and np.array_equal(dists, dists2)
    other = make(name, d, "l2", **params)
    with pytest.raises(pyvsag.VsagError):
        other.deserialize(path)
    for i in (idx, plain, again, other):
        i.close()


@pytest.mark.parametrize("metric", ["l2", "ip", "cosine"])
@pytest.mark.parametrize("quant,floor", [("fp32", 0.99), ("sq8", 0.84), ("sq4_uniform", 0.5), ("sq8_uniform", 0.84)])
def test_brute_force_build_and_search(lib, metric, quant, floor):
    n, d, nq, k = 2000, 64, 50, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) * 3 + 7
    idx = make("brute_force", d, metric, base_quantization_type=quant)
    assert idx.build(x, labels, n, d) == 0
    assert idx.get_num_elements() == n
    gt, gt_d = ground_truth(x, q, k, metric)
    ids, dists = idx.knn_search_batch(q, k, "{}")
    assert ids.shape == (nq, k)
    assert recall(ids, gt, labels) >= floor * RECALL_THRESHOLD
    assert np.all(np.diff(dists, axis=1) >= 0)
    # one query per call, as the reference's KnnSearch is used: same result as the batch row
    for i in range(5):
        sid, sd = idx.knn_search(q[i], k, "{}")
        assert sid.shape == (k,) and np.array_equal(sid, ids[i]) and np.array_equal(sd, dists[i])
    if quant == "fp32":
        assert np.allclose(dists, gt_d, rtol=1e-4, atol=2e-6)
        assert recall(ids, gt, labels) == 1.0
    idx.close()


def test_brute_force_conventions(lib):
    d = 16
    idx = make("brute_force", d, "l2")
    # empty index -> empty result, not an error
    ids, dists = idx.knn_search(np.zeros(d, np.float32), 5, "{}")
    assert ids.size == 0
    x = vectors(7, d)
    labels = np.array([10, 11, 12, 13, 14, 15, 10], np.int64)  # one duplicate id
    assert idx.build(x, labels, 7, d) == 1
    assert idx.get_num_elements() == 6
    # fewer results than k -> short result
    ids, dists = idx.knn_search(x[2], 20, "{}")
    assert ids.size == 6 and ids[0] == 12 and dists[0] <= 2e-6
    # adding more, duplicates are reported
    assert idx.add(vectors(3, d, seed=5), np.array([15, 16, 17], np.int64), 3, d) == 1
    assert idx.get_num_elements() == 8
    with pytest.raises(pyvsag.VsagError) as e:
        idx.build(x, labels, 7, d)
    assert e.value.code == -5  # BUILD_TWICE
    with pytest.raises(pyvsag.VsagError) as e:
        idx.knn_search(np.zeros(d + 1, np.float32), 5, "{}")
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        idx.knn_search(np.zeros(d, np.float32), 0, "{}")
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        idx.knn_search(np.zeros(d, np.float32), 3, "{bad")
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        idx.add(vectors(2, d + 2), np.array([100, 101], np.int64), 2, d + 2)
    assert e.value.code == -3
    idx.close()


IVF_SEARCH = json.dumps({"ivf": {"scan_buckets_count": 30}})


@pytest.mark.parametrize("metric", ["l2", "ip", "cosine"])
@pytest.mark.parametrize("quant,reorder,floor", [("fp32", False, 0.90), ("sq8", False, 0.84),
                                                 ("sq8_uniform", True, 0.89), ("sq4_uniform", True, 0.80)])
def test_ivf_recall_floors(lib, metric, quant, reorder, floor):
    n, d, nq, k = 2400, 64, 100, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) + 1000
    params = {"buckets_count": 50, "base_quantization_type": quant, "train_sample_count": 2400}
    if reorder:
        params.update(use_reorder=True, precise_quantization_type="fp32")
    idx = make("ivf", d, metric, **params)
    assert idx.build(x, labels, n, d) == 0
    gt, _ = ground_truth(x, q, k, metric)
    search = json.dumps({"ivf": {"scan_buckets_count": 30, "factor": 4.0}})
    ids, dists = idx.knn_search_batch(q, k, search)
    r = recall(ids, gt, labels)
    assert r >= floor * RECALL_THRESHOLD, r
    assert np.all(np.diff(dists, axis=1) >= 0)
    # batch == serial, bit for bit
    for i in range(8):
        sid, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(sid, ids[i]) and np.array_equal(sd, dists[i])
    idx.close()


def test_ivf_self_query_is_exact_after_fp32_reorder(lib):
    n, d = 2000, 32
    x = vectors(n, d)
    labels = np.arange(n, dtype=np.int64)
    idx = make("ivf", d, "l2", buckets_count=20, base_quantization_type="sq8", use_reorder=True,
               precise_quantization_type="fp32", train_sample_count=2000)
    idx.build(x, labels, n, d)
    search = json.dumps({"ivf": {"scan_buckets_count": 20, "factor": 5.0}})
    ids, dists = idx.knn_search_batch(x[:200], 1, search)
    assert np.array_equal(ids[:, 0], labels[:200])
    assert np.all(np.abs(dists[:, 0]) < 2e-6)
    idx.close()


def test_ivf_probing_every_bucket_equals_brute_force(lib):
    n, d, nq, k = 3000, 48, 40, 10
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64)
    bf = make("brute_force", d, "l2", base_quantization_type="fp32")
    bf.build(x, labels, n, d)
    ivf = make("ivf", d, "l2", buckets_count=64, base_quantization_type="fp32", train_sample_count=3000)
    ivf.build(x, labels, n, d)
    a_ids, a_d = bf.knn_search_batch(q, k, "{}")
    b_ids, b_d = ivf.knn_search_batch(q, k, json.dumps({"ivf": {"scan_buckets_count": 1000}}))
    assert np.array_equal(a_ids, b_ids) and np.array_equal(a_d, b_d)
    # incremental add keeps the lists consistent
    x2 = vectors(500, d, seed=9, normalize=False)
    l2 = np.arange(500, dtype=np.int64) + n
    assert bf.add(x2, l2, 500, d) == 0 and ivf.add(x2, l2, 500, d) == 0
    a_ids, a_d = bf.knn_search_batch(q, k, "{}")
    b_ids, b_d = ivf.knn_search_batch(q, k, json.dumps({"ivf": {"scan_buckets_count": 64}}))
    assert np.array_equal(a_ids, b_ids) and np.array_equal(a_d, b_d)
    bf.close()
    ivf.close()


def test_ivf_routing_only_and_errors(lib):
    n, d = 1500, 24
    x = vectors(n, d)
    idx = make("ivf", d, "l2", buckets_count=16, train_sample_count=1500)
    idx.build(x, np.arange(n, dtype=np.int64), n, d)
    ids, dists = idx.knn_search(x[0], 4, json.dumps({"ivf": {"scan_buckets_count": 4, "disable_bucket_scan": True}}))
    assert ids.size == 4 and np.all((ids >= 0) & (ids < 16)) and np.all(np.diff(dists) >= 0)
    with pytest.raises(pyvsag.VsagError) as e:
        idx.knn_search(x[0], 4, "{}")
    assert e.value.code == -3 and "ivf" in e.value.message
    with pytest.raises(pyvsag.VsagError) as e:
        idx.knn_search(x[0], 4, json.dumps({"ivf": {"factor": 2.0}}))
    assert e.value.code == -3 and "scan_buckets_count" in e.value.message
    small = make("ivf", d, "l2", buckets_count=64, train_sample_count=512)
    with pytest.raises(pyvsag.VsagError) as e:
        small.build(x[:10], np.arange(10, dtype=np.int64), 10, d)
    assert e.value.code == -3 and "k cannot be larger than count" in e.value.message
    idx.close()
    small.close()


@pytest.mark.parametrize("query_bits", [4, 32, None])  # None: the reference's default, fp32 queries
def test_ivf_rabitq_with_reorder(lib, query_bits):
    # tests/test_ivf.cpp:1212-1230: rabitq base codes, fp32 reorder
    n, d, nq, k = 3000, 128, 50, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64)
    extra = {} if query_bits is None else {"rabitq_bits_per_dim_query": query_bits}
    idx = make("ivf", d, "l2", buckets_count=10, base_quantization_type="rabitq",
               use_reorder=True, precise_quantization_type="fp32", train_sample_count=3000, **extra)
    idx.build(x, labels, n, d)
    gt, _ = ground_truth(x, q, k, "l2")
    ids, _ = idx.knn_search_batch(q, k, json.dumps({"ivf": {"scan_buckets_count": 10, "factor": 20.0}}))
    assert recall(ids, gt, labels) >= 0.85
    idx.close()


@pytest.mark.parametrize("metric", ["l2", "ip", "cosine"])
@pytest.mark.parametrize("bits,fast,floor", [(2, True, 0.55), (4, True, 0.85), (8, True, 0.97), (4, False, 0.85)])
def test_ivf_rabitq_multibit_base_codes(lib, tmp_path, metric, bits, fast, floor):
    """rabitq_bits_per_dim_base 2..8 (rabitq_quantizer.cpp:774-809,1799-1808) WITHOUT reorder: the recall of the code
    itself rises with the bits, and 8 bits all but equal the exact search.  Single queries, batches and a reloaded
    index agree."""
    n, d, nq, k = 3000, 64, 40, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) + 7
    idx = make("ivf", d, metric, buckets_count=10, base_quantization_type="rabitq", rabitq_bits_per_dim_base=bits,
               fast_encode_rabitq=fast, train_sample_count=3000)
    idx.build(x, labels, n, d)
    gt, _ = ground_truth(x, q, k, metric)
    search = json.dumps({"ivf": {"scan_buckets_count": 10}})
    ids, dists = idx.knn_search_batch(q, k, search)
    r = recall(ids, gt, labels)
    assert r >= floor, r
    one_bit = make("ivf", d, metric, buckets_count=10, base_quantization_type="rabitq", train_sample_count=3000)
    one_bit.build(x, labels, n, d)
    ids1, _ = one_bit.knn_search_batch(q, k, search)
    assert r > recall(ids1, gt, labels)
    one_bit.close()
    for i in range(5):
        sid, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(sid, ids[i]) and np.allclose(sd, dists[i], rtol=1e-5, atol=1e-6)
    path = tmp_path / "multibit.index"
    idx.serialize(path)
    again = make("ivf", d, metric, buckets_count=10, base_quantization_type="rabitq", rabitq_bits_per_dim_base=bits,
                 fast_encode_rabitq=fast, train_sample_count=3000)
    again.deserialize(path)
    ids2, dists2 = again.knn_search_batch(q, k, search)
    assert np.array_equal(ids2, ids) and np.array_equal(dists2, dists)
    again.close()
    idx.close()


def test_rabitq_multibit_parameters(lib):
    """RaBitQuantizerParameter::FromJson (rabitq_quantizer_parameter.cpp:30-112) and the constructor
    (rabitq_quantizer.cpp:67-100): the reference's ranges and messages."""
    d = 32
    for extra, text in (({"rabitq_bits_per_dim_base": 0}, "rabitq_bits_per_dim_base in [1, 8], but got 0"),
                        ({"rabitq_bits_per_dim_base": 9}, "rabitq_bits_per_dim_base in [1, 8], but got 9"),
                        ({"rabitq_bits_per_dim_base": 4, "rabitq_bits_per_dim_query": 4},
                         "not support num_bits_per_dim_query_ == 4 with num_bits_per_dim_base_ != 1"),
                        ({"rabitq_bits_per_dim_base": 4, "fast_encode_rabitq_rounds": 0},
                         "fast_encode_rabitq_rounds must be in [1, 32], but got 0"),
                        ({"rabitq_bits_per_dim_base": 4, "fast_encode_rabitq_rounds": 33},
                         "fast_encode_rabitq_rounds must be in [1, 32], but got 33"),
                        ({"rabitq_version": "v9"}, "unsupported rabitq_version: v9"),
                        ({"rabitq_version": "split"}, "split"),
                        ({"rabitq_error_rate": -1.0}, "rabitq_error_rate must be finite and positive")):
        with pytest.raises(pyvsag.VsagError) as e:
            make("ivf", d, "l2", buckets_count=4, base_quantization_type="rabitq", **extra)
        assert e.value.code == -3 and text in e.value.message, (extra, e.value.message)
    # brute force takes the same codes
    n, nq, k = 1500, 20, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=3)
    labels = np.arange(n, dtype=np.int64)
    idx = make("brute_force", d, "l2", base_quantization_type="rabitq", rabitq_bits_per_dim_base=8,
               fast_encode_rabitq_rounds=3)
    idx.build(x, labels, n, d)
    gt, _ = ground_truth(x, q, k, "l2")
    ids, _ = idx.knn_search_batch(q, k, "{}")
    assert recall(ids, gt, labels) >= 0.97
    idx.close()


# ------------------------------------------------------------------------------------------------------------------
# Pre-filters and range search, after TestIndex::TestFilterSearch / TestRangeSearch
# (tests/test_index/test_index_search.cpp:100-160,263-350): filter(label) == True filters the vector out; the range
# radius sits between the (k-1)-th and k-th exact distances; results never contain a filtered label.
def _filtered_truth(x, q, labels, k, metric, keep):
    allowed = np.nonzero(keep)[0]
    gt, gt_d = ground_truth(x[allowed], q, k, metric)
    return labels[allowed][gt], gt_d


@pytest.mark.parametrize("name,params,search", [
    ("brute_force", {"base_quantization_type": "fp32"}, "{}"),
    ("brute_force", {"base_quantization_type": "sq8"}, "{}"),
    ("ivf", {"buckets_count": 20, "base_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 20}})),
    ("ivf", {"buckets_count": 20, "base_quantization_type": "sq8", "use_reorder": True,
             "precise_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 20, "factor": 4.0}})),
])
def test_filter_search(lib, name, params, search):
    n, d, nq, k = 3000, 32, 20, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) * 5 + 3
    idx = make(name, d, "l2", **params)
    assert idx.build(x, labels, n, d) == 0
    flt = lambda label: label % 3 != 0  # noqa: E731  (keeps a third, like the fixtures' valid_ratio cases)
    keep = np.array([not flt(int(v)) for v in labels])
    gt_labels, gt_d = _filtered_truth(x, q, labels, k, "l2", keep)
    hits = range_hits = 0
    for i in range(nq):
        ids, dists = idx.knn_search(q[i], k, search, filter=flt)
        assert ids.size == k and np.all(np.diff(dists) >= 0)
        assert not any(flt(int(v)) for v in ids)
        hits += len(set(ids.tolist()) & set(gt_labels[i].tolist()))
        threshold = 0.5 * float(gt_d[i][k - 2] + gt_d[i][k - 1])
        rids, rd = idx.range_search(q[i], threshold, search, filter=flt)
        assert not any(flt(int(v)) for v in rids)
        assert np.all(rd <= threshold + 2e-6) or params["base_quantization_type"] != "fp32"
        range_hits += len(set(rids.tolist()) & set(gt_labels[i][:k - 1].tolist()))
    floor = 0.99 if params["base_quantization_type"] == "fp32" else 0.8
    assert hits / float(nq * k) > floor * RECALL_THRESHOLD
    assert range_hits / float(nq * (k - 1)) > floor * RECALL_THRESHOLD
    # nothing survives the filter: empty result, not an error
    ids, dists = idx.knn_search(q[0], k, search, filter=lambda label: True)
    assert ids.size == 0
    idx.close()


@pytest.mark.parametrize("name,params,search", [
    ("brute_force", {"base_quantization_type": "fp32"}, "{}"),
    ("ivf", {"buckets_count": 16, "base_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 16}})),
])
def test_range_search(lib, name, params, search):
    n, d, nq = 5000, 16, 12
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) + 100
    idx = make(name, d, "l2", **params)
    assert idx.build(x, labels, n, d) == 0
    x64 = x.astype(np.float64)
    for i in range(nq):
        dd = ((x64 - q[i].astype(np.float64)) ** 2).sum(1)
        order = np.argsort(dd, kind="stable")
        # a radius that takes in 1500 vectors: more than one device scan of 1024
        for count in (7, 1500):
            radius = 0.5 * float(dd[order[count - 1]] + dd[order[count]])
            ids, dists = idx.range_search(q[i], radius, search)
            # the bucket searcher admits radius + 2e-6 (THRESHOLD_ERROR, impl/searcher/basic_searcher.h:39)
            slack = 2e-6 if name == "ivf" else 0.0
            extra = int(np.sum((dd > radius) & (dd <= radius + slack + 1e-7)))
            assert count <= ids.size <= count + extra, (i, count, ids.size)
            assert np.all(np.diff(dists) >= 0) and dists[-1] <= radius + slack + 1e-7
            assert set(ids[:count].tolist()) == set(labels[order[:count]].tolist())
            np.testing.assert_allclose(dists[:count], dd[order[:count]], rtol=1e-4, atol=1e-6)
            lim_ids, lim_d = idx.range_search(q[i], radius, search, limit=5)
            assert lim_ids.size == 5 and set(lim_ids.tolist()) == set(labels[order[:5]].tolist())
        ids, _ = idx.range_search(q[i], 0.0, search)  # nothing that close
        assert ids.size == 0
    with pytest.raises(pyvsag.VsagError) as e:
        idx.range_search(q[0], -1.0, search)
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        idx.range_search(q[0], 1.0, search, limit=0)
    assert e.value.code == -3
    idx.close()


@pytest.mark.parametrize("name,params,search", [
    ("brute_force", {"base_quantization_type": "fp32"}, "{}"),
    ("ivf", {"buckets_count": 16, "base_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 16}})),
    ("ivf", {"buckets_count": 16, "base_quantization_type": "sq8", "use_reorder": True,
             "precise_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 16, "factor": 1.5}})),
])
def test_k_above_one_device_scan(lib, name, params, search):
    """k larger than the 1024 results of one device scan: several scans per query, for one query per call and for a
    batch (whose rows are the single-query results)."""
    n, d, k = 6000, 16, 2500
    x = vectors(n, d)
    q = vectors(3, d, seed=165)
    labels = np.arange(n, dtype=np.int64) * 2
    idx = make(name, d, "l2", **params)
    assert idx.build(x, labels, n, d) == 0
    gt, gt_d = ground_truth(x, q, k, "l2")
    bids, bdists = idx.knn_search_batch(q, k, search)
    assert bids.shape == (3, k)
    for i in range(3):
        ids, dists = idx.knn_search(q[i], k, search)
        assert ids.size == k and np.unique(ids).size == k
        assert np.all(np.diff(dists) >= 0)
        hit = len(set(ids.tolist()) & set(labels[gt[i]].tolist())) / float(k)
        if params["base_quantization_type"] == "fp32":
            assert hit >= 0.999
            np.testing.assert_allclose(dists, gt_d[i], rtol=1e-4, atol=1e-6)
        else:
            assert hit >= 0.9
        assert np.array_equal(bids[i], ids) and np.array_equal(bdists[i], dists)
    # more than the index holds: the rows end with -1 / inf
    few = make(name, d, "l2", **params)
    few.build(x[:1500], labels[:1500], 1500, d)
    fids, fd = few.knn_search_batch(q, 2000, search)
    assert fids.shape == (3, 2000) and np.all(fids[:, 1500:] == -1) and np.all(np.isinf(fd[:, 1500:]))
    assert all(np.unique(fids[i, :1500]).size == 1500 for i in range(3)) or params["base_quantization_type"] != "fp32"
    few.close()
    idx.close()


@pytest.mark.parametrize("quant,metric", [("sq4_uniform", "l2"), ("sq8_uniform", "ip"), ("sq8", "l2"), ("sq8", "cosine"),
                                          ("sq4", "l2"), ("rabitq", "l2")])
@pytest.mark.parametrize("reorder", [True, False])
def test_ivf_large_batch_equals_one_by_one(lib, reorder, quant, metric):
    """A batch large enough for the matrix-core pass over the posting lists (sq4_uniform, sq8_uniform, sq8, sq4, rabitq)
    returns what single queries (chunked streaming scan) return."""
    n, d, nq, k = 60000, 64, 2200, 10
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 2 + 1
    params = dict(buckets_count=64, base_quantization_type=quant, train_sample_count=20000)
    if reorder:
        params.update(use_reorder=True, precise_quantization_type="fp32")
    idx = make("ivf", d, metric, **params)
    assert idx.build(x, labels, n, d) == 0
    search = json.dumps({"ivf": {"scan_buckets_count": 16, "factor": 4.0}})
    ids, dists = idx.knn_search_batch(q, k, search)
    for i in range(0, nq, 61):
        si, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(si, ids[i]) and np.array_equal(sd.view(np.uint32), dists[i].view(np.uint32)), i
    idx.close()


def test_rabitq_large_batch_equals_one_by_one(lib):
    """brute_force over 1-bit RaBitQ codes with 4-bit queries: a batch served by the int8 matrix cores returns what
    single queries (streaming popcount scan) return."""
    n, d, nq, k = 70000, 256, 600, 50
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) * 3 + 2
    idx = make("brute_force", d, "ip", base_quantization_type="rabitq", rabitq_bits_per_dim_query=4)
    assert idx.build(x, labels, n, d) == 0
    ids, dists = idx.knn_search_batch(q, k, "{}")
    tile, passes, nbytes = C.c_int(), C.c_uint64(), C.c_uint64()
    capi.load_library().vsag_amd_last_scan_info(C.byref(tile), C.byref(passes), C.byref(nbytes))
    assert tile.value == 128, "the batch did not take the matrix-core route"
    for i in range(0, nq, 41):
        si, sd = idx.knn_search(q[i], k, "{}")
        assert np.array_equal(si, ids[i]) and np.array_equal(sd.view(np.uint32), dists[i].view(np.uint32)), i
    idx.close()


@pytest.mark.parametrize("quant", ["fp32", "sq8", "sq4", "sq8_uniform", "sq4_uniform"])
def test_large_batch_equals_one_by_one(lib, quant):
    """A batch large enough for the matrix-core path of the flat scan returns what single queries return."""
    n, d, nq, k = 70000, 32, 600, 10
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) + 5
    idx = make("brute_force", d, "l2", base_quantization_type=quant)
    assert idx.build(x, labels, n, d) == 0
    ids, dists = idx.knn_search_batch(q, k, "{}")
    for i in range(0, nq, 37):
        si, sd = idx.knn_search(q[i], k, "{}")
        assert np.array_equal(si, ids[i]) and np.array_equal(sd.view(np.uint32), dists[i].view(np.uint32)), i
    if quant == "fp32":
        gt, _ = ground_truth(x, q[:50], k, "l2")
        assert recall(ids[:50], gt, labels) >= 0.999
    idx.close()


@pytest.mark.parametrize("name,metric", [("brute_force", "l2"), ("brute_force", "cosine"), ("ivf", "l2"), ("ivf", "ip")])
def test_sq8_beyond_128_dimensions_large_batch_equals_one_by_one(lib, name, metric):
    """sq8 codes of 200 dimensions: a batch large enough for the fp16 matrix cores (flat store: prefilter_h16_kernel,
    posting lists: ivf_h16_kernel) returns what single queries (streaming scan) return, ids and distance bits."""
    n, d, k = 70000, 200, 10
    nq = 600 if name == "brute_force" else 2200
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 3 + 2
    params = dict(base_quantization_type="sq8")
    search = "{}"
    if name == "ivf":
        params.update(buckets_count=64, train_sample_count=20000)
        search = json.dumps({"ivf": {"scan_buckets_count": 16}})
    idx = make(name, d, metric, **params)
    assert idx.build(x, labels, n, d) == 0
    ids, dists = idx.knn_search_batch(q, k, search)
    for i in range(0, nq, 53):
        si, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(si, ids[i]) and np.array_equal(sd.view(np.uint32), dists[i].view(np.uint32)), i
    gt, _ = ground_truth(x, q[:40], k, metric)
    assert recall(ids[:40], gt, labels) >= (0.95 if name == "brute_force" else 0.3)  # (16 of 64 lists of unclustered rows)
    idx.close()


def test_ivf_with_a_thousand_buckets_routes_large_batches_through_the_table(lib):
    """1024 buckets: Add classifies 65 536 rows a call and a search batch of 1100 queries routes through the table of
    approximate centroid distances; both must give what single queries give (exact routing either way)."""
    n, d, nq, k = 70000, 32, 1100, 10
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 3 + 7
    idx = make("ivf", d, "l2", buckets_count=1024, base_quantization_type="sq8", train_sample_count=30000)
    assert idx.build(x, labels, n, d) == 0
    search = json.dumps({"ivf": {"scan_buckets_count": 32}})
    ids, dists = idx.knn_search_batch(q, k, search)
    for i in range(0, nq, 53):
        si, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(si, ids[i]) and np.array_equal(sd.view(np.uint32), dists[i].view(np.uint32)), i
    # every bucket probed: the exact sq8 neighbours, whichever way the rows were classified
    every = json.dumps({"ivf": {"scan_buckets_count": 1024}})
    ai, _ = idx.knn_search_batch(q[:1024], k, every)
    gt, _ = ground_truth(x, q[:100], k, "l2")
    assert recall(ai[:100], gt, labels) >= 0.9
    idx.close()


@pytest.mark.parametrize("metric", ["l2", "ip", "cosine"])
@pytest.mark.parametrize("residual", [False, True])
def test_ivf_pqfs_recall_floor_and_conventions(lib, metric, residual):
    """base_quantization_type "pqfs" with fp32 reorder: the reference's floor for "pqfs,fp32" is 0.82, with a subspace
    per dimension (tests/test_ivf.cpp:94-102,166-172,1292-1300), with and without use_residual."""
    n, d, nq, k = 2400, 64, 100, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) + 1000
    idx = make("ivf", d, metric, buckets_count=50, base_quantization_type="pqfs", base_pq_dim=d, use_reorder=True,
               precise_quantization_type="fp32", train_sample_count=2400, use_residual=residual)
    assert idx.build(x, labels, n, d) == 0
    gt, _ = ground_truth(x, q, k, metric)
    search = json.dumps({"ivf": {"scan_buckets_count": 30, "factor": 4.0}})
    ids, dists = idx.knn_search_batch(q, k, search)
    r = recall(ids, gt, labels)
    assert r >= 0.82 * RECALL_THRESHOLD, r
    assert np.all(np.diff(dists, axis=1) >= 0)
    for i in range(8):  # batch == serial, bit for bit
        sid, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(sid, ids[i]) and np.array_equal(sd, dists[i])
    idx.close()


def test_ivf_fp32_cosine_with_residual(lib, tmp_path):
    """use_residual with fp32 codes under cosine: FP32Quantizer::EncodeOneImpl (fp32_quantizer.cpp:58-72) normalises
    the residual it is handed, so the lists estimate the angle from the direction of x - c alone; with the fp32
    reorder behind it the search still finds the neighbours, and a reloaded index answers alike."""
    n, d, nq, k = 3000, 32, 50, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64)
    params = dict(buckets_count=20, base_quantization_type="fp32", use_residual=True, use_reorder=True,
                  precise_quantization_type="fp32", train_sample_count=3000)
    idx = make("ivf", d, "cosine", **params)
    assert idx.build(x, labels, n, d) == 0
    gt, _ = ground_truth(x, q, k, "cosine")
    search = json.dumps({"ivf": {"scan_buckets_count": 20, "factor": 10.0}})
    ids, dists = idx.knn_search_batch(q, k, search)
    assert recall(ids, gt, labels) >= 0.9
    assert np.all(np.diff(dists, axis=1) >= 0)
    sid, sd = idx.knn_search(q[0], k, search)
    assert np.array_equal(sid, ids[0]) and np.allclose(sd, dists[0], rtol=1e-5, atol=1e-6)
    idx.serialize(tmp_path / "res.index")
    again = make("ivf", d, "cosine", **params)
    again.deserialize(tmp_path / "res.index")
    ids2, dists2 = again.knn_search_batch(q, k, search)
    assert np.array_equal(ids2, ids) and np.array_equal(dists2, dists)
    again.close()
    idx.close()


def test_pqfs_parameters_and_brute_force(lib):
    d = 48
    # pq_fastscan_quantizer.cpp:31-36: pq_dim must divide the dimension; the default pq_dim is 1
    with pytest.raises(pyvsag.VsagError) as e:
        make("ivf", d, "l2", buckets_count=8, base_quantization_type="pqfs", base_pq_dim=7)
    assert "does not divide evenly" in str(e.value)
    with pytest.raises(pyvsag.VsagError):
        make("ivf", d, "l2", buckets_count=8, base_quantization_type="sq8", use_reorder=True,
             precise_quantization_type="pqfs")
    # a flat store of pqfs codes scans like any other kind: against the checker on the same codebooks it would be
    # bit-exact (tests/test_pqfs_gpu.py); here the approximation itself, with a subspace per dimension
    n, nq, k = 3000, 40, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64)
    idx = make("brute_force", d, "l2", base_quantization_type="pqfs", base_pq_dim=d)
    assert idx.build(x, labels, n, d) == 0
    ids, dists = idx.knn_search_batch(q, k, "{}")
    gt, gt_d = ground_truth(x, q, k, "l2")
    assert recall(ids, gt, labels) >= 0.5
    true = ((q[:, None].astype(np.float64) - x[ids].astype(np.float64)) ** 2).sum(-1)
    assert np.abs(dists - true).max() <= 0.08  # the bound of the reference's own quantizer test
    idx.close()
