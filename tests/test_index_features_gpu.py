"""The rest of the index interface for brute_force / ivf: Train, Add in pieces, SearchWithRequest with injected buckets,
CalDistanceById, buckets_per_data, use_residual, a quantised precise store, statistics by phase and concurrent searches.
Modelled on the reference's functional tests: tests/test_ivf.cpp:465-479 (CalDistanceById within 2e-6 of the search's
distances), tests/test_ivf.cpp:1002-1060 (buckets_per_data / residual recall floors), tests/test_index/
test_index_search.cpp:430-520 (concurrent searches give the serial results), src/algorithm/ivf/ivf_test.cpp (bucket_ids_
validation)."""
import json
import threading

import numpy as np
import pytest

from test_index_api_gpu import RECALL_THRESHOLD, ground_truth, make, recall, vectors
from vsag_amd import pyvsag

pytestmark = pytest.mark.gpu


def clustered(count, dim, centres, seed=47, spread=0.05):
    rng = np.random.Generator(np.random.MT19937(seed))
    c = rng.uniform(-1.0, 1.0, (centres, dim)).astype(np.float32)
    which = rng.integers(0, centres, count)
    return (c[which] + spread * rng.standard_normal((count, dim))).astype(np.float32)


def routed(idx, x, nprobe):
    """The nprobe nearest lists of every row, through the routing-only search (IVF::route_buckets_only)."""
    search = json.dumps({"ivf": {"scan_buckets_count": nprobe, "disable_bucket_scan": True}})
    ids, _ = idx.knn_search_batch(x, nprobe, search)
    return ids


def members(idx, nlist, dim, room):
    """Labels held by every list: one search per list with that list injected (one query per call, so that a list
    longer than one device scan is still returned whole)."""
    q = np.zeros((1, dim), np.float32) + 0.5
    held = []
    for b in range(nlist):
        ids, _ = idx.knn_search_batch(q, room, json.dumps({"ivf": {"scan_buckets_count": 1}}), bucket_ids=[[b]])
        held.append(set(ids[0][ids[0] >= 0].tolist()))
    return held


@pytest.mark.parametrize("metric", ["l2", "ip", "cosine"])
def test_ivf_membership_follows_the_router_metric(lib, metric):
    # IVFNearestPartition::ClassifyDatas searches the router index, which measures the index metric: with vectors of
    # different lengths the ip-nearest centroid is not the l2-nearest one.
    n, d, nlist = 3000, 24, 16
    x = vectors(n, d, normalize=False) * np.linspace(0.3, 3.0, n, dtype=np.float32)[:, None]
    labels = np.arange(n, dtype=np.int64)
    idx = make("ivf", d, metric, buckets_count=nlist, train_sample_count=3000)
    assert idx.build(x, labels, n, d) == 0
    held = members(idx, nlist, d, n)
    assert sum(len(h) for h in held) == n
    want = routed(idx, x, 1)[:, 0]
    got = np.full(n, -1)
    for b, h in enumerate(held):
        got[list(h)] = b
    assert np.array_equal(got, want)
    idx.close()


def test_ivf_buckets_per_data(lib):
    n, d, nq, k, nlist = 3000, 32, 60, 10, 32
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 2 + 1
    one = make("ivf", d, "l2", buckets_count=nlist, train_sample_count=3000)
    two = make("ivf", d, "l2", buckets_count=nlist, train_sample_count=3000, buckets_per_data=2)
    assert one.build(x, labels, n, d) == 0 and two.build(x, labels, n, d) == 0
    assert two.get_num_elements() == n
    # every vector sits in its two nearest lists
    held = members(two, nlist, d, n)
    assert sum(len(h) for h in held) == 2 * n
    want = routed(two, x, 2)
    for i in range(0, n, 37):
        assert labels[i] in held[want[i, 0]] and labels[i] in held[want[i, 1]]
    # all lists probed: the brute-force answer, every label once
    bf = make("brute_force", d, "l2")
    bf.build(x, labels, n, d)
    a_ids, a_d = bf.knn_search_batch(q, k, "{}")
    b_ids, b_d = two.knn_search_batch(q, k, json.dumps({"ivf": {"scan_buckets_count": nlist}}))
    assert np.array_equal(a_ids, b_ids) and np.array_equal(a_d, b_d)
    # few lists probed: no label twice, and no worse than one list per vector
    search = json.dumps({"ivf": {"scan_buckets_count": 3}})
    gt, _ = ground_truth(x, q, k, "l2")
    ids1, _ = one.knn_search_batch(q, k, search)
    ids2, d2 = two.knn_search_batch(q, k, search)
    for row in ids2:
        assert len(set(row.tolist())) == k
    assert np.all(np.diff(d2, axis=1) >= 0)
    assert recall(ids2, gt, labels) >= recall(ids1, gt, labels)
    for i in range(5):
        sid, sd = two.knn_search(q[i], k, search)
        assert np.array_equal(sid, ids2[i]) and np.array_equal(sd, d2[i])
    # a filter and a range search see vectors, not postings
    flt = lambda label: label % 4 == 1  # noqa: E731
    fid, _ = two.knn_search(q[0], k, search, filter=flt)
    assert fid.size == k and len(set(fid.tolist())) == k and not any(flt(int(v)) for v in fid)
    rid, rd = two.range_search(q[0], float(a_d[0, -1]) * 1.0001, json.dumps({"ivf": {"scan_buckets_count": nlist}}))
    assert np.array_equal(np.sort(rid), np.sort(a_ids[0])) and len(set(rid.tolist())) == rid.size
    for idx in (one, two, bf):
        idx.close()


# improves: the codes of x - c span one cluster instead of the whole data, so the distances get more accurate.  Not so
# where the reference's arithmetic works against it, which is kept as it is: under cosine the quantizer normalises what
# it encodes, the residual included (sq8_quantizer.cpp EncodeOneImpl), and the uniform kinds encode the query with the
# quantizer trained on the residuals, which clips it (bucket_datacell.h:575-591 hands the raw query to SetQuery).
@pytest.mark.parametrize("metric,quant,improves", [("l2", "fp32", False), ("ip", "fp32", False), ("l2", "sq8", True),
                                                   ("ip", "sq8", True), ("l2", "sq4", True), ("cosine", "sq8", False),
                                                   ("l2", "sq8_uniform", False), ("l2", "rabitq", False),
                                                   ("ip", "rabitq", False)])
def test_ivf_use_residual(lib, metric, quant, improves):
    n, d, nq, k, nlist = 4000, 32, 50, 10, 32
    # fewer clusters than lists, so that k-means splits clusters rather than merging them
    both = clustered(n + nq, d, 8)
    x, q = both[:n], both[n:]
    labels = np.arange(n, dtype=np.int64)
    plain = make("ivf", d, metric, buckets_count=nlist, base_quantization_type=quant, train_sample_count=4000)
    res = make("ivf", d, metric, buckets_count=nlist, base_quantization_type=quant, train_sample_count=4000,
               use_residual=True)
    assert plain.build(x, labels, n, d) == 0 and res.build(x, labels, n, d) == 0
    search = json.dumps({"ivf": {"scan_buckets_count": nlist}})
    gt, gt_d = ground_truth(x, q, 100, metric)
    ids_p, d_p = plain.knn_search_batch(q, 100, search)
    ids_r, d_r = res.knn_search_batch(q, 100, search)
    assert np.all(np.diff(d_r, axis=1) >= 0)
    assert all(len(set(row.tolist())) == 100 for row in ids_r)

    def error(ids, dists):
        exact = ground_truth_at(x, q, ids, metric)
        return float(np.mean(np.abs(dists - exact)))

    if quant == "fp32":
        # nothing is lost: (x - c) + c differs from x by rounding only
        assert recall(ids_r[:, :k], gt[:, :k], labels) >= 0.99
        assert error(ids_r, d_r) < 1e-5
    elif improves:
        assert error(ids_r, d_r) < 0.85 * error(ids_p, d_p)
        assert recall(ids_r[:, :k], gt[:, :k], labels) >= recall(ids_p[:, :k], gt[:, :k], labels) - 0.02
    # batch == serial, CalDistanceById == the search's distances (tests/test_ivf.cpp:465-479)
    for i in range(4):
        sid, sd = res.knn_search(q[i], k, search)
        assert np.array_equal(sid, ids_r[i, :k]) and np.array_equal(sd, d_r[i, :k])
        assert np.allclose(res.cal_distance_by_id(q[i], sid), sd, rtol=0, atol=2e-6)
    # added later: the same codes and distances as when built in one go
    x2 = clustered(n + 300, d, 8)[n:] + np.float32(0.01)
    l2 = np.arange(300, dtype=np.int64) + n
    assert res.add(x2, l2, 300, d) == 0 and res.get_num_elements() == n + 300
    whole = make("ivf", d, metric, buckets_count=nlist, base_quantization_type=quant, train_sample_count=4000,
                 use_residual=True)
    whole.train(x, labels, n, d)
    whole.add(np.concatenate([x, x2]), np.concatenate([labels, l2]), n + 300, d)
    a_ids, a_d = res.knn_search_batch(q, k, search)
    b_ids, b_d = whole.knn_search_batch(q, k, search)
    assert np.array_equal(a_ids, b_ids) and np.array_equal(a_d, b_d)
    if metric == "l2" and (improves or quant == "fp32"):
        ids2, _ = res.knn_search_batch(x2[:50], 1, search)
        assert np.mean(ids2[:, 0] == l2[:50]) >= 0.9
    for idx in (plain, res, whole):
        idx.close()


def ground_truth_at(x, q, ids, metric):
    x64, q64 = x.astype(np.float64)[ids], q.astype(np.float64)[:, None, :]
    if metric == "l2":
        return ((x64 - q64) ** 2).sum(2)
    if metric == "ip":
        return 1 - (x64 * q64).sum(2)
    return 1 - (x64 * q64).sum(2) / (np.linalg.norm(x64, axis=2) * np.linalg.norm(q64, axis=2))


def test_ivf_reorder_with_quantised_precise_codes(lib):
    n, d, nq, k = 3000, 48, 40, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) + 5
    idx = make("ivf", d, "l2", buckets_count=16, base_quantization_type="sq4_uniform", use_reorder=True,
               precise_quantization_type="sq8", train_sample_count=3000)
    assert idx.build(x, labels, n, d) == 0
    search = json.dumps({"ivf": {"scan_buckets_count": 16, "factor": 8.0}})
    ids, dists = idx.knn_search_batch(q, k, search)
    assert np.all(np.diff(dists, axis=1) >= 0)
    gt, _ = ground_truth(x, q, k, "l2")
    assert recall(ids, gt, labels) >= 0.9 * RECALL_THRESHOLD
    # the distances are those of the sq8 codes: the same quantizer, trained on the same rows, in a brute_force index
    bf = make("brute_force", d, "l2", base_quantization_type="sq8")
    bf.build(x, labels, n, d)
    assert np.array_equal(bf.cal_distance_by_id(q, ids), dists)
    assert np.array_equal(idx.cal_distance_by_id(q, ids, precise=True), dists)
    # precise = False: the sq4_uniform codes of the lists, what a search without the reorder returns
    raw_ids, raw_d = idx.knn_search_batch(q, k, json.dumps({"ivf": {"scan_buckets_count": 16, "enable_reorder": False}}))
    assert np.allclose(idx.cal_distance_by_id(q, raw_ids, precise=False), raw_d, rtol=0, atol=2e-6)
    for i in range(4):
        sid, sd = idx.knn_search(q[i], k, search)
        assert np.array_equal(sid, ids[i]) and np.array_equal(sd, dists[i])
    idx.close()
    bf.close()


def test_search_with_injected_buckets(lib):
    n, d, nq, k, nlist = 3000, 32, 30, 10, 24
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    idx = make("ivf", d, "l2", buckets_count=nlist, base_quantization_type="sq8", use_reorder=True,
               precise_quantization_type="fp32", train_sample_count=3000)
    idx.build(x, np.arange(n, dtype=np.int64), n, d)
    search = json.dumps({"ivf": {"scan_buckets_count": 5, "factor": 3.0}})
    want_ids, want_d = idx.knn_search_batch(q, k, search)
    buckets = routed(idx, q, 5)
    got_ids, got_d = idx.knn_search_batch(q, k, search, bucket_ids=[row.tolist() for row in buckets])
    assert np.array_equal(got_ids, want_ids) and np.array_equal(got_d, want_d)
    # rows of different lengths: the short ones scan fewer lists
    ragged = [row[:1 + (i % 5)].tolist() for i, row in enumerate(buckets)]
    rag_ids, rag_d = idx.knn_search_batch(q, k, search, bucket_ids=ragged)
    for i in (0, 1, 7, 13):
        one_ids, one_d = idx.knn_search_batch(q[i:i + 1], k, search, bucket_ids=[ragged[i]])
        assert np.array_equal(one_ids[0], rag_ids[i]) and np.array_equal(one_d[0], rag_d[i])
    assert np.array_equal(rag_ids[4], want_ids[4])  # row 4 has all five
    for bad, text in [([[]] + ragged[1:], "must not be empty"), ([[nlist]] + ragged[1:], "out of range"),
                      ([[-1]] + ragged[1:], "out of range"), ([[3, 3]] + ragged[1:], "duplicate bucket_id"),
                      (ragged[1:], "must match the number of query vectors")]:
        with pytest.raises(pyvsag.VsagError) as e:
            idx.knn_search_batch(q, k, search, bucket_ids=bad)
        assert e.value.code == -3 and text in e.value.message, e.value.message
    with pytest.raises(pyvsag.VsagError) as e:
        idx.knn_search_batch(q, k, json.dumps({"ivf": {"scan_buckets_count": 5, "disable_bucket_scan": True}}),
                             bucket_ids=ragged)
    assert e.value.code == -3 and "disable_bucket_scan" in e.value.message
    idx.close()


@pytest.mark.parametrize("name,params,search", [
    ("brute_force", {"base_quantization_type": "sq8"}, "{}"),
    ("ivf", {"buckets_count": 20, "base_quantization_type": "sq8", "use_reorder": True,
             "precise_quantization_type": "fp32", "train_sample_count": 4000},
     json.dumps({"ivf": {"scan_buckets_count": 6, "factor": 3.0}})),
    ("ivf", {"buckets_count": 20, "base_quantization_type": "sq8_uniform", "use_residual": True,
             "buckets_per_data": 2, "train_sample_count": 4000}, json.dumps({"ivf": {"scan_buckets_count": 6}})),
])
def test_train_then_add_in_pieces_equals_build(lib, name, params, search):
    n, d, nq, k = 4000, 32, 40, 10
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64) + 11
    whole = make(name, d, "l2", **params)
    assert whole.build(x, labels, n, d) == 0
    parts = make(name, d, "l2", **params)
    if name == "ivf":
        with pytest.raises(pyvsag.VsagError) as e:
            parts.add(x[:10], labels[:10], 10, d)
        assert e.value.code == -2 and "add without train" in e.value.message
    parts.train(x, labels, n, d)
    assert parts.get_num_elements() == 0
    ids, _ = parts.knn_search(q[0], k, search)
    assert ids.size == 0
    cuts = [0, 1, 700, 701, 2500, n]
    for a, b in zip(cuts[:-1], cuts[1:]):
        assert parts.add(x[a:b], labels[a:b], b - a, d) == 0
    assert parts.add(x[:5], labels[:5], 5, d) == 5  # all duplicates
    assert parts.get_num_elements() == n
    a_ids, a_d = whole.knn_search_batch(q, k, search)
    b_ids, b_d = parts.knn_search_batch(q, k, search)
    assert np.array_equal(a_ids, b_ids) and np.array_equal(a_d, b_d)
    whole.close()
    parts.close()


@pytest.mark.parametrize("name,params,search", [
    ("brute_force", {"base_quantization_type": "fp32"}, "{}"),
    ("brute_force", {"base_quantization_type": "sq8"}, "{}"),
    ("brute_force", {"base_quantization_type": "rabitq"}, "{}"),
    ("ivf", {"buckets_count": 12, "base_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 12}})),
    ("ivf", {"buckets_count": 12, "base_quantization_type": "sq8", "use_reorder": True,
             "precise_quantization_type": "fp32"}, json.dumps({"ivf": {"scan_buckets_count": 12, "factor": 3.0}})),
    ("ivf", {"buckets_count": 12, "base_quantization_type": "sq4", "buckets_per_data": 3},
     json.dumps({"ivf": {"scan_buckets_count": 12}})),
])
@pytest.mark.parametrize("metric", ["l2", "cosine"])
def test_cal_distance_by_id(lib, name, params, search, metric):
    n, d, nq, k = 2000, 64, 6, 20
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 7 + 2
    idx = make(name, d, metric, train_sample_count=2000, **params) if name == "ivf" else make(name, d, metric, **params)
    idx.build(x, labels, n, d)
    ids, dists = idx.knn_search_batch(q, k, search)
    # tests/test_ivf.cpp:465-479: within 2e-6 of what the search reported
    got = idx.cal_distance_by_id(q, ids)
    assert got.shape == (nq, k) and np.allclose(got, dists, rtol=0, atol=2e-6)
    one = idx.cal_distance_by_id(q[2], ids[2])
    assert np.array_equal(one, got[2])
    if params.get("use_reorder"):
        # precise: the fp32 rows; not precise: the sq8 codes of the lists
        exact = ground_truth_at(x, q, (ids - 2) // 7, metric)
        assert np.allclose(got, exact, rtol=1e-4, atol=2e-6)
        raw = idx.cal_distance_by_id(q, ids, precise=False)
        assert not np.array_equal(raw, got) and np.allclose(raw, exact, rtol=0.05, atol=0.05)
    # unknown labels: -1, and last when the smallest are selected
    mixed = ids.copy()
    mixed[:, 3] = 1  # no vector has label 1
    mixed[:, 11] = -5
    plain = idx.cal_distance_by_id(q, mixed)
    assert np.all(plain[:, 3] == -1) and np.all(plain[:, 11] == -1)
    keep = np.ones(k, bool)
    keep[[3, 11]] = False
    assert np.array_equal(plain[:, keep], got[:, keep])
    top_ids, top_d = idx.cal_distance_by_id(q, mixed, topk=k)
    assert np.array_equal(top_d[:, :k - 2], np.sort(got[:, keep], axis=1)) and np.all(top_d[:, k - 2:] == -1)
    assert np.all(np.isin(top_ids[:, k - 2:], [1, -5]))
    few_ids, few_d = idx.cal_distance_by_id(q[0], mixed[0], topk=4)
    assert few_d.shape == (4,) and np.array_equal(few_d, top_d[0, :4]) and np.array_equal(few_ids, top_ids[0, :4])
    with pytest.raises(pyvsag.VsagError) as e:
        idx.cal_distance_by_id(q[0], mixed[0], topk=0)
    assert e.value.code == -3
    idx.close()


def test_statistics_by_phase(lib):
    n, d, nlist, k = 3000, 32, 16, 10
    x = vectors(n, d)
    labels = np.arange(n, dtype=np.int64)
    bf = make("brute_force", d, "l2", base_quantization_type="sq8")
    bf.build(x, labels, n, d)
    _, _, text = bf.knn_search(x[0], k, "{}", statistics=True)
    s = json.loads(text)
    assert s["dist_cmp"] == n and s["distance_evaluations"] == n and not s["is_timeout"]
    assert s["distance_evaluations_by_phase"] == {"routing": 0, "approximate": n, "rerank": 0}
    assert s["distance_evaluations_by_backend"] == {"sq8": n}
    ivf = make("ivf", d, "l2", buckets_count=nlist, base_quantization_type="sq8", use_reorder=True,
               precise_quantization_type="fp32", train_sample_count=3000)
    ivf.build(x, labels, n, d)
    _, _, text = ivf.knn_search(x[0], k, json.dumps({"ivf": {"scan_buckets_count": nlist, "factor": 3.0}}),
                                statistics=True)
    s = json.loads(text)
    assert s["distance_evaluations_by_phase"] == {"routing": nlist, "approximate": n, "rerank": 3 * k}
    assert s["distance_evaluations_by_backend"] == {"fp32": nlist + 3 * k, "sq8": n}
    assert s["distance_evaluations"] == nlist + n + 3 * k
    held = members(ivf, nlist, d, n)
    near = routed(ivf, x[:1], 3)[0]
    _, _, text = ivf.knn_search(x[0], k, json.dumps({"ivf": {"scan_buckets_count": 3, "enable_reorder": False}}),
                                statistics=True)
    s = json.loads(text)
    assert s["distance_evaluations_by_phase"] == {"routing": nlist, "approximate": sum(len(held[b]) for b in near),
                                                  "rerank": 0}
    bf.close()
    ivf.close()


@pytest.mark.parametrize("name,params,search", [
    ("brute_force", {"base_quantization_type": "sq8"}, "{}"),
    ("ivf", {"buckets_count": 24, "base_quantization_type": "sq8_uniform", "use_reorder": True,
             "precise_quantization_type": "fp32", "train_sample_count": 20000},
     json.dumps({"ivf": {"scan_buckets_count": 6, "factor": 3.0}})),
])
def test_concurrent_searches_equal_serial(lib, name, params, search):
    # SUPPORT_SEARCH_CONCURRENT: sixteen threads, one query per call (the shape of tools/eval's search loop), mixed with
    # batches, filters and CalDistanceById on the same index.
    n, d, nq, k, threads = 20000, 64, 320, 10, 16
    x = vectors(n, d)
    q = vectors(nq, d, seed=165)
    labels = np.arange(n, dtype=np.int64)
    idx = make(name, d, "l2", **params)
    idx.build(x, labels, n, d)
    want_ids, want_d = idx.knn_search_batch(q, k, search)
    flt = lambda label: label % 2 == 0  # noqa: E731
    want_f = [idx.knn_search(q[i], k, search, filter=flt) for i in range(threads)]
    want_c = idx.cal_distance_by_id(q[:threads], want_ids[:threads])
    errors = []

    def worker(t):
        try:
            mine = range(t, nq, threads)
            for i in mine:
                ids, dists = idx.knn_search(q[i], k, search)
                if not (np.array_equal(ids, want_ids[i]) and np.array_equal(dists, want_d[i])):
                    errors.append(("single", t, i))
            rows = np.array(list(mine))
            ids, dists = idx.knn_search_batch(q[rows], k, search)
            if not (np.array_equal(ids, want_ids[rows]) and np.array_equal(dists, want_d[rows])):
                errors.append(("batch", t))
            fid, fd = idx.knn_search(q[t], k, search, filter=flt)
            if not (np.array_equal(fid, want_f[t][0]) and np.array_equal(fd, want_f[t][1])):
                errors.append(("filter", t))
            if not np.array_equal(idx.cal_distance_by_id(q[t], want_ids[t]), want_c[t]):
                errors.append(("distance", t))
        except Exception as exc:  # noqa: BLE001
            errors.append(("raised", t, repr(exc)))

    pool = [threading.Thread(target=worker, args=(t,)) for t in range(threads)]
    for th in pool:
        th.start()
    for th in pool:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in pool)
    assert not errors, errors[:5]
    # The evaluator's loop natively (tools/eval/case/search_eval_case.cpp:233-277): sixteen caller threads, one query per
    # call; calls that meet are served as one device batch and must still return the single-query results, also with
    # another k and other parameters in between, and short rows (k above what a probe can return) as short rows.
    for t in (1, threads):
        ids, dists, seconds = idx.eval_knn_search(q, k, search, t)
        assert np.array_equal(ids, want_ids) and np.array_equal(dists, want_d) and seconds > 0
    ids3, dists3, _ = idx.eval_knn_search(q[:64], 3, search, threads)
    assert np.array_equal(ids3, want_ids[:64, :3]) and np.array_equal(dists3, want_d[:64, :3])
    one_i, one_d = idx.knn_search(q[5], k, search, statistics=False)
    assert np.array_equal(one_i, want_ids[5]) and np.array_equal(one_d, want_d[5])
    idx.close()
