"""Serialize / Deserialize of brute_force and ivf (Index::Serialize(std::ostream&), include/vsag/index.h:903-940) in the
reference's stream layout.  No file written by the reference exists offline, so the layout is checked field by field
against the reference's writers as read from its sources (flatten_datacell.h:481-486, basic_io.h:196-207,
quantizer.h:161-168, scalar_quantizer.cpp:199-204, sq8_uniform_quantizer.cpp:273-281, bucket_datacell.h:892-904,
ivf.cpp:990-1057, serialization.cpp:196-222) with an independent parser (numpy / struct / zlib), the codes against the
CPU checker's encoder, and the round trip against the index that was saved.  Parity with a reference-written file stays
unpinned."""
import json
import struct
import zlib

import os

import numpy as np
import pytest

import oracle as orc
from test_index_api_gpu import make, vectors
from vsag_amd import pyvsag

pytestmark = pytest.mark.gpu


class Cursor:
    def __init__(self, data, at=0):
        self.data, self.at = data, at

    def take(self, fmt):
        size = struct.calcsize("<" + fmt)
        out = struct.unpack_from("<" + fmt, self.data, self.at)
        self.at += size
        return out if len(out) > 1 else out[0]

    def array(self, dtype, count):
        out = np.frombuffer(self.data, dtype, count, self.at)
        self.at += out.nbytes
        return out

    def vector(self, dtype):
        return self.array(dtype, self.take("Q"))


def footer_of(data):
    """[magic][u64 len][json][u32 crc][u64 footer length][cigam]: the metadata and where the footer starts."""
    assert data[-8:] == b"0000gasv"
    length = struct.unpack_from("<Q", data, len(data) - 16)[0]
    start = len(data) - length
    assert data[start:start + 8] == b"vsag0000"
    mlen = struct.unpack_from("<Q", data, start + 8)[0]
    assert length == 8 + 8 + mlen + 4 + 8 + 8
    text = data[start + 16:start + 16 + mlen]
    assert struct.unpack_from("<I", data, start + 16 + mlen)[0] == zlib.crc32(text)
    return json.loads(text), start


def with_footer(body, metadata):
    text = json.dumps(metadata, separators=(",", ":")).encode()
    foot = b"vsag0000" + struct.pack("<Q", len(text)) + text + struct.pack("<I", zlib.crc32(text))
    return body + foot + struct.pack("<Q", len(foot) + 16) + b"0000gasv"


def same_results(a, b, q, k, search):
    a_ids, a_d = a.knn_search_batch(q, k, search)
    b_ids, b_d = b.knn_search_batch(q, k, search)
    return np.array_equal(a_ids, b_ids) and np.array_equal(a_d, b_d)


@pytest.mark.parametrize("metric", ["l2", "ip", "cosine"])
@pytest.mark.parametrize("quant", ["fp32", "sq8", "sq4", "sq8_uniform", "sq4_uniform", "rabitq"])
def test_brute_force_round_trip(lib, tmp_path, metric, quant):
    n, d, nq, k = 1500, 48, 20, 10
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 3 - 17
    a = make("brute_force", d, metric, base_quantization_type=quant)
    a.build(x, labels, n, d)
    path = tmp_path / "bf.index"
    a.serialize(path)
    b = make("brute_force", d, metric, base_quantization_type=quant)
    b.deserialize(path)
    assert b.get_num_elements() == n
    assert same_results(a, b, q, k, "{}")
    # the loaded index goes on like the saved one: same quantizer, same duplicates
    x2 = vectors(100, d, seed=9, normalize=False)
    l2 = np.concatenate([labels[:3], np.arange(97, dtype=np.int64) + 10 ** 6])
    assert a.add(x2, l2, 100, d) == 3 and b.add(x2, l2, 100, d) == 3
    assert same_results(a, b, q, k, "{}")
    with pytest.raises(pyvsag.VsagError) as e:
        b.deserialize(path)
    assert e.value.code == -6  # INDEX_NOT_EMPTY
    # a second save of the loaded index (before the add it would have been) has the same codes: save b, load into c
    path2 = tmp_path / "bf2.index"
    b.serialize(path2)
    c = make("brute_force", d, metric, base_quantization_type=quant)
    c.deserialize(path2)
    assert same_results(b, c, q, k, "{}")
    for idx in (a, b, c):
        idx.close()


def test_brute_force_sq8_layout_field_by_field(lib, tmp_path):
    n, d = 1000, 40
    x = vectors(n, d, normalize=False)
    labels = np.arange(n, dtype=np.int64) + 5
    idx = make("brute_force", d, "l2", base_quantization_type="sq8")
    idx.build(x, labels, n, d)
    path = tmp_path / "sq8.index"
    idx.serialize(path)
    data = path.read_bytes()
    meta, foot = footer_of(data)
    info = dict(meta["basic_info"])
    assert json.loads(info.pop("index_param"))["base_codes"]["quantization_params"] == {"type": "sq8"}
    assert info == {"dim": d, "extra_info_size": 0, "has_extra_info": False, "is_multi_vector": False, "total_count": n}
    c = Cursor(data)
    total, cap, code_size = c.take("III")  # FlattenInterface::Serialize
    assert (total, code_size) == (n, d) and cap >= n
    assert c.take("Q") == n * d  # BasicIO::Serialize: size, then the bytes
    codes = c.array(np.uint8, n * d).reshape(n, d)
    assert c.take("QiQB") == (d, 0, d, 1)  # Quantizer::Serialize: dim, metric, code size, trained
    diff = c.vector(np.float32)
    lower = c.vector(np.float32)
    assert diff.size == d and lower.size == d
    got_labels = c.vector(np.int64)  # LabelTable::Serialize
    assert np.array_equal(got_labels, labels) and c.at == foot
    # the bounds are the trained ones and the codes what the CPU checker encodes with them
    want_lower, want_diff = orc.sq_train(x, 8)
    assert np.array_equal(lower, want_lower) and np.array_equal(diff, want_diff)
    assert np.array_equal(codes, orc.sq_encode(x, 8, lower, diff, orc.L2))
    idx.close()


@pytest.mark.parametrize("metric", ["l2", "ip"])
def test_brute_force_sq8_uniform_layout(lib, tmp_path, metric):
    n, d = 800, 50  # 50 bytes of codes, aligned to 8 (l2: u64 sum of squares) or 4 (ip: f32 sum)
    x = vectors(n, d, normalize=False)
    idx = make("brute_force", d, metric, base_quantization_type="sq8_uniform")
    idx.build(x, np.arange(n, dtype=np.int64), n, d)
    path = tmp_path / "squ.index"
    idx.serialize(path)
    data = path.read_bytes()
    c = Cursor(data)
    behind = 56 if metric == "l2" else 52
    cs = behind + (8 if metric == "l2" else 4)
    assert c.take("III")[2] == cs and c.take("Q") == n * cs
    codes = c.array(np.uint8, n * cs).reshape(n, cs)
    assert c.take("QiQB") == (d, 0 if metric == "l2" else 1, cs, 1)
    diff, lower = c.take("ff")
    assert c.take("QQQ") == ((0, behind, 0) if metric == "l2" else (0, 0, behind))
    assert np.all(codes[:, d:behind] == 0)
    if metric == "l2":
        norms = codes[:, behind:].copy().view(np.uint64)[:, 0]
        assert np.array_equal(norms, (codes[:, :d].astype(np.uint64) ** 2).sum(1))
    want = orc.squ_encode(x, 8, lower, diff, orc.L2 if metric == "l2" else orc.IP)
    assert np.array_equal(codes, want)
    idx.close()


IVF_CASES = [
    ({"base_quantization_type": "sq8", "use_reorder": True, "precise_quantization_type": "fp32"}, "l2", 3.0),
    ({"base_quantization_type": "sq4_uniform", "use_reorder": True, "precise_quantization_type": "sq8"}, "ip", 4.0),
    ({"base_quantization_type": "sq8", "use_residual": True}, "l2", None),
    ({"base_quantization_type": "fp32", "buckets_per_data": 2}, "cosine", None),
    ({"base_quantization_type": "rabitq", "use_reorder": True, "precise_quantization_type": "fp32"}, "l2", 10.0),
    ({"base_quantization_type": "pqfs", "base_pq_dim": 16, "use_reorder": True, "precise_quantization_type": "fp32"},
     "l2", 5.0),
    ({"base_quantization_type": "pqfs", "base_pq_dim": 32, "use_residual": True}, "cosine", None),
    ({"base_quantization_type": "rabitq", "use_residual": True}, "l2", None),
]


@pytest.mark.parametrize("params,metric,factor", IVF_CASES)
def test_ivf_round_trip(lib, tmp_path, params, metric, factor):
    n, d, nq, k, nlist = 3000, 32, 30, 10, 16
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    labels = np.arange(n, dtype=np.int64) * 2 + 9
    full = dict(params, buckets_count=nlist, train_sample_count=3000)
    a = make("ivf", d, metric, **full)
    a.build(x, labels, n, d)
    search = json.dumps({"ivf": {"scan_buckets_count": 5, **({"factor": factor} if factor else {})}})
    path = tmp_path / "ivf.index"
    a.serialize(path)
    b = make("ivf", d, metric, **full)
    b.deserialize(path)
    assert b.get_num_elements() == n
    assert same_results(a, b, q, k, search)
    assert np.array_equal(a.cal_distance_by_id(q[:4], np.tile(labels[:6], (4, 1))),
                          b.cal_distance_by_id(q[:4], np.tile(labels[:6], (4, 1))))
    x2 = vectors(200, d, seed=9, normalize=False)
    l2 = np.arange(200, dtype=np.int64) + 10 ** 6
    assert a.add(x2, l2, 200, d) == 0 and b.add(x2, l2, 200, d) == 0
    assert same_results(a, b, q, k, search)
    # the cells tile the stream up to the footer
    data = path.read_bytes()
    meta, foot = footer_of(data)
    names = ["bucket", "partition_strategy", "label_table"] + (["reorder_codes"] if params.get("use_reorder") else [])
    at = 0
    for name in names:
        assert meta["datacell_offsets"][name] == at
        at += meta["datacell_sizes"][name]
    assert at == foot
    info = meta["basic_info"]
    assert (info["total_elements"], info["dim"], info["is_trained"], info["use_reorder"]) == \
        (n, d, True, bool(params.get("use_reorder")))
    a.close()
    b.close()


def test_ivf_bucket_cell_layout(lib, tmp_path):
    n, d, nlist = 2000, 24, 8
    x = vectors(n, d, normalize=False)
    labels = np.arange(n, dtype=np.int64)
    idx = make("ivf", d, "l2", buckets_count=nlist, train_sample_count=2000, base_quantization_type="sq8",
               use_residual=True)
    idx.build(x, labels, n, d)
    path = tmp_path / "ivf.index"
    idx.serialize(path)
    data = path.read_bytes()
    meta, _ = footer_of(data)
    c = Cursor(data, meta["datacell_offsets"]["bucket"])
    assert c.take("iI") == (nlist, d)  # BucketInterface::Serialize: bucket count, code size
    assert c.take("QiQB") == (d, 0, d, 1)
    diff, lower = c.vector(np.float32), c.vector(np.float32)
    seen, sizes, per_list = [], [], []
    for _ in range(nlist):
        size = c.take("Q")
        codes = c.array(np.uint8, size).reshape(-1, d)
        ids = c.vector(np.uint32)
        bias = c.vector(np.float32)  # residual lists carry a bias per code (l2)
        assert codes.shape[0] == ids.size == bias.size
        seen.append(ids)
        sizes.append(ids.size)
        per_list.append((codes, ids, bias))
    assert np.array_equal(c.vector(np.uint32), np.array(sizes, np.uint32))
    assert c.at == meta["datacell_offsets"]["bucket"] + meta["datacell_sizes"]["bucket"]
    assert np.array_equal(np.sort(np.concatenate(seen)), np.arange(n, dtype=np.uint32))
    # the partition cell: trained, bucket count, dim, then this index's tag and the centroids
    p = Cursor(data, meta["datacell_offsets"]["partition_strategy"])
    assert p.take("BiqQ") == (1, nlist, d, int.from_bytes(b"VSAGAMDR", "little"))
    centroids = p.vector(np.float32).reshape(nlist, d)
    # codes and bias of a list are those of x - centroid (bucket_datacell.h:594-639), by the CPU checker
    for l, (codes, ids, bias) in enumerate(per_list):
        res = orc.residual_rows(x[ids], np.full(ids.size, l, np.int32), centroids, orc.L2)
        want = orc.sq_encode(res, 8, lower, diff, orc.L2)
        assert np.array_equal(codes, want)
        want_bias = orc.residual_bias(orc.sq_decode(want, d, 8, lower, diff), np.full(ids.size, l, np.int32), centroids)
        np.testing.assert_allclose(bias, want_bias, rtol=1e-5, atol=1e-5)
    idx.close()


def test_ivf_reads_a_router_graph_image(lib, tmp_path):
    # The reference writes its router (an hgraph over the centroids) behind the partition header
    # (ivf_nearest_partition.cpp:150-153): label table, label -> inner id pairs, the flat cell of fp32 codes, then the
    # graph.  Of that image the labels and codes are read; here one is put together with the codes in another order.
    n, d, nq, k, nlist = 2500, 16, 20, 10, 12
    x = vectors(n, d, normalize=False)
    q = vectors(nq, d, seed=165, normalize=False)
    a = make("ivf", d, "l2", buckets_count=nlist, train_sample_count=2500, base_quantization_type="sq8")
    a.build(x, np.arange(n, dtype=np.int64), n, d)
    path = tmp_path / "ivf.index"
    a.serialize(path)
    data = path.read_bytes()
    meta, foot = footer_of(data)
    off, size = meta["datacell_offsets"]["partition_strategy"], meta["datacell_sizes"]["partition_strategy"]
    cell = Cursor(data, off)
    head = data[off:off + 13]
    cell.at += 13 + 8
    centroids = cell.vector(np.float32).reshape(nlist, d)
    order = np.random.Generator(np.random.MT19937(3)).permutation(nlist)  # inner id i of the graph holds bucket order[i]
    image = struct.pack("<Q", nlist) + order.astype(np.int64).tobytes()
    image += struct.pack("<Q", nlist) + b"".join(struct.pack("<qI", int(b), i) for i, b in enumerate(order))
    image += struct.pack("<IIIQ", nlist, 800, 4 * d, 800 * 4 * d) + centroids[order].tobytes() + bytes((800 - nlist) * 4 * d)
    image += struct.pack("<QiQB", d, 0, 4 * d, 1) + b"graph, route graphs and the router's own footer follow" * 7
    new_cell = head + image
    body = data[:off] + new_cell + data[off + size:foot]
    shift = len(new_cell) - size
    meta["datacell_sizes"]["partition_strategy"] = len(new_cell)
    for name, at in meta["datacell_offsets"].items():
        if at > off:
            meta["datacell_offsets"][name] = at + shift
    other = tmp_path / "ivf_ref_router.index"
    other.write_bytes(with_footer(body, meta))
    b = make("ivf", d, "l2", buckets_count=nlist, train_sample_count=2500, base_quantization_type="sq8")
    b.deserialize(other)
    assert same_results(a, b, q, k, json.dumps({"ivf": {"scan_buckets_count": 3}}))
    a.close()
    b.close()


def test_brute_force_reads_the_form_without_a_footer(lib, tmp_path):
    # bruteforce.cpp:1008-1016: dim and count first, then the cells
    n, d = 600, 20
    x = vectors(n, d)
    a = make("brute_force", d, "l2", base_quantization_type="sq8")
    a.build(x, np.arange(n, dtype=np.int64), n, d)
    path = tmp_path / "bf.index"
    a.serialize(path)
    data = path.read_bytes()
    _, foot = footer_of(data)
    old = tmp_path / "bf_old.index"
    old.write_bytes(struct.pack("<qQ", d, n) + data[:foot])
    b = make("brute_force", d, "l2", base_quantization_type="sq8")
    b.deserialize(old)
    assert same_results(a, b, x[:10], 5, "{}")
    a.close()
    b.close()


def test_deserialize_errors(lib, tmp_path):
    n, d = 500, 16
    x = vectors(n, d)
    a = make("brute_force", d, "l2", base_quantization_type="sq8")
    a.build(x, np.arange(n, dtype=np.int64), n, d)
    path = tmp_path / "bf.index"
    a.serialize(path)
    data = path.read_bytes()
    with pytest.raises(pyvsag.VsagError) as e:
        make("brute_force", d, "l2", base_quantization_type="sq8").deserialize(tmp_path / "missing.index")
    assert e.value.code == -13
    with pytest.raises(pyvsag.VsagError) as e:
        make("brute_force", d + 4, "l2", base_quantization_type="sq8").deserialize(path)
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        make("brute_force", d, "l2", base_quantization_type="sq4").deserialize(path)
    assert e.value.code == -3
    with pytest.raises(pyvsag.VsagError) as e:
        make("brute_force", d, "ip", base_quantization_type="sq8").deserialize(path)
    assert e.value.code == -3
    cut = tmp_path / "cut.index"
    cut.write_bytes(data[:len(data) // 2])
    with pytest.raises(pyvsag.VsagError) as e:
        make("brute_force", d, "l2", base_quantization_type="sq8").deserialize(cut)
    assert e.value.code in (-3, -12, -14)
    # a flipped bit in the metadata: the checksum no longer matches, the footer is not taken for one
    meta, foot = footer_of(data)
    bad = bytearray(data)
    bad[foot + 20] ^= 1
    broken = tmp_path / "crc.index"
    broken.write_bytes(bytes(bad))
    with pytest.raises(pyvsag.VsagError):
        make("brute_force", d, "l2", base_quantization_type="sq8").deserialize(broken)
    with pytest.raises(pyvsag.VsagError) as e:
        make("ivf", d, "l2", buckets_count=4).deserialize(path)
    assert e.value.code in (-3, -14)
    # an empty index writes a file too; it loads as an empty index
    empty = make("brute_force", d, "l2")
    empty.serialize(tmp_path / "empty.index")
    fresh = make("brute_force", d, "l2")
    fresh.deserialize(tmp_path / "empty.index")
    assert fresh.get_num_elements() == 0
    # a device that takes no bytes: the write (at the latest the closing flush) fails, and the call says so
    if os.path.exists("/dev/full"):
        with pytest.raises(pyvsag.VsagError):
            a.serialize("/dev/full")
    a.close()


def test_ivf_pqfs_bucket_cell_holds_packaged_blocks(lib, tmp_path):
    """A pqfs bucket is serialized as BucketDataCell keeps it (package_fastscan, bucket_datacell.h:943-966): whole
    blocks of 32 codes in the fast-scan order of PQFastScanQuantizer::Package32; the quantizer writes pq_dim, the
    subspace dimension and the codebooks (pq_fastscan_quantizer.cpp:201-207)."""
    n, d, nlist, pq_dim = 1500, 24, 6, 12
    x = vectors(n, d, normalize=False)
    labels = np.arange(n, dtype=np.int64)
    idx = make("ivf", d, "l2", buckets_count=nlist, train_sample_count=1500, base_quantization_type="pqfs",
               base_pq_dim=pq_dim)
    idx.build(x, labels, n, d)
    path = tmp_path / "ivf.index"
    idx.serialize(path)
    data = path.read_bytes()
    meta, _ = footer_of(data)
    cs = pq_dim // 2
    c = Cursor(data, meta["datacell_offsets"]["bucket"])
    assert c.take("iI") == (nlist, cs)
    assert c.take("QiQB") == (d, 0, cs, 1)
    assert c.take("qq") == (pq_dim, d // pq_dim)
    cb = c.vector(np.float32).reshape(pq_dim, 16, d // pq_dim)
    seen = []
    for _ in range(nlist):
        size = c.take("Q")
        packaged = c.array(np.uint8, size)
        ids = c.vector(np.uint32)
        assert size == (ids.size + 31) // 32 * 32 * cs
        want = orc.pq_encode(x[ids], pq_dim, cb, orc.L2)
        for b in range(0, ids.size, 32):
            blk = np.zeros((32, cs), np.uint8)
            blk[:min(32, ids.size - b)] = want[b:b + 32]
            assert np.array_equal(packaged[b * cs:(b + 32) * cs], orc.pqfs_package32(blk, pq_dim, valid=min(32, ids.size - b)))
        seen.append(ids)
    assert np.array_equal(np.sort(np.concatenate(seen)), np.arange(n, dtype=np.uint32))
    idx.close()


def _reparam(data, edit):
    """The same stream with its index_param edited (edit(dict) -> dict or None to drop it) and the footer rewritten."""
    meta, start = footer_of(data)
    info = meta["basic_info"]
    param = edit(json.loads(info["index_param"]))
    if param is None:
        del info["index_param"]
    else:
        info["index_param"] = json.dumps(param, separators=(",", ":"))
    return with_footer(data[:start], meta)


def test_index_param_in_the_footer_and_its_compatibility_check(lib, tmp_path):
    """basic_info carries index_param, the creating parameters in the reference's internal form (ivf.cpp:1045,
    bruteforce.cpp:703); a reader refuses a file whose parameters its own are not compatible with
    (ivf.cpp:1201-1208 with IVFParameter::CheckCompatibility, ivf_parameter.cpp:133-148; bruteforce.cpp:887-891) and
    reads a file without the field (older writers)."""
    n, d = 1500, 32
    x = vectors(n, d)
    labels = np.arange(n, dtype=np.int64)
    params = dict(buckets_count=10, base_quantization_type="sq8", use_reorder=True, precise_quantization_type="fp32",
                  train_sample_count=1500)
    a = make("ivf", d, "l2", **params)
    a.build(x, labels, n, d)
    path = tmp_path / "ivf.index"
    a.serialize(path)
    data = path.read_bytes()
    meta, _ = footer_of(data)
    p = json.loads(meta["basic_info"]["index_param"])
    assert p["type"] == "ivf" and p["use_reorder"] is True and p["reorder_source"] == "precise"
    assert p["buckets_params"] == {"buckets_count": 10, "io_params": {"type": "memory_io"},
                                   "quantization_params": {"type": "sq8"}, "use_residual": False}
    assert p["precise_codes"]["quantization_params"] == {"type": "fp32"} and p["precise_codes"]["codes_type"] == "flatten"
    assert p["partition_strategy"]["partition_strategy_type"] == "ivf" and p["partition_strategy"]["ivf_train_type"] == "kmeans"
    assert p["precise_codes_layout"] == "flat" and p["buckets_per_data"] == 1 and p["graph_build_threshold"] == 0
    q = vectors(10, d, seed=3)
    search = json.dumps({"ivf": {"scan_buckets_count": 10, "factor": 2.0}})

    def load(blob, **override):
        f = tmp_path / "edited.index"
        f.write_bytes(blob)
        b = make("ivf", d, "l2", **{**params, **override})
        try:
            b.deserialize(f)
            return b
        except pyvsag.VsagError:
            b.close()
            raise

    # unchanged, and without the field: read
    for blob in (data, _reparam(data, lambda p: None)):
        b = load(blob)
        assert same_results(a, b, q, 5, search)
        b.close()
    # every field the reference compares, one at a time
    def edited(path_keys, value):
        def edit(p):
            node = p
            for key in path_keys[:-1]:
                node = node[key]
            node[path_keys[-1]] = value
            return p
        return _reparam(data, edit)
    for keys, value in ((("buckets_params", "quantization_params", "type"), "sq4"), (("buckets_params", "buckets_count"), 11),
                        (("buckets_params", "use_residual"), True), (("precise_codes", "quantization_params", "type"), "sq8"),
                        (("use_reorder",), False), (("reorder_source",), "base"), (("use_attribute_filter",), True),
                        (("label_remap_type",), "robin"), (("precise_codes_layout",), "bucket"), (("buckets_per_data",), 2),
                        (("graph_build_threshold",), 100), (("partition_strategy", "partition_strategy_type"), "gno_imi"),
                        (("partition_strategy", "route_max_degree"), 32)):
        with pytest.raises(pyvsag.VsagError) as e:
            load(edited(keys, value))
        assert e.value.code == -3 and "IVF index parameter not match, current: " in e.value.message, (keys, e.value.message)
    # fields it does not compare do not matter
    for keys, value in ((("train_sample_count",), 99999), (("build_thread_count",), 8),
                        (("partition_strategy", "ivf_train_type"), "random")):
        load(edited(keys, value)).close()
    a.close()

    # quantizer fields: rabitq bits, pq_dim
    r = make("ivf", d, "l2", buckets_count=4, base_quantization_type="rabitq", rabitq_bits_per_dim_base=4, train_sample_count=1500)
    r.build(x, labels, n, d)
    r.serialize(tmp_path / "rabitq.index")
    rp = json.loads(footer_of((tmp_path / "rabitq.index").read_bytes())[0]["basic_info"]["index_param"])
    assert rp["buckets_params"]["quantization_params"]["rabitq_bits_per_dim_base"] == 4
    assert rp["buckets_params"]["quantization_params"]["rabitq_bits_per_dim_query"] == 32
    with pytest.raises(pyvsag.VsagError) as e:
        make("ivf", d, "l2", buckets_count=4, base_quantization_type="rabitq", rabitq_bits_per_dim_base=2,
             train_sample_count=1500).deserialize(tmp_path / "rabitq.index")
    assert e.value.code == -3 and "parameter not match" in e.value.message
    r.close()

    # brute force
    bf = make("brute_force", d, "l2", base_quantization_type="sq8")
    bf.build(x, labels, n, d)
    bf.serialize(tmp_path / "bf.index")
    bdata = (tmp_path / "bf.index").read_bytes()
    bp = json.loads(footer_of(bdata)[0]["basic_info"]["index_param"])
    assert bp["type"] == "brute_force" and bp["base_codes"]["quantization_params"] == {"type": "sq8"}
    (tmp_path / "bf_sq4.index").write_bytes(_reparam(bdata, lambda p: {**p, "base_codes": {**p["base_codes"],
                                                                                             "quantization_params": {"type": "sq4"}}}))
    with pytest.raises(pyvsag.VsagError) as e:
        make("brute_force", d, "l2", base_quantization_type="sq8").deserialize(tmp_path / "bf_sq4.index")
    assert e.value.code == -3 and "BruteForce index parameter not match" in e.value.message
    (tmp_path / "bf_plain.index").write_bytes(_reparam(bdata, lambda p: None))
    c = make("brute_force", d, "l2", base_quantization_type="sq8")
    c.deserialize(tmp_path / "bf_plain.index")
    assert c.get_num_elements() == n
    c.close()
    bf.close()
