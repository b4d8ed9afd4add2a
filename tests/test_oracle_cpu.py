"""Pins the CPU checker (oracle/) itself, on the CPU:
  * against the known answers the reference's own unit tests hold (cited per test),
  * against the reference's scalar kernels compiled from its sources (oracle/_ref, when built),
  * against closed forms / brute force chosen so that a dropped term, a wrong index or a swapped operand fails.
The same vectors are committed under tests/golden/ so that the checks also run where the reference sources
are not mounted."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# get_common_used_dims() of the reference fixtures (tests/fixtures/core/common.cpp:59-65)
DIMS = [7, 8, 9, 32, 33, 48, 64, 65, 70, 96, 97, 109, 128, 129, 160, 161, 192, 193, 224, 225, 256, 512, 784, 960,
        1024, 1536]


# ------------------------------------------------------------------ reference known answers
def test_sq8_sq4_nan_and_half_known_answers():
    # scalar_quantizer_test.cpp:101-135: train on {0,0},{1,1}; encode {NaN, 0.5}
    train = np.array([[0, 0], [1, 1]], np.float32)
    query = np.array([[np.nan, 0.5]], np.float32)
    lb, diff = orc.sq_train(train, 8)
    assert np.array_equal(lb, [0, 0]) and np.array_equal(diff, [1, 1])
    c8 = orc.sq_encode(query, 8, lb, diff)
    assert c8[0, 0] == 0 and c8[0, 1] == int(np.float32(255.0) * np.float32(0.5)) == 127
    dec = orc.sq_decode(c8, 2, 8, lb, diff)
    assert abs(dec[0, 0]) <= 1e-6 and abs(dec[0, 1] - 127.0 / 255.0) <= 1e-6
    lb4, diff4 = orc.sq_train(train, 4)
    c4 = orc.sq_encode(query, 4, lb4, diff4)
    assert (c4[0, 0] & 0x0F) == 0 and ((c4[0, 0] >> 4) & 0x0F) == 7
    dec = orc.sq_decode(c4, 2, 4, lb4, diff4)
    assert abs(dec[0, 0]) <= 1e-6 and abs(dec[0, 1] - 7.0 / 15.0) <= 1e-6


def test_sq4_uniform_byte_images():
    # rabitq_quantizer_test.cpp:1012-1024: trunc_rate 0, one training vector, IP layout [nibbles|sum|code sum]
    data = np.array([[1, 2, 4, 8, 15, 0]], np.float32)
    lb, diff = orc.sq_train_uniform(data, 4, orc.IP, mode=3, trunc_rate=0.0)
    assert lb == 0 and diff == 15
    code = orc.squ_encode(data, 4, lb, diff, orc.IP)[0]
    assert code.shape[0] == 4 + 4 + 4
    assert bytes(code[:3]) == bytes([0x21, 0x84, 0x0F])
    assert abs(code[4:8].view(np.float32)[0] - 30) < 1e-5 and abs(code[8:12].view(np.float32)[0] - 30) < 1e-5
    # :1069-1081, dim 15
    data = np.array([[1, 2, 4, 8, 0, 3, 11, 15, 9, 13, 10, 6, 7, 12, 14]], np.float32)
    lb, diff = orc.sq_train_uniform(data, 4, orc.IP, mode=3, trunc_rate=0.0)
    code = orc.squ_encode(data, 4, lb, diff, orc.IP)[0]
    assert bytes(code[:8]) == bytes([0x21, 0x84, 0x30, 0xFB, 0xD9, 0x6A, 0xC7, 0x0E])


def test_uniform_zero_range_gives_zero_codes():
    # sq4_uniform_quantizer_test.cpp:82, sq8_uniform_quantizer_test.cpp:51
    data = np.full((10, 12), 0.25, np.float32)
    for bits in (4, 8):
        lb, diff = orc.sq_train_uniform(data, bits, orc.L2, mode=3 if bits == 4 else 1)
        assert diff == 0
        codes = orc.squ_encode(data, bits, lb, diff, orc.L2)
        assert not codes.any()


def test_rabitq_query_sq_and_planes_known_answers():
    # rabitq_quantizer_test.cpp:1126-1175 (dim 6) and :1190-1243 (dim 15): EncodeSQ keeps integer inputs,
    # ReOrderSQ puts bit b of every dim into plane b, planes 64 bytes apart.
    quant, ub, lb, delta, qsum = orc.rabitq_encode_sq(np.array([1, 2, 4, 8, 15, 0], np.float32))
    assert list(quant) == [1, 2, 4, 8, 15, 0] and lb == 0 and ub == 15 and delta == 1 and qsum == 30
    planes, pb = orc.rabitq_reorder_sq(quant)
    assert pb == 64
    expect = np.zeros(256, np.uint8)
    expect[0], expect[64], expect[128], expect[192] = 0x11, 0x12, 0x14, 0x18
    assert np.array_equal(planes, expect)
    data15 = np.array([1, 2, 4, 8, 0, 3, 11, 15, 9, 13, 10, 6, 7, 12, 14], np.float32)
    quant, *_ = orc.rabitq_encode_sq(data15)
    assert list(quant) == list(data15.astype(np.uint8))
    planes, pb = orc.rabitq_reorder_sq(quant)
    expect = np.zeros(256, np.uint8)
    expect[0:2] = [0xE1, 0x13]
    expect[64:66] = [0xE2, 0x5C]
    expect[128:130] = [0x84, 0x7A]
    expect[192:194] = [0xC8, 0x67]
    assert np.array_equal(planes, expect)
    # :1245-1272: an all-equal vector has delta 0 -> all-zero codes
    quant, ub, lb, delta, qsum = orc.rabitq_encode_sq(np.full(9, 0.5, np.float32))
    assert delta == 0 and not quant.any() and qsum == 0


def test_rabitq_binary_ip_known_answers():
    # simd/rabitq_simd_test.cpp:118-144
    codes = np.zeros(64, np.uint8)
    codes[:8] = [0xFF, 0xFF, 0x0F, 0x0F, 0xF0, 0xF0, 0x00, 0x00]
    bits = np.zeros(64, np.uint8)
    bits[:2] = [0xAA, 0x55]
    L = orc.lib()
    for dim in range(17):
        r = L.orc_rabitq_sq4u_binary_ip(codes.ctypes.data_as(C.c_void_p), bits.ctypes.data_as(C.c_void_p),
                                        C.c_uint64(dim))
        assert r == (0 if dim == 0 else 36 if dim <= 8 else 32), (dim, r)


def test_code_sizes_of_the_benchmark_configs():
    # the arithmetic of the constructors: sq4_uniform_quantizer.cpp:33-72 (d=128, l2 -> 64+8),
    # rabitq_quantizer.cpp:102-133 (d=768, ip, 4-bit query -> 96 + 4*4), query 4 planes of 128 B + 5 floats.
    assert orc.squ_code_size(128, 4, orc.L2) == 72
    assert orc.squ_code_size(128, 8, orc.L2) == 136 and orc.squ_code_size(128, 8, orc.IP) == 132
    assert orc.squ_code_size(6, 4, orc.IP) == 12 and orc.squ_code_size(15, 4, orc.IP) == 16
    assert orc.rabitq_code_size(768, orc.IP) == 112 and orc.rabitq_code_size(768, orc.L2) == 108
    assert orc.rabitq_query_code_size(768, orc.IP) == 4 * 128 + 20


# ------------------------------------------------------------------ compiled reference kernels
def _vec_cases():
    rng = np.random.default_rng(47)
    for d in DIMS:
        q = rng.uniform(0.1, 0.9, d).astype(np.float32)
        x = rng.uniform(0.1, 0.9, d).astype(np.float32)
        lb = rng.uniform(-0.2, 0.1, d).astype(np.float32)
        diff = rng.uniform(0.5, 1.5, d).astype(np.float32)
        c8 = rng.integers(0, 256, d).astype(np.uint8)
        c8b = rng.integers(0, 256, d).astype(np.uint8)
        c4 = rng.integers(0, 256, (d + 1) // 2).astype(np.uint8)
        c4b = rng.integers(0, 256, (d + 1) // 2).astype(np.uint8)
        if d % 2:
            c4[-1] &= 0x0F
            c4b[-1] &= 0x0F
        yield d, q, x, lb, diff, c8, c8b, c4, c4b


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _primitive_values(fns):
    """name -> list of values over DIMS, computed with `fns` (oracle or reference symbols)."""
    out = {}
    for d, q, x, lb, diff, c8, c8b, c4, c4b in _vec_cases():
        n = C.c_uint64(d)
        vals = {
            "fp32_ip": fns["fp32_ip"](_p(q), _p(x), n),
            "fp32_l2": fns["fp32_l2"](_p(q), _p(x), n),
            "sq8_ip": fns["sq8_ip"](_p(q), _p(c8), _p(lb), _p(diff), n),
            "sq8_l2": fns["sq8_l2"](_p(q), _p(c8), _p(lb), _p(diff), n),
            "sq4_ip": fns["sq4_ip"](_p(q), _p(c4), _p(lb), _p(diff), n),
            "sq4_l2": fns["sq4_l2"](_p(q), _p(c4), _p(lb), _p(diff), n),
            "sq4u_ip": float(fns["sq4u_ip"](_p(c4), _p(c4b), n)),
            "sq8u_ip": float(fns["sq8u_ip"](_p(c8), _p(c8b), n)),
        }
        for k, v in vals.items():
            out.setdefault(k, []).append(float(v))
    return out


def _oracle_fns():
    L = orc.lib()
    L.orc_sq4u_codes_ip.restype = C.c_int32
    L.orc_sq8u_codes_ip.restype = C.c_int32
    return {"fp32_ip": L.orc_fp32_ip, "fp32_l2": L.orc_fp32_l2sqr, "sq8_ip": L.orc_sq8_ip, "sq8_l2": L.orc_sq8_l2sqr,
            "sq4_ip": L.orc_sq4_ip, "sq4_l2": L.orc_sq4_l2sqr, "sq4u_ip": L.orc_sq4u_codes_ip,
            "sq8u_ip": L.orc_sq8u_codes_ip}


def test_primitives_match_compiled_reference_kernels():
    ref = orc.ref()
    if ref is None:
        pytest.skip("oracle/_ref is not built (reference sources not mounted)")
    rfns = {"fp32_ip": ref["FP32ComputeIP"], "fp32_l2": ref["FP32ComputeL2Sqr"], "sq8_ip": ref["SQ8ComputeIP"],
            "sq8_l2": ref["SQ8ComputeL2Sqr"], "sq4_ip": ref["SQ4ComputeIP"], "sq4_l2": ref["SQ4ComputeL2Sqr"],
            "sq4u_ip": ref["SQ4UniformComputeCodesIP"], "sq8u_ip": ref["SQ8UniformComputeCodesIP"]}
    a, b = _primitive_values(_oracle_fns()), _primitive_values(rfns)
    for name in a:
        va, vb = np.array(a[name]), np.array(b[name])
        if name.endswith("u_ip"):
            assert np.array_equal(va, vb), name
        else:
            # same scalar arithmetic; the reference build may contract a*b+c into an fma
            assert np.allclose(va, vb, rtol=2e-6, atol=1e-6), (name, np.abs(va - vb).max())


def test_primitives_match_committed_golden_vectors():
    """tests/golden/simd_generic.json holds the values of vsag::generic::* on the seeded vectors above
    (written by tests/golden/make_simd_golden.py from the compiled reference)."""
    path = os.path.join(GOLDEN, "simd_generic.json")
    gold = json.load(open(path))
    a = _primitive_values(_oracle_fns())
    for name, vals in gold["values"].items():
        va, vb = np.array(a[name]), np.array(vals)
        if name.endswith("u_ip"):
            assert np.array_equal(va, vb), name
        else:
            assert np.allclose(va, vb, rtol=2e-6, atol=1e-6), (name, np.abs(va - vb).max())


def test_rabitq_bit_kernels_match_reference():
    ref = orc.ref()
    if ref is None:
        pytest.skip("oracle/_ref is not built (reference sources not mounted)")
    rng = np.random.default_rng(165)
    L = orc.lib()
    for d in DIMS:
        nb = (d + 7) // 8
        planes = rng.integers(0, 256, 4 * nb).astype(np.uint8)
        bits = rng.integers(0, 256, nb).astype(np.uint8)
        if d % 8:  # the kernels require zero padding bits
            mask = (1 << (d % 8)) - 1
            bits[-1] &= mask
            for b in range(4):
                planes[b * nb + nb - 1] &= mask
        assert L.orc_rabitq_sq4u_binary_ip(_p(planes), _p(bits), C.c_uint64(d)) == \
            ref["RaBitQSQ4UBinaryIP"](_p(planes), _p(bits), C.c_uint64(d))
        v = rng.standard_normal(d).astype(np.float32)
        inv = C.c_float(1.0 / np.sqrt(np.float32(d)))
        a = L.orc_rabitq_float_binary_ip(_p(v), _p(bits), C.c_uint64(d), inv)
        b = ref["RaBitQFloatBinaryIP"](_p(v), _p(bits), C.c_uint64(d), inv)
        assert abs(a - b) <= 2e-6 * max(1.0, abs(b))
        cen = rng.standard_normal(d).astype(np.float32)
        o1, o2 = np.empty(d, np.float32), np.empty(d, np.float32)
        n1 = L.orc_normalize_with_centroid(_p(v), _p(cen), _p(o1), C.c_uint64(d))
        n2 = ref["NormalizeWithCentroid"](_p(v), _p(cen), _p(o2), C.c_uint64(d))
        assert abs(n1 - n2) <= 2e-6 * n2 and np.allclose(o1, o2, rtol=2e-6, atol=1e-7)


def test_rabitq_multibit_kernels_match_reference():
    """The bit-plane inner product against the reference's compiled RaBitQFloatSplitCodeIP (generic.cpp:743-771, as
    RaBitQFloatSQIPByPlanes calls it: top plane = one-bit code, lower planes = supplement) and RaBitQFloatSQIP
    (:799-811) on the unpacked codes: the two agree by construction in the reference, and so must the restatements."""
    ref = orc.ref()
    if ref is None:
        pytest.skip("oracle/_ref is not built (reference sources not mounted)")
    rng = np.random.default_rng(744)
    for d in DIMS:
        nb = (d + 7) // 8
        v = rng.standard_normal(d).astype(np.float32)
        for bits in (2, 3, 4, 5, 8):
            scalar = rng.integers(0, 1 << bits, d).astype(np.uint8)
            planes = orc.rabitq_pack_planes(scalar, bits)
            # plane b holds bit b of every dimension
            for b in range(bits):
                want = np.packbits((scalar >> b) & 1, bitorder="little")
                assert np.array_equal(planes[b * nb:(b + 1) * nb], want)
            mine = orc.rabitq_float_planes_ip(v, planes, bits)
            one_bit = np.ascontiguousarray(planes[(bits - 1) * nb:])
            theirs = ref["RaBitQFloatSplitCodeIP"](_p(v), _p(one_bit), _p(planes), C.c_uint64(d), C.c_uint32(bits - 1))
            assert mine == theirs
            sq_mine = orc.rabitq_float_sq_ip(v, scalar)
            sq_theirs = ref["RaBitQFloatSQIP"](_p(v), _p(scalar), C.c_uint64(d))
            assert sq_mine == sq_theirs == mine


# ------------------------------------------------------------------ closed forms and brute force
def test_popcount_identity_of_the_binary_ip():
    # sum_b 2^b popcount(plane_b & bits) == sum over set bits of the 4-bit code
    rng = np.random.default_rng(1)
    L = orc.lib()
    for d in (6, 15, 64, 127, 768):
        code = rng.integers(0, 16, d).astype(np.uint8)
        bit = rng.integers(0, 2, d).astype(np.uint8)
        planes, pb = orc.rabitq_reorder_sq(code)
        bits = np.zeros(pb, np.uint8)
        for i in range(d):
            bits[i // 8] |= bit[i] << (i % 8)
        got = L.orc_rabitq_sq4u_binary_ip(_p(planes), _p(bits), C.c_uint64(pb * 8))
        assert got == int((code.astype(np.int64) * bit).sum())


def test_sq_train_is_the_order_statistic():
    rng = np.random.default_rng(2)
    for n, d, bits, rate in [(5000, 5, 8, 0.001), (5000, 5, 4, 0.05), (120000, 3, 8, 0.001), (10, 2, 4, 0.05)]:
        x = rng.standard_normal((n, d)).astype(np.float32)
        x[:, 0] = np.round(x[:, 0] * 3) / 3
        lb, diff = orc.sq_train(x, bits, trunc_rate=rate)
        if n <= 100000:
            sample = x
        else:
            step = 2147483647 % n
            sample = x[(np.arange(100000, dtype=np.int64) * step) % n]
        cnt = sample.shape[0]
        ignore = max(1, int((cnt - 1) * (rate if bits == 4 else 0.001)))
        s = np.sort(sample, axis=0)
        assert np.array_equal(lb, s[ignore - 1]) and np.array_equal(lb + diff, (s[cnt - ignore] - lb) + lb)
        assert np.array_equal(diff, s[cnt - ignore] - s[ignore - 1])
    # uniform: TRUNC_BOUND takes min of uppers / max of lowers; CLASSIC the global extremes
    x = rng.random((3000, 6), dtype=np.float32)
    lb, diff = orc.sq_train_uniform(x, 8, mode=1)
    assert lb == x.min() and np.float32(lb + diff) == np.float32(x.min() + (x.max() - x.min()))
    lb4, diff4 = orc.sq_train_uniform(x, 4, mode=3, trunc_rate=0.05)
    s = np.sort(x, axis=0)
    ignore = int(2999 * 0.05)
    assert lb4 == s[ignore - 1].max() and diff4 == np.float32(s[3000 - ignore].min() - s[ignore - 1].max())


def test_sq_codes_round_trip_on_the_integer_grid():
    # quantizer_test.h:134-175: values on the code grid come back exactly
    rng = np.random.default_rng(3)
    for bits in (8, 4):
        levels = (1 << bits) - 1
        d = 40
        grid = rng.integers(0, levels + 1, (200, d)).astype(np.float32)
        lb = np.zeros(d, np.float32)
        diff = np.full(d, levels, np.float32)
        codes = orc.sq_encode(grid, bits, lb, diff)
        dec = orc.sq_decode(codes, d, bits, lb, diff)
        # delta > 0.999 is clamped to 1 (scalar_quantization_utils.h:19-30): the top level maps to itself too
        assert np.array_equal(dec, grid)


def test_sq_distance_is_distance_to_the_decoded_vector():
    rng = np.random.default_rng(4)
    d, n = 96, 50
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((3, d), dtype=np.float32)
    for bits, kind in ((8, orc.SQ8), (4, orc.SQ4)):
        lb, diff = orc.sq_train(x, bits)
        codes = orc.sq_encode(x, bits, lb, diff)
        dec = orc.sq_decode(codes, d, bits, lb, diff).astype(np.float64)
        l2 = orc.flat_dists(kind, orc.L2, d, codes, q, lb=lb, diff=diff)
        ip = orc.flat_dists(kind, orc.IP, d, codes, q, lb=lb, diff=diff)
        assert np.allclose(l2, ((q[:, None, :].astype(np.float64) - dec[None]) ** 2).sum(2), rtol=1e-5)
        assert np.allclose(ip, 1.0 - q.astype(np.float64) @ dec.T, rtol=1e-5, atol=1e-5)


def test_uniform_l2_closed_form_and_ip_quirk():
    rng = np.random.default_rng(5)
    d, n = 33, 40
    x = rng.random((n, d), dtype=np.float32)
    for bits, kind in ((4, orc.SQ4U), (8, orc.SQ8U)):
        levels = (1 << bits) - 1
        lb, diff = orc.sq_train_uniform(x, bits, orc.L2, mode=3 if bits == 4 else 1)
        codes = orc.squ_encode(x, bits, lb, diff, orc.L2)
        dists = orc.flat_dists(kind, orc.L2, d, codes, codes[:5], lb=lb, diff=diff)
        # integer codes: unpack and compare with (n1 + n2 - 2 ip) (diff / L)^2
        if bits == 4:
            raw = np.zeros((n, d), np.int64)
            for i in range(d):
                raw[:, i] = (codes[:, i // 2] >> (4 * (i % 2))) & 0xF
        else:
            raw = codes[:, :d].astype(np.int64)
        norms = codes[:, -8:].view(np.uint64)[:, 0].astype(np.int64)
        assert np.array_equal(norms, (raw ** 2).sum(1))
        expect = ((raw[:5, None, :] - raw[None]) ** 2).sum(2) * (float(diff) / levels) ** 2
        assert np.allclose(dists, expect, rtol=1e-5, atol=1e-7)
        assert np.allclose(np.diag(dists[:, :5]), 0, atol=1e-7)
        # IP keeps the reference's form lb (sum_q + sum_o) + rate <c_q, c_o> + lb^2 with raw-value sums
        codes_ip = orc.squ_encode(x, bits, lb, diff, orc.IP)
        got = orc.flat_dists(kind, orc.IP, d, codes_ip, codes_ip[:5], lb=lb, diff=diff)
        sums = x.astype(np.float64).sum(1)
        rate = (float(diff) / levels) ** 2
        expect = 1.0 - (lb * (sums[:5, None] + sums[None]) + rate * (raw[:5] @ raw.T) + float(lb) ** 2)
        assert np.allclose(got, expect, rtol=1e-4, atol=1e-4)


def _rotation(rng, d):
    q, r = np.linalg.qr(rng.standard_normal((d, d)))
    return (q * np.sign(np.diag(r))).astype(np.float32)


def test_rabitq_encode_invariants_and_estimator():
    rng = np.random.default_rng(6)
    d, n = 128, 400
    x = rng.standard_normal((n, d)).astype(np.float32)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    assert np.allclose(cen, rot.astype(np.float64) @ x.astype(np.float64).mean(0), atol=1e-5)
    codes = orc.rabitq_encode(x, rot, cen, orc.IP)
    nb = d // 8
    y = (x.astype(np.float64) @ rot.astype(np.float64).T) - cen
    norm = np.linalg.norm(y, axis=1)
    o = y / norm[:, None]
    bits = np.unpackbits(codes[:, :nb], axis=1, bitorder="little")[:, :d]
    near_zero = np.abs(o) < 1e-6
    assert np.all((bits == (o >= 0)) | near_zero)
    f = codes[:, nb:].view(np.float32)  # norm, error, sum, raw norm
    assert np.allclose(f[:, 0], norm, rtol=1e-5)
    assert np.allclose(f[:, 1], np.abs(o).sum(1) / np.sqrt(d), rtol=1e-4)  # error = <o_bar, o> = sum|o_d| / sqrt(d)
    assert np.array_equal(f[:, 2], bits.sum(1).astype(np.float32))
    assert np.allclose(f[:, 3], 1.0, rtol=1e-5)
    # estimator: the 4-bit and the fp32 query forms agree within the query quantisation error, and both
    # estimate the true inner-product distance with the error RaBitQ promises at this dimension
    q = rng.standard_normal((20, d)).astype(np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    d4 = orc.flat_dists(orc.RABITQ, orc.IP, d, codes, orc.rabitq_process_query(q, rot, cen, orc.IP, 4), qbits=4)
    codes32 = orc.rabitq_encode(x, rot, cen, orc.IP, qbits=32)
    d32 = orc.flat_dists(orc.RABITQ, orc.IP, d, codes32, orc.rabitq_process_query(q, rot, cen, orc.IP, 32), qbits=32)
    true = 1.0 - q.astype(np.float64) @ x.astype(np.float64).T
    assert np.abs(d4 - d32).max() < 0.05
    assert np.abs(d32 - true).mean() < 0.08 and np.abs(d4 - true).mean() < 0.08
    assert np.corrcoef(d4.ravel(), true.ravel())[0, 1] > 0.7


@pytest.mark.parametrize("d", [8, 33, 128, 200])
def test_rabitq_decode_is_the_sign_point_rotated_back(d):
    """RaBitQuantizer::DecodeOneImpl (rabitq_quantizer.cpp:871-899), which the l2 bias of residual lists is computed
    from.  (1) The scale step equals the reference's compiled InverseNormalizeWithCentroid on the identity rotation.
    (2) What the definition fixes for any rotation: R x' - centroid has the code's signs and the single magnitude
    norm / sqrt(d).  (3) A row built to sit exactly on such a point encodes to those signs and decodes to itself.
    (4) Multi-bit codes: the reference returns false."""
    rng = np.random.default_rng(90 + d)
    rot = _rotation(rng, d)
    n = 40
    x = rng.standard_normal((n, d)).astype(np.float32)
    cen = orc.rabitq_train(x, rot)
    for metric in (orc.L2, orc.IP):
        codes = orc.rabitq_encode(x, rot, cen, metric)
        dec = orc.rabitq_decode(codes, d, rot, cen, metric)
        nb = (d + 7) // 8
        bits = np.unpackbits(codes[:, :nb], axis=1, bitorder="little")[:, :d].astype(np.float64)
        norms = np.ascontiguousarray(codes[:, -(16 if metric == orc.IP else 12):][:, :4]).view(np.float32)[:, 0].astype(np.float64)
        back = dec.astype(np.float64) @ rot.astype(np.float64).T - cen.astype(np.float64)
        want = (2.0 * bits - 1.0) * norms[:, None] / np.sqrt(d)
        np.testing.assert_allclose(back, want, rtol=0, atol=2e-5 * (1.0 + np.abs(want).max() + np.abs(cen).max()))
        # the stored norm is |R x - centroid|: the decoded point lies at that distance from the centroid as well
        np.testing.assert_allclose(np.linalg.norm(back, axis=1), norms, rtol=1e-5)
    ref = orc.ref()
    if ref is not None:
        eye = np.eye(d, dtype=np.float32)
        codes = orc.rabitq_encode(x, eye, cen, orc.L2)
        dec = orc.rabitq_decode(codes, d, eye, cen, orc.L2)
        inv = np.float32(1.0) / np.sqrt(np.float32(d))
        for i in range(n):
            signs = np.where(np.unpackbits(codes[i, :(d + 7) // 8], bitorder="little")[:d] != 0, inv, -inv).astype(np.float32)
            norm = np.ascontiguousarray(codes[i, -12:-8]).view(np.float32)[0]
            out = np.empty(d, np.float32)
            ref["InverseNormalizeWithCentroid"].restype = None
            ref["InverseNormalizeWithCentroid"](_p(signs), _p(cen), _p(out), C.c_uint64(d), C.c_float(norm))
            # (a fused and an unfused multiply-add differ by an ulp of the result)
            np.testing.assert_allclose(dec[i], out, rtol=3e-7, atol=1e-7)
    # (3) a fixed point: x = R^T (centroid + r s / sqrt(d)) for a sign vector s
    s = np.where(rng.random((n, d)) < 0.5, -1.0, 1.0)
    r = rng.uniform(0.5, 2.0, n)
    pts = ((cen.astype(np.float64) + s * r[:, None] / np.sqrt(d)) @ rot.astype(np.float64)).astype(np.float32)
    codes = orc.rabitq_encode(pts, rot, cen, orc.L2)
    got_bits = np.unpackbits(codes[:, :(d + 7) // 8], axis=1, bitorder="little")[:, :d]
    assert np.array_equal(got_bits, (s > 0).astype(np.uint8))
    np.testing.assert_allclose(orc.rabitq_decode(codes, d, rot, cen, orc.L2), pts, rtol=0, atol=1e-5 * (1 + np.abs(pts).max()))
    x4 = orc.rabitq_encode_multibit(x, rot, cen, orc.L2, 4)
    assert orc.rabitq_decode(x4, d, rot, cen, orc.L2, qbits=orc.rabitq_bits(32, 4)) is None


FHT_DIMS = [1, 2, 7, 8, 33, 64, 100, 128, 200, 256, 960]


def test_fht_primitives_match_compiled_reference_kernels():
    """FlipSign, VecRescale, FHTRotate and KacsWalk (generic.cpp:953-985, butterfly.h) against the reference's own
    compiled generic kernels: sums and differences only, so bit for bit."""
    ref = orc.ref()
    if ref is None:
        pytest.skip("oracle/_ref is not built (reference sources not mounted)")
    rng = np.random.default_rng(953)
    for d in FHT_DIMS:
        v = rng.standard_normal(d).astype(np.float32)
        flip = rng.integers(0, 256, (d + 7) // 8).astype(np.uint8)
        for which, name in enumerate(["FlipSign", "VecRescale", "FHTRotate", "KacsWalk"]):
            if name == "FHTRotate" and d & (d - 1):
                continue  # a power-of-two block only
            want = v.copy()
            fn = ref[name]
            fn.restype = None
            if name == "FlipSign":
                fn(_p(flip), _p(want), C.c_uint64(d))
            elif name == "VecRescale":
                fn(_p(want), C.c_uint64(d), C.c_float(0.37))
            else:
                fn(_p(want), C.c_uint64(d))
            got = orc.fht_primitive(which, v, flip=flip, val=0.37)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (name, d)


@pytest.mark.parametrize("d", FHT_DIMS)
def test_fht_kac_rotator_is_orthogonal_and_inverts(d):
    """FhtKacRotator::Transform (fht_kac_rotate_transformer.cpp:64-96) by the reference test's own properties
    (fht_kac_rotate_transformer_test.cpp:64-86: lengths kept, the inverse returns the input within 1e-4), by
    orthogonality of the whole map, and -- a power of two without flips -- by the closed form (H / sqrt(d))^4 = I."""
    rng = np.random.default_rng(64 + d)
    flip = rng.integers(0, 256, 4 * ((d + 7) // 8)).astype(np.uint8)
    x = rng.standard_normal((6, d)).astype(np.float32)
    y = orc.fht_kac_transform(flip, x)
    back = orc.fht_kac_transform(flip, y, inverse=True)
    assert np.max(np.abs(back - x)) < 1e-4
    np.testing.assert_allclose((y.astype(np.float64) ** 2).sum(1), (x.astype(np.float64) ** 2).sum(1), rtol=1e-5)
    m = orc.fht_kac_transform(flip, np.eye(d, dtype=np.float32)).T.astype(np.float64)  # column j = the image of e_j
    np.testing.assert_allclose(m @ m.T, np.eye(d), atol=2e-6 * max(8, d) ** 0.5)
    if d > 2:
        assert np.abs(m - np.eye(d)).max() > 0.05  # and it does mix
    if d & (d - 1) == 0:
        none = np.zeros_like(flip)
        np.testing.assert_allclose(orc.fht_kac_transform(none, x), x, rtol=0, atol=1e-5)
        # one round with known flips: H diag(s) x / sqrt(d), H the Sylvester matrix
        h = np.array([[1.0]])
        while h.shape[0] < d:
            h = np.block([[h, h], [h, -h]])
        s = 1.0 - 2.0 * np.unpackbits(flip[:(d + 7) // 8], bitorder="little")[:d]
        one = orc.fht_primitive(1, orc.fht_primitive(2, orc.fht_primitive(0, x[0], flip=flip)), val=1.0 / np.sqrt(np.float32(d)))
        np.testing.assert_allclose(one, h @ (s * x[0]) / np.sqrt(d), rtol=0, atol=1e-5 * (1 + np.abs(x[0]).max()) * np.sqrt(d))


def _rabitq_dist(qcode, code, d, metric, qbits):
    L = orc.lib()
    return float(L.orc_rabitq_dist(_p(np.ascontiguousarray(qcode)), _p(np.ascontiguousarray(code)), C.c_uint64(d), metric,
                                   qbits))


def _rabitq_case(seed, d, n, metric, unit):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, d)).astype(np.float32)
    if unit:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    rot = _rotation(rng, d)
    cen = orc.rabitq_train(x, rot)
    return rng, x, rot, cen


@pytest.mark.parametrize("d", [64, 128, 200, 768])
def test_rabitq_estimator_self_distance_is_exact(d):
    """A 32-bit query equal to a stored vector: <o, o_bar> of the query IS the code's error field (the same
    RaBitQFloatBinaryIP over the same normalised vector), so ip_est = error / error = 1 and the estimate collapses to
    (|o| - |q|)^2 = 0 exactly, the inner-product distance to 1 - |x|^2 and cosine to 0.  Dropping the division by the
    error, dividing by the norm instead, or a wrong sign in l2_ube all leave 2 n^2 (1 - error) or worse here.  The
    reference tests self-distances the same way (rabitq_quantizer_test.cpp:72-103)."""
    rng, x, rot, cen = _rabitq_case(60 + d, d, 50, orc.L2, unit=False)
    for metric in (orc.L2, orc.IP, orc.COSINE):
        codes = orc.rabitq_encode(x, rot, cen, metric, qbits=32)
        qcodes = orc.rabitq_process_query(x, rot, cen, metric, 32)
        nb = (d + 7) // 8
        nb4 = (nb + 3) // 4 * 4
        for i in range(x.shape[0]):
            f = codes[i, nb4:].view(np.float32)  # norm, error, (raw norm)
            assert 0.5 < f[1] < 1.0  # the error factor is far from 1, so a dropped division would show
            got = _rabitq_dist(qcodes[i], codes[i], d, metric, 32)
            if metric == orc.L2:
                assert got == 0.0
            elif metric == orc.IP:
                r = np.float32(f[2])
                assert got == float(np.float32(1) - (r * r + r * r - np.float32(0)) * np.float32(0.5))
                assert abs(got - (1.0 - float((x[i].astype(np.float64) ** 2).sum()))) < 1e-4 * d
            else:
                assert abs(got) < 1e-6


def test_rabitq_estimator_error_clamp_and_zero_norms():
    """|error| < 1e-5 is replaced by +1 / -1 by its sign (rabitq_quantizer.cpp:1824-1827); a raw norm below 1e-5 on
    either side makes the inner-product and cosine distance 1 (:1838-1857)."""
    d = 128
    rng, x, rot, cen = _rabitq_case(71, d, 8, orc.IP, unit=True)
    nb = d // 8
    L = orc.lib()
    q = rng.standard_normal((1, d)).astype(np.float32)
    q32 = orc.rabitq_process_query(q, rot, cen, orc.L2, 32)[0]
    codes = orc.rabitq_encode(x, rot, cen, orc.L2, qbits=32)
    inv = C.c_float(1.0 / np.sqrt(np.float32(d)))
    for i in range(4):
        code = codes[i].copy()
        f = code[nb:].view(np.float32)  # norm, error
        ip_bq = np.float32(L.orc_rabitq_float_binary_ip(_p(q32), _p(code), C.c_uint64(d), inv))
        n_o, n_q = np.float32(f[0]), q32[4 * d:].view(np.float32)[0]
        for forced, divisor in ((1e-6, 1.0), (-1e-6, -1.0), (0.0, 1.0), (9.9e-6, 1.0), (-9.9e-6, -1.0), (2e-5, 2e-5),
                                (-2e-5, -2e-5)):
            f[1] = forced
            est = np.float32(ip_bq / np.float32(divisor))
            expect = n_o * n_o + n_q * n_q + np.float32(-2) * n_o * n_q * est
            got = _rabitq_dist(q32, code, d, orc.L2, 32)
            assert got == float(expect), (forced, got, float(expect))
    # zero raw norms
    for metric in (orc.IP, orc.COSINE):
        for qbits in (4, 32):
            codes = orc.rabitq_encode(x, rot, cen, metric, qbits=qbits)
            qc = orc.rabitq_process_query(q, rot, cen, metric, qbits)[0]
            normal = _rabitq_dist(qc, codes[0], d, metric, qbits)
            assert normal != 1.0
            code = codes[0].copy()
            code[-4:].view(np.float32)[0] = 5e-6  # the base's raw norm is the last field
            assert _rabitq_dist(qc, code, d, metric, qbits) == 1.0
            qz = qc.copy()
            qz[-4:].view(np.float32)[0] = 0.0  # and so is the query's
            assert _rabitq_dist(qz, codes[0], d, metric, qbits) == 1.0
            zero_q = orc.rabitq_process_query(np.zeros((1, d), np.float32), rot, cen, metric, qbits)[0]
            assert _rabitq_dist(zero_q, codes[0], d, metric, qbits) == 1.0


@pytest.mark.parametrize("d", [6, 15, 128, 200, 768])
def test_rabitq_4bit_estimate_equals_the_fp32_form_on_the_dequantised_query(d):
    """The 4-bit branch (rabitq_quantizer.cpp:924-939, equation 19-20 of the paper) is algebra on
    <bits, lb + delta c> : feeding the dequantised query lb + delta c_d through the fp32 branch (RaBitQFloatBinaryIP,
    pinned against the reference's own compiled kernel) must give the same distance up to fp32 rounding.  A dropped
    or mis-signed term of the four (2 delta ip, 2 lb sum_b, delta sum_q, lb d) is off by far more."""
    rng, x, rot, cen = _rabitq_case(80 + d, d, 40, orc.IP, unit=True)
    q = rng.standard_normal((6, d)).astype(np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    nb = (d + 7) // 8
    nb4 = (nb + 3) // 4 * 4
    for metric in (orc.L2, orc.IP, orc.COSINE):
        codes4 = orc.rabitq_encode(x, rot, cen, metric, qbits=4)
        codes32 = orc.rabitq_encode(x, rot, cen, metric, qbits=32)
        # the two base layouts hold the same bits, norm, error and raw norm
        assert np.array_equal(codes4[:, :nb4 + 8], codes32[:, :nb4 + 8])
        q4 = orc.rabitq_process_query(q, rot, cen, metric, 4)
        q32 = orc.rabitq_process_query(q, rot, cen, metric, 32)
        qs32 = q32.shape[1]
        pb = (d + 511) // 512 * 512 // 8
        for i in range(q.shape[0]):
            planes = q4[i, :4 * pb].reshape(4, pb)
            c = np.zeros(d, np.int64)
            for b in range(4):
                c += np.unpackbits(planes[b], bitorder="little")[:d].astype(np.int64) << b
            tail = q4[i, 4 * pb:].view(np.float32)  # lb, delta, sum, norm, (raw norm)
            lb, delta, qsum = tail[0], tail[1], tail[2]
            assert qsum == np.float32(c.sum())
            deq = np.zeros(qs32, np.uint8)
            deq[:4 * d] = (np.float32(lb) + np.float32(delta) * c.astype(np.float32)).astype(np.float32).view(np.uint8)
            deq[4 * d:] = q32[i, 4 * d:]  # same norm and raw norm fields
            assert np.array_equal(tail[3:].view(np.uint8), q32[i, 4 * d:])
            for j in range(x.shape[0]):
                a = _rabitq_dist(q4[i], codes4[j], d, metric, 4)
                b = _rabitq_dist(deq, codes32[j], d, metric, 32)
                assert abs(a - b) <= 2e-5 * (1.0 + abs(b)), (metric, i, j, a, b)


def test_kmeans_assign_is_the_exact_argmin():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((800, 24)).astype(np.float32)
    cent = rng.standard_normal((37, 24)).astype(np.float32)
    cent[20] = cent[5]  # a tie: the first minimum wins
    labels, mind, loss = orc.kmeans_assign(x, cent)
    d2 = ((x[:, None, :].astype(np.float64) - cent[None].astype(np.float64)) ** 2).sum(2)
    assert np.array_equal(labels, d2.argmin(1)) and 20 not in labels
    xn = (x.astype(np.float64) ** 2).sum(1)
    assert np.allclose(mind + xn, d2.min(1), atol=1e-4)
    assert abs(loss - d2.min(1).mean()) < 1e-4
    # update = mean of members, empty clusters reported
    newc, counts = orc.kmeans_update(x, labels, cent)
    for j in range(37):
        m = labels == j
        assert counts[j] == m.sum()
        if m.any():
            assert np.allclose(newc[j], x[m].mean(0), atol=1e-5)
        else:
            assert np.array_equal(newc[j], cent[j])


def test_kmeans_plus_plus_seeding_follows_the_squared_distance_law():
    """select_initial_centroids_kmeans_plus_plus (kmeans_cluster.cpp:383-435) with the draws given, against an
    independent restatement: smallest squared distances in float64 from the definition, cumulative sums and the first
    index that reaches the threshold by searchsorted.  Draws that land within rounding of a boundary are left out."""
    rng = np.random.default_rng(12)
    n, d, k = 500, 9, 40
    x = rng.standard_normal((n, d)).astype(np.float32)
    draws = rng.random(k - 1)
    cent, picks = orc.kmeans_init_pp(x, k, 17, draws)
    assert picks[0] == 17 and np.array_equal(cent, x[picks.astype(np.int64)])
    x64 = x.astype(np.float64)
    chosen = [17]
    for c in range(1, k):
        d2 = ((x64[:, None, :] - x64[chosen][None]) ** 2).sum(2).min(1)
        cum = np.cumsum(d2)
        thr = draws[c - 1] * cum[-1]
        i = int(np.searchsorted(cum, thr, side="left"))
        near = np.abs(cum[max(i - 1, 0):i + 1] - thr).min() < 1e-5 * cum[-1]  # fp32 distances vs float64 ones
        assert near or picks[c] == i, (c, picks[c], i)
        chosen.append(int(picks[c]))
    assert len(set(chosen)) == k, "a chosen row has distance 0 and cannot be drawn again"
    # k = n: every row is picked exactly once, whatever the draws
    _, all_picks = orc.kmeans_init_pp(x[:60], 60, 3, rng.random(59))
    assert sorted(all_picks.tolist()) == list(range(60))
    # coincident rows: once every distinct point is a centroid the total weight is 0 and the draw picks any row
    y = np.repeat(rng.standard_normal((3, d)).astype(np.float32), 5, axis=0)
    _, p = orc.kmeans_init_pp(y, 6, 0, np.array([0.5, 0.99, 0.0, 0.5, 0.999]))
    assert len({int(v) // 5 for v in p[:3]}) == 3 and list(p[3:]) == [0, 7, 14]


def test_heaps_equal_sorting():
    rng = np.random.default_rng(8)
    n, d, k = 700, 10, 13
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((6, d), dtype=np.float32)
    codes = x.view(np.uint8).reshape(n, 4 * d)
    all_d = orc.flat_dists(orc.FP32, orc.L2, d, codes, q)
    for strict in (False, True):
        ids, ds = orc.flat_scan_topk(orc.FP32, orc.L2, d, codes, q, k, strict=strict)
        order = np.argsort(all_d, axis=1, kind="stable")[:, :k]
        assert np.array_equal(ds, np.take_along_axis(all_d, order, 1))
        assert np.array_equal(ids, order.astype(np.uint32))
    ids, ds = orc.flat_scan_topk(orc.FP32, orc.L2, d, codes[:5], q, k)
    assert np.all(ids[:, 5:] == 0xFFFFFFFF) and np.all(np.isinf(ds[:, 5:]))


def test_ivf_probing_every_list_equals_the_flat_scan():
    rng = np.random.default_rng(9)
    n, d, nlist, nq, k = 1500, 16, 12, 9, 10
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((nq, d), dtype=np.float32)
    cent = x[:nlist].copy()
    labels, _, _ = orc.kmeans_assign(x, cent)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    # stable counting sort: inside a list inner ids ascend; lists are contiguous in label order
    for j in range(nlist):
        seg = order[int(offsets[j]):int(offsets[j + 1])]
        assert np.all(labels[seg] == j) and np.all(np.diff(seg.astype(np.int64)) > 0)
    codes = x.view(np.uint8).reshape(n, 4 * d)
    buckets = np.tile(np.arange(nlist, dtype=np.int32), (nq, 1))
    ids, ds = orc.ivf_scan(orc.FP32, orc.L2, d, codes[order], offsets, order, q, buckets, k)
    fids, fds = orc.flat_scan_topk(orc.FP32, orc.L2, d, codes, q, k, strict=True)
    assert np.array_equal(ds, fds) and np.array_equal(np.sort(ids, 1), np.sort(fids, 1))
    # routing is the exact centroid top-nprobe; rerank of exact candidates returns them sorted
    b, bd = orc.ivf_route(cent, q, 4)
    dc = ((q[:, None, :].astype(np.float64) - cent[None].astype(np.float64)) ** 2).sum(2)
    assert np.array_equal(b, np.argsort(dc, 1, kind="stable")[:, :4].astype(np.int32))
    rids, rds = orc.rerank_fp32(x, q, ids, 5)
    assert np.array_equal(rds, fds[:, :5])


def test_residual_scan_closed_forms():
    """use_residual: with fp32 codes of x - c the corrected distance is the plain distance to x (l2: |q - x|^2, ip:
    1 - <q, x>); with sq8 codes it is the distance to c + decoded.  A dropped bias, a missing factor 2 or a wrong sign
    of <q, c> is off by the size of |c|^2."""
    rng = np.random.default_rng(12)
    n, d, nlist, nq, k = 900, 24, 7, 5, 30
    x = (rng.random((n, d), dtype=np.float32) - 0.2).astype(np.float32)
    q = (rng.random((nq, d), dtype=np.float32) - 0.2).astype(np.float32)
    cent = x[:nlist].copy() + 0.5
    labels, _, _ = orc.kmeans_assign(x, cent)
    offsets, order = orc.ivf_build_lists(labels, nlist)
    buckets = np.tile(np.arange(nlist, dtype=np.int32), (nq, 1))
    for metric in (orc.L2, orc.IP):
        res = orc.residual_rows(x, labels, cent, metric)
        assert np.array_equal(res, x - cent[labels])
        bias = orc.residual_bias(res, labels, cent) if metric == orc.L2 else None
        ids, ds = orc.ivf_scan_residual(orc.FP32, metric, d, res.view(np.uint8).reshape(n, 4 * d)[order], offsets, order, q,
                                        q, cent, None if bias is None else bias[order], buckets, k)
        x64, q64 = x.astype(np.float64), q.astype(np.float64)
        full = ((q64[:, None, :] - x64[None]) ** 2).sum(2) if metric == orc.L2 else 1.0 - q64 @ x64.T
        want = np.sort(full, axis=1)[:, :k]
        assert np.allclose(ds, want, rtol=1e-4, atol=2e-5)
        # sq8 codes of the residual: distance to c + decoded
        lb, diff = orc.sq_train(res, 8, metric)
        codes = orc.sq_encode(res, 8, lb, diff, metric)
        dec = orc.sq_decode(codes, d, 8, lb, diff)
        bias = orc.residual_bias(dec, labels, cent) if metric == orc.L2 else None
        ids, ds = orc.ivf_scan_residual(orc.SQ8, metric, d, codes[order], offsets, order, q, q, cent,
                                        None if bias is None else bias[order], buckets, k, lb=lb, diff=diff)
        y64 = (dec + cent[labels]).astype(np.float64)
        full = ((q64[:, None, :] - y64[None]) ** 2).sum(2) if metric == orc.L2 else 1.0 - q64 @ y64.T
        assert np.allclose(ds, np.sort(full, axis=1)[:, :k], rtol=1e-4, atol=5e-5)
    # cosine normalises the row before the centroid comes off; uniform decode is lb + code / levels * diff
    res = orc.residual_rows(x, labels, cent, orc.COSINE)
    xn = x / np.linalg.norm(x, axis=1, keepdims=True)
    assert np.allclose(res, xn - cent[labels], atol=1e-6)
    l, dd = orc.sq_train_uniform(res, 4, orc.L2, mode=3)
    c4 = orc.squ_encode(res, 4, l, dd, orc.L2)
    raw = np.stack([(c4[:, i // 2] >> (4 * (i % 2))) & 15 for i in range(d)], 1)
    assert np.allclose(orc.squ_decode(c4, d, 4, l, dd, orc.L2), l + raw / 15.0 * dd, atol=1e-6)


# ------------------------------------------------------------------ pqfs (PQ fast scan)
def _pqfs_lookup_cases():
    """The reference's own shapes (src/simd/pqfs_simd_test.cpp: pq_dim 8, 16, 31, 256), seeded."""
    rng = np.random.default_rng(903)
    for pq_dim in (8, 16, 31, 256):
        lut = rng.integers(0, 256, pq_dim * 16).astype(np.uint8)
        packaged = rng.integers(0, 256, pq_dim * 16).astype(np.uint8)
        yield pq_dim, lut, packaged


def test_pqfs_lookup32_matches_compiled_reference_and_golden_vectors():
    gold = json.load(open(os.path.join(GOLDEN, "pqfs_lookup32.json")))
    for (pq_dim, lut, packaged), want in zip(_pqfs_lookup_cases(), gold["values"]):
        got = orc.pqfs_lookup32(lut, packaged, pq_dim)
        assert got.tolist() == want, pq_dim
        # the function accumulates into its output (the caller zeroes it between blocks)
        L = orc.lib()
        twice = got.copy()
        L.orc_pqfs_lookup32(_p(lut), _p(packaged), C.c_uint64(pq_dim), _p(twice))
        assert np.array_equal(twice, 2 * got)
    tiers = ["generic", "sse", "avx"] + (["avx2"] if orc.lib().orc_cpu_has_avx2() else []) + \
            (["avx512"] if orc.lib().orc_cpu_has_avx512() else [])
    ran = 0
    for isa in tiers:
        fn = orc.ref_pqfs_lookup32(isa)
        if fn is None:
            continue
        ran += 1
        for pq_dim, lut, packaged in _pqfs_lookup_cases():
            out = np.zeros(32, np.int32)
            fn(_p(lut), _p(packaged), C.c_uint64(pq_dim), _p(out))
            assert np.array_equal(out, orc.pqfs_lookup32(lut, packaged, pq_dim)), (isa, pq_dim)
    if orc.ref() is not None:
        assert ran >= 3


@pytest.mark.parametrize("pq_dim", [1, 7, 64, 128])
def test_pqfs_package32_round_trip_and_order(pq_dim):
    """Package32 / Unpack32 (pq_fastscan_quantizer.cpp:241-297; the reference's own round-trip test) and what the
    order means: entry v of PQFastScanLookUp32's result on a packaged block is the table sum of vector v."""
    rng = np.random.default_rng(pq_dim)
    cs = (pq_dim + 1) // 2
    codes = rng.integers(0, 256, (32, cs)).astype(np.uint8)
    if pq_dim % 2:
        codes[:, -1] &= 0x0F
    packaged = orc.pqfs_package32(codes, pq_dim)
    assert np.array_equal(orc.pqfs_unpack32(packaged, pq_dim), codes)
    lut = rng.integers(0, 256, pq_dim * 16).astype(np.uint8)
    sums = orc.pqfs_lookup32(lut, packaged, pq_dim)
    for v in range(32):
        nib = [int(codes[v, i // 2] >> 4) if i % 2 else int(codes[v, i // 2] & 15) for i in range(pq_dim)]
        assert sums[v] == sum(int(lut[16 * i + n]) for i, n in enumerate(nib)), v
    # a partly filled block: the vectors beyond valid_size read as code 0 in every subspace
    part = orc.pqfs_package32(codes, pq_dim, valid=5)
    back = orc.pqfs_unpack32(part, pq_dim)
    assert np.array_equal(back[:5], codes[:5]) and not back[5:].any()


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
def test_pqfs_encode_table_and_distance_closed_forms(metric):
    rng = np.random.default_rng(31 + metric)
    n, d, pq_dim = 200, 24, 6
    sd = d // pq_dim
    x = rng.standard_normal((n, d)).astype(np.float32)
    cb = rng.standard_normal((pq_dim, 16, sd)).astype(np.float32)
    xn = x / np.linalg.norm(x, axis=1, keepdims=True) if metric == orc.COSINE else x
    codes = orc.pq_encode(x, pq_dim, cb, metric)
    # the nearest centroid per subspace, in float64, ties aside
    sub = xn.reshape(n, pq_dim, 1, sd).astype(np.float64)
    dist = ((sub - cb[None].astype(np.float64)) ** 2).sum(-1)  # n x pq_dim x 16
    nib = np.stack([(codes[:, i // 2] >> 4) if i % 2 else (codes[:, i // 2] & 15) for i in range(pq_dim)], 1)
    best = dist.min(-1)
    got = np.take_along_axis(dist, nib[..., None].astype(np.int64), -1)[..., 0]
    assert np.all(got <= best * (1 + 1e-5) + 1e-6)
    # decode returns the named centroids; encoding them again names them again
    dec = orc.pq_decode(codes, d, pq_dim, cb)
    assert np.array_equal(dec.reshape(n, pq_dim, sd), cb[np.arange(pq_dim)[None], nib])
    if metric != orc.COSINE:
        assert np.array_equal(orc.pq_encode(dec, pq_dim, cb, metric), codes)
    # the query table: bytes = trunc((value - lower) / diff * 255) between the smallest and largest entry
    q = rng.standard_normal((3, d)).astype(np.float32)
    qn = q / np.linalg.norm(q, axis=1, keepdims=True) if metric == orc.COSINE else q
    qc = orc.pqfs_process_query(q, pq_dim, cb, metric)
    for r in range(3):
        qs = qn[r].reshape(pq_dim, 1, sd).astype(np.float64)
        c64 = cb.astype(np.float64)
        table = ((qs - c64) ** 2).sum(-1) if metric == orc.L2 else (qs * c64).sum(-1)  # pq_dim x 16
        diff, lower = qc[r, pq_dim * 16:].view(np.float32)
        assert abs(lower - table.min()) <= 1e-5 * max(1.0, abs(table.min()))
        assert abs(diff - (table.max() - table.min())) <= 1e-5 * (table.max() - table.min())
        want = (table - table.min()) / (table.max() - table.min()) * 255.0
        lut8 = qc[r, :pq_dim * 16].reshape(pq_dim, 16).astype(np.float64)
        assert np.all(np.abs(lut8 - np.floor(want)) <= 1.0 + 1e-9) and np.mean(lut8 == np.floor(want)) > 0.98
        assert lut8.min() == 0 and lut8.max() == 255
        # distance of a code = float(sum of its table bytes) / 255 * diff + lower (1 - that for ip / cosine),
        # and the block scan over packaged codes returns the same floats
        sums = lut8[np.arange(pq_dim)[None], nib].sum(1)
        d_flat = orc.flat_dists(orc.PQFS, metric, pq_dim, codes, qc[r:r + 1])[0]
        v = (sums.astype(np.float32) / np.float32(255.0)) * np.float32(diff) + np.float32(lower)
        v = v if metric == orc.L2 else np.float32(1.0) - v
        assert np.array_equal(d_flat.view(np.uint32), v.astype(np.float32).view(np.uint32))
        pad = np.zeros((224, codes.shape[1]), np.uint8)
        pad[:n] = codes
        packaged = np.concatenate([orc.pqfs_package32(pad[b:b + 32], pq_dim, valid=min(32, n - b)) for b in range(0, 224, 32)])
        d_scan = orc.pqfs_scan_batch(qc[r], packaged, n, pq_dim, metric)
        assert np.array_equal(d_scan.view(np.uint32), d_flat.view(np.uint32))


@pytest.mark.parametrize("metric", [orc.L2, orc.IP, orc.COSINE])
def test_pqfs_distances_meet_the_reference_tests_bound(metric):
    """pq_fastscan_quantizer_test.cpp "PQFSQuantizer Compute": with one subspace per dimension, trained codebooks and
    unit vectors, every distance is within 0.08 of the true one (dim 128, 300 vectors, 100 queries)."""
    rng = np.random.default_rng(128 + metric)
    n, nq, d = 300, 100, 128
    x = rng.random((n, d), dtype=np.float32)
    q = rng.random((nq, d), dtype=np.float32)
    if metric != orc.COSINE:  # the reference's fixture normalises the vectors for l2 / ip and lets cosine do it
        x /= np.linalg.norm(x, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    cb = orc.pq_train(x, d, metric)
    codes = orc.pq_encode(x, d, cb, metric)
    got = orc.flat_dists(orc.PQFS, metric, d, codes, orc.pqfs_process_query(q, d, cb, metric))
    x64, q64 = x.astype(np.float64), q.astype(np.float64)
    if metric == orc.COSINE:
        x64 /= np.linalg.norm(x64, axis=1, keepdims=True)
        q64 /= np.linalg.norm(q64, axis=1, keepdims=True)
    true = ((q64[:, None] - x64[None]) ** 2).sum(-1) if metric == orc.L2 else 1.0 - q64 @ x64.T
    assert np.abs(got - true).max() <= 0.08, float(np.abs(got - true).max())


# ------------------------------------------------------------------ multi-bit RaBitQ (rabitq_bits_per_dim_base 2..8)
def _alignment(o, code, bits):
    y = code.astype(np.float64) - 0.5 * ((1 << bits) - 1)
    ip = float(o.astype(np.float64) @ y)
    return ip * ip / float(y @ y)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_rabitq_fast_encode_known_input_of_the_reference_test(bits):
    """rabitq_quantizer_test.cpp:107-183: on sin(0.37 d) + 0.2 cos(0.11 d), one round is at least as aligned as the
    floor grid it starts from, six rounds at least as one, codes stay in range, and the norm is |code - centre|."""
    dgrid = np.arange(64, dtype=np.float32)
    data = (np.sin(dgrid * np.float32(0.37)) + np.float32(0.2) * np.cos(dgrid * np.float32(0.11))).astype(np.float32)
    code_max = (1 << bits) - 1
    max_abs = float(np.abs(data.astype(np.float64)).max())
    delta = 2.0 * max_abs / (code_max + 1)
    lvq = np.clip(np.floor((data.astype(np.float64) + max_abs) / delta), 0, code_max).astype(np.uint8)
    one, _ = orc.rabitq_fast_encode(data, bits, rounds=1)
    six, norm = orc.rabitq_fast_encode(data, bits, rounds=6)
    assert _alignment(data, one, bits) + 1e-7 >= _alignment(data, lvq, bits)
    assert _alignment(data, six, bits) + 1e-7 >= _alignment(data, one, bits)
    assert six.max() <= code_max and norm > 0
    y = six.astype(np.float64) - 0.5 * code_max
    assert abs(norm - np.sqrt(float(y @ y))) <= 1e-5
    # a fixed point: after convergence no single one-level move raises the alignment by more than the tolerance
    conv, _ = orc.rabitq_fast_encode(data, bits, rounds=32)
    base = _alignment(data, conv, bits)
    for dd in range(64):
        for step in (-1, 1):
            c = int(conv[dd]) + step
            if 0 <= c <= code_max:
                moved = conv.copy()
                moved[dd] = c
                y = moved.astype(np.float64) - 0.5 * code_max
                if float(data.astype(np.float64) @ y) >= 0:
                    assert _alignment(data, moved, bits) <= base + 1e-8 * max(1.0, base) + 1e-12


@pytest.mark.parametrize("bits", [2, 4])
def test_rabitq_encoders_against_the_exhaustive_optimum(bits):
    """rabitq_quantizer_test.cpp:185-226 for the fast encoder (never above the best of all 2^(3 bits) codes).  The
    extended encoder (rabitq_quantizer.cpp:455-607) walks the scale on the even grid 0, +-2, ... but rounds to the odd
    one, so it is near the optimum, not at it: within 3 % at 4 bits; at 2 bits the walk is traced by hand below."""
    import itertools
    levels = 1 << bits
    rng = np.random.default_rng(bits)
    cases = [np.array([0.73, -0.41, 0.19], np.float32)] + [rng.standard_normal(3).astype(np.float32) for _ in range(20)]
    for data in cases:
        data = (data / np.linalg.norm(data)).astype(np.float32)
        best = 0.0
        for cand in itertools.product(range(levels), repeat=3):
            y = np.array(cand, np.float64) - 0.5 * (levels - 1)
            ip = float(data.astype(np.float64) @ y)
            if ip > 0:
                best = max(best, ip * ip / float(y @ y))
        fast, _ = orc.rabitq_fast_encode(data, bits)
        assert _alignment(data, fast, bits) <= best + 1e-10
        ext, norm = orc.rabitq_extend_encode(data, bits)
        y = ext.astype(np.float64) - 0.5 * (levels - 1)
        assert float(data.astype(np.float64) @ y) > 0
        if bits == 4 and np.abs(data).min() > 0.05:
            assert _alignment(data, ext, bits) >= best * 0.97, (data, ext, best)
        assert abs(norm - np.sqrt(float(y @ y))) <= 1e-5
    # By hand from the source, 2 bits (y2_max = 3, one event per coordinate at t = 1 / (2 |o|)): events in order
    # coordinate 1 (t 0.662: <y2, o> / |y2| = 0.755), coordinate 2 (t 0.838: 0.955, the best), coordinate 0 (t 1.83:
    # 0.938).  At t = 0.838: 2 t o = (0.458, -1.266, -1.000 - eps) -> odd grid (1, -1, -1) -> codes (2, 1, 1), norm
    # sqrt(0.75).
    ext, norm = orc.rabitq_extend_encode(np.array([0.2729807, -0.75481445, -0.5964367], np.float32), 2)
    assert ext.tolist() == [2, 1, 1] and abs(norm - np.sqrt(0.75)) < 1e-6
    # 3 bits (y2_max = 7, steps to +-2, +-4, +-6 at t = (1, 3, 5) / (2 |o|)) on (0.6, -0.8): events t = 0.625 (c1),
    # 0.833 (c0), 1.875 (c1), 2.5 (c0), 3.125 (c1), 4.167 (c0) with y2 = (0,-2), (2,-2), (2,-4), (4,-4), (4,-6), (6,-6)
    # and <y2, o> / |y2| = 0.8, 0.98995, 0.98387, 0.98995, 0.99846 (the best), 0.98995.  At t = 3.125:
    # 2 t o = (3.75, -5) -> round to (4, -5), 4 is even -> 5 -> odd grid (5, -5) -> codes ((5 + 7) / 2, (-5 + 7) / 2).
    ext, norm = orc.rabitq_extend_encode(np.array([0.6, -0.8], np.float32), 3)
    assert ext.tolist() == [6, 1] and abs(norm - np.sqrt(2.5 ** 2 * 2)) < 1e-6


def test_rabitq_multibit_zero_vector():
    """rabitq_quantizer_test.cpp:227-238: a zero vector encodes to code_max / 2 everywhere with norm 1."""
    for enc in (lambda o: orc.rabitq_fast_encode(o, 8), lambda o: orc.rabitq_extend_encode(o, 8)):
        code, norm = enc(np.zeros(16, np.float32))
        assert norm == 1.0 and np.all(code == 127)


@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_rabitq_multibit_self_distance_and_accuracy(bits, fast):
    """rabitq_quantizer_test.cpp:75-105: a query equal to a stored vector is at distance |d| <= 1e-3 (the error field
    is the same <o, code> the scan computes, so ip_est = 1); and more bits estimate better than fewer."""
    d, n = 32, 200
    rng, x, rot, cen = _rabitq_case(900 + bits, d, n, orc.L2, unit=False)
    qb = orc.rabitq_bits(32, bits)
    for metric in (orc.L2, orc.IP, orc.COSINE):
        codes = orc.rabitq_encode_multibit(x, rot, cen, metric, bits, fast=fast)
        assert codes.shape[1] == orc.rabitq_code_size(d, metric, qb)
        qcodes = orc.rabitq_process_query(x, rot, cen, metric, qb)
        for i in range(n):
            got = _rabitq_dist(qcodes[i], codes[i], d, metric, qb)
            if metric == orc.L2:
                assert abs(got) <= 1e-3
            elif metric == orc.COSINE:
                assert abs(got) <= 1e-5
            else:
                assert abs(got - (1.0 - float((x[i].astype(np.float64) ** 2).sum()))) <= 1e-3 * d
    # layout: planes, norm_code, norm, error (rabitq_quantizer.cpp:102-133)
    codes = orc.rabitq_encode_multibit(x, rot, cen, orc.L2, bits, fast=fast)
    nb = (d + 7) // 8 * bits
    f = codes[:, nb:].copy().view(np.float32)
    assert codes.shape[1] == nb + 12
    assert np.all(f[:, 0] > 0) and np.all(f[:, 1] > 0) and np.all((f[:, 2] > 0.5) & (f[:, 2] <= 1.0 + 1e-6))
    # error = cos(o, y): closer to 1 with more bits
    assert f[:, 2].mean() > {2: 0.85, 4: 0.98, 8: 0.9995}[bits]
    q = rng.standard_normal((30, d)).astype(np.float32)
    true = ((q[:, None, :].astype(np.float64) - x[None].astype(np.float64)) ** 2).sum(-1)
    est = orc.flat_dists(orc.RABITQ, orc.L2, d, codes, orc.rabitq_process_query(q, rot, cen, orc.L2, qb), qbits=qb)
    one = orc.flat_dists(orc.RABITQ, orc.L2, d, orc.rabitq_encode(x, rot, cen, orc.L2, 32),
                         orc.rabitq_process_query(q, rot, cen, orc.L2, 32), qbits=32)
    err, err1 = np.abs(est - true).mean(), np.abs(one - true).mean()
    assert err < err1 * {2: 0.8, 4: 0.3, 8: 0.05}[bits], (err, err1)


def test_rabitq_multibit_estimator_closed_form():
    """ip_obar_q (rabitq_quantizer.cpp:256-267) and the branch at :1799-1808 by hand on a 3-dimensional code: the
    estimate is (<q, u> - c sum q) / |u - c| / error inside l2_ube.  A dropped centre term, the wrong plane weight or
    a missing division each change the number."""
    d, bits = 3, 3
    rot = np.eye(d, dtype=np.float32)
    cen = np.zeros(d, np.float32)
    x = np.array([[3.0, -1.0, 0.5]], np.float32)
    q = np.array([[1.0, 2.0, -0.5]], np.float32)
    qb = orc.rabitq_bits(32, bits)
    code = orc.rabitq_encode_multibit(x, rot, cen, orc.L2, bits, fast=True)[0]
    qcode = orc.rabitq_process_query(q, rot, cen, orc.L2, qb)[0]
    planes = code[:3]
    u = np.array([sum(((int(planes[b]) >> dd) & 1) << b for b in range(bits)) for dd in range(d)], np.float64)
    c = 0.5 * 7
    norm_code, norm, error = code[4:16].view(np.float32)
    o = x[0].astype(np.float64) / np.linalg.norm(x[0])
    assert abs(norm - np.linalg.norm(x[0])) < 1e-6 and abs(norm_code - np.linalg.norm(u - c)) < 1e-6
    assert abs(error - float(o @ (u - c)) / np.linalg.norm(u - c)) < 1e-6
    qn = q[0].astype(np.float64) / np.linalg.norm(q[0])
    qf = qcode.view(np.float32)
    assert np.allclose(qf[:3], qn, atol=1e-6) and abs(qf[3] - qn.sum()) < 1e-6 and abs(qf[4] - np.linalg.norm(q[0])) < 1e-6
    ip_est = (float(qn @ u) - c * qn.sum()) / np.linalg.norm(u - c) / float(error)
    want = norm ** 2 + np.linalg.norm(q[0]) ** 2 - 2 * norm * np.linalg.norm(q[0]) * ip_est
    got = _rabitq_dist(qcode, code, d, orc.L2, qb)
    assert abs(got - want) < 1e-5
