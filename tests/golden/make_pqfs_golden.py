#!/usr/bin/env python3
"""Writes tests/golden/pqfs_lookup32.json: the result of vsag::generic::PQFastScanLookUp32 (compiled from the
reference's own src/simd/generic.cpp by oracle/Makefile into oracle/_ref) on the seeded tables and packaged codes
that tests/test_oracle_cpu.py regenerates (the shapes of the reference's src/simd/pqfs_simd_test.cpp).  Run where
the reference sources are mounted:

    make -C oracle && python tests/golden/make_pqfs_golden.py
"""
import ctypes as C
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import oracle as orc  # noqa: E402
import test_oracle_cpu as t  # noqa: E402


def main():
    fn = orc.ref_pqfs_lookup32("generic")
    if fn is None:
        raise SystemExit("oracle/_ref/libvsag_simd.so is not built")
    values = []
    for pq_dim, lut, packaged in t._pqfs_lookup_cases():
        out = np.zeros(32, np.int32)
        fn(t._p(lut), t._p(packaged), C.c_uint64(pq_dim), t._p(out))
        values.append(out.tolist())
    with open(os.path.join(HERE, "pqfs_lookup32.json"), "w") as f:
        json.dump({"source": "vsag::generic::PQFastScanLookUp32 compiled from src/simd/generic.cpp",
                   "pq_dims": [8, 16, 31, 256], "seed": 903, "values": values}, f)
    print("wrote", len(values), "result blocks")


if __name__ == "__main__":
    main()
