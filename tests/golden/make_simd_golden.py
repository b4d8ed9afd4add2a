#!/usr/bin/env python3
"""Writes tests/golden/simd_generic.json: the values of the reference's scalar kernels (vsag::generic::*,
compiled from the reference's own src/simd/generic.cpp by oracle/Makefile into oracle/_ref) on the seeded
vectors that tests/test_oracle_cpu.py regenerates.  Run where the reference sources are mounted:

    make -C oracle && python tests/golden/make_simd_golden.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import oracle as orc  # noqa: E402
import test_oracle_cpu as t  # noqa: E402


def main():
    ref = orc.ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libvsag_simd.so is not built")
    fns = {"fp32_ip": ref["FP32ComputeIP"], "fp32_l2": ref["FP32ComputeL2Sqr"], "sq8_ip": ref["SQ8ComputeIP"],
           "sq8_l2": ref["SQ8ComputeL2Sqr"], "sq4_ip": ref["SQ4ComputeIP"], "sq4_l2": ref["SQ4ComputeL2Sqr"],
           "sq4u_ip": ref["SQ4UniformComputeCodesIP"], "sq8u_ip": ref["SQ8UniformComputeCodesIP"]}
    values = t._primitive_values(fns)
    out = {"source": "vsag::generic::* compiled from src/simd/generic.cpp", "dims": t.DIMS, "seed": 47,
           "values": values}
    with open(os.path.join(HERE, "simd_generic.json"), "w") as f:
        json.dump(out, f, indent=0)
    print("wrote", len(values), "series of", len(t.DIMS), "values")


if __name__ == "__main__":
    main()
