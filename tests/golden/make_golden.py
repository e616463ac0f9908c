"""Writes tests/golden/*.npz from the reference's OWN host check loops.

Run in the authoring container only (needs oracle/_ref, which oracle/Makefile builds from the
driver sources under /root/reference):  python tests/golden/make_golden.py

Each fixture holds seeded inputs (C_in, A, B) and C_out = what post_Correctness() of the named
reference driver leaves in its check buffer.  The fixtures are data; no reference source is kept.
"""
import ctypes
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

EXPR_DIR = os.path.join(os.path.dirname(os.path.dirname(HERE)), "cgo2019-ae_amd", "expressions")

# (fixture name, reference driver library, expression file or text, element type, extents)
CASES = [
    ("tccg01_3d_1k", "ref_tccg_01", "tccg_01.in", "f64", [5, 6, 3, 7]),
    ("tccg09_4d_1k", "ref_tccg_09", "tccg_09.in", "f64", [3, 4, 5, 2, 6]),
    ("tccg12_gemm", "ref_tccg_12", "tccg_12.in", "f64", [9, 7, 11]),
    ("tccg13_2d_2k", "ref_tccg_13", "tccg_13.in", "f64", [5, 4, 3, 6]),
    ("tccg20_4d_2k", "ref_tccg_20", "tccg_20.in", "f64", [3, 4, 2, 5, 3, 4]),
    ("tccg29_4d_2k", "ref_tccg_29", "tccg_29.in", "f64", [4, 3, 5, 2, 3, 4]),
    ("tccg31_6d_minus", "ref_tccg_31", "tccg_31.in", "f64", [3, 2, 4, 3, 2, 3, 5]),
    ("tccg40_6d", "ref_tccg_40", "tccg_40.in", "f64", [2, 3, 4, 3, 2, 3, 5]),
    ("tccg45_6d", "ref_tccg_45", "tccg_45.in", "f64", [3, 3, 2, 4, 2, 3, 4]),
    ("tccg43_6d_f32", "ref_float_tccg_43", "tccg_43.in", "f32", [3, 2, 4, 3, 2, 3, 5]),
    ("tccg48_6d_f32", "ref_float_tccg_48", "tccg_48.in", "f32", [2, 3, 3, 4, 3, 2, 6]),
]


def main():
    out = []
    for name, libname, exprfile, ty, sizes in CASES:
        lib = helpers.ref_lib(libname)
        if lib is None:
            raise SystemExit("oracle/_ref/%s.so missing: run make -C oracle" % libname)
        text = open(os.path.join(EXPR_DIR, exprfile)).read()
        expr = helpers.parse_expression(text)
        line = [l for l in text.splitlines() if not l.startswith("#")][0]
        dtype = np.float64 if ty == "f64" else np.float32
        nC, nA, nB = helpers.tensor_sizes(expr, sizes)
        A, B, C = helpers.uniform(nA, 11, dtype), helpers.uniform(nB, 12, dtype), helpers.uniform(nC, 13, dtype)
        chk, dummy = C.copy(), np.zeros_like(C)
        p = lambda x: x.ctypes.data_as(ctypes.c_void_p)
        lib.post_Correctness(p(dummy), p(chk), p(A), p(B), *[ctypes.c_int(s) for s in sizes])
        np.savez_compressed(os.path.join(HERE, name + ".npz"), C_in=C, A=A, B=B, C_out=chk)
        out.append({"name": name, "file": name + ".npz", "expression": line, "sizes": sizes, "dtype": ty,
                    "reference_driver": libname})
    with open(os.path.join(HERE, "cases.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", len(out), "fixtures")


if __name__ == "__main__":
    main()
