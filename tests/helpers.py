"""Test-side helpers: an independent reading of the expression grammar, the ctypes
binding of the CPU oracle (oracle/liboracle.so) and of the reference's own compiled
check loops (oracle/_ref/*.so), and the seeded input stream restated in numpy."""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
MAX_IDX = 16


def parse_expression(text):
    """Second, independent reading of the grammar (positional tokens after deleting '[', ']', ';'),
    used to drive the oracle and to check the C++ parser."""
    lines = [l for l in text.splitlines() if not l.startswith("#")]
    assert len(lines) == 1, "one expression expected"
    tok = lines[0].replace("[", "").replace("]", "").replace(";", "").split()
    out_pairs = tok[1].split(",")
    sum_pairs = tok[3].replace("sum(", "").replace(")", "").split(",")
    out_idx, rep = out_pairs[0::2], [int(v) for v in out_pairs[1::2]]
    sum_idx, rep_k = sum_pairs[0::2], [int(v) for v in sum_pairs[1::2]]
    return {
        "out": tok[0], "op": tok[2], "a": tok[5], "b": tok[8],
        "out_idx": out_idx, "sum_idx": sum_idx,
        "a_idx": tok[6].split(","), "b_idx": tok[9].split(","),
        "rep_sizes": rep + rep_k,
        "all_idx": out_idx + sum_idx,
    }


class TcDesc(ctypes.Structure):
    _fields_ = [("n_all", ctypes.c_int), ("extent", ctypes.c_int * MAX_IDX),
                ("n_out", ctypes.c_int), ("out_idx", ctypes.c_int * MAX_IDX),
                ("n_int", ctypes.c_int), ("int_idx", ctypes.c_int * MAX_IDX),
                ("n_a", ctypes.c_int), ("a_idx", ctypes.c_int * MAX_IDX),
                ("n_b", ctypes.c_int), ("b_idx", ctypes.c_int * MAX_IDX),
                ("sign", ctypes.c_int), ("last_lo", ctypes.c_int), ("last_hi", ctypes.c_int)]


def make_desc(expr, sizes, last_range=None):
    """expr: parse_expression() result; sizes: extents in entry-point order."""
    ids = {n: i for i, n in enumerate(expr["all_idx"])}
    assert len(sizes) == len(ids)
    d = TcDesc()
    d.n_all = len(ids)
    for i, s in enumerate(sizes):
        d.extent[i] = int(s)
    for field, cnt, names in (("out_idx", "n_out", expr["out_idx"]), ("int_idx", "n_int", expr["sum_idx"]),
                              ("a_idx", "n_a", expr["a_idx"]), ("b_idx", "n_b", expr["b_idx"])):
        setattr(d, cnt, len(names))
        arr = getattr(d, field)
        for j, n in enumerate(names):
            arr[j] = ids[n]
    d.sign = -1 if expr["op"] == "-=" else 1
    d.last_lo, d.last_hi = (0, 0) if last_range is None else last_range
    return d


def tensor_sizes(expr, sizes):
    ext = dict(zip(expr["all_idx"], sizes))
    n = lambda names: int(np.prod([ext[k] for k in names], dtype=np.int64))
    return n(expr["out_idx"]), n(expr["a_idx"]), n(expr["b_idx"])


class Oracle:
    def __init__(self):
        path = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/liboracle.so missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(path)
        for name, ct in (("tc_oracle_f64", ctypes.c_double), ("tc_oracle_f32", ctypes.c_float)):
            fn = getattr(lib, name)
            fn.argtypes = [ctypes.POINTER(TcDesc), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
            fn.restype = ctypes.c_int
        lib.tc_oracle_f32_acc64.argtypes = [ctypes.POINTER(TcDesc)] + [ctypes.c_void_p] * 4 + [ctypes.c_int]
        lib.tc_oracle_f32_acc64.restype = ctypes.c_int
        lib.tc_oracle_max_threads.restype = ctypes.c_int
        lib.tc_oracle_now.restype = ctypes.c_double
        self.lib = lib

    def max_threads(self):
        return self.lib.tc_oracle_max_threads()

    def contract(self, expr, sizes, C, A, B, threads=None, last_range=None):
        """In place: C <- C +/- sum(A*B) with the reference loop's summation order.  Flat arrays."""
        d = make_desc(expr, sizes, last_range)
        assert C.dtype == A.dtype == B.dtype and C.flags["C_CONTIGUOUS"]
        fn = self.lib.tc_oracle_f64 if C.dtype == np.float64 else self.lib.tc_oracle_f32
        rc = fn(ctypes.byref(d), C.ctypes.data, A.ctypes.data, B.ctypes.data, threads or self.max_threads())
        assert rc == 0
        return C

    def contract_f32_acc64(self, expr, sizes, Cin, A, B, threads=None):
        d = make_desc(expr, sizes)
        D = np.empty(Cin.size, dtype=np.float64)
        rc = self.lib.tc_oracle_f32_acc64(ctypes.byref(d), D.ctypes.data, Cin.ctypes.data, A.ctypes.data, B.ctypes.data,
                                          threads or self.max_threads())
        assert rc == 0
        return D


def ref_lib(name):
    """One of the reference's drivers compiled by oracle/Makefile, or None when not built."""
    path = os.path.join(ORACLE_DIR, "_ref", name + ".so")
    return ctypes.CDLL(path) if os.path.exists(path) else None


# ---- seeded inputs: numpy restatement of cogent_fill_uniform_* (splitmix64 of seed + (i+1)*golden)
def _mix64(z):
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def uniform(n, seed, dtype):
    with np.errstate(over="ignore"):
        i = np.arange(1, n + 1, dtype=np.uint64)
        z = _mix64(np.uint64(seed) + i * np.uint64(0x9E3779B97F4A7C15))
    if np.dtype(dtype) == np.float64:
        return 2.0 * ((z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)) - 1.0
    return (np.float32(2.0) * ((z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)) - np.float32(1.0)).astype(np.float32)


def einsum_reference(expr, sizes, Cin, A, B, acc_dtype=np.float64):
    """numpy restatement through Fortran-ordered views: C_in +/- einsum, in float64."""
    ext = dict(zip(expr["all_idx"], sizes))
    letters = {n: chr(ord("a") + i) for i, n in enumerate(expr["all_idx"])}
    shape = lambda names: tuple(ext[k] for k in names)
    sub = lambda names: "".join(letters[k] for k in names)
    a = A.astype(acc_dtype).reshape(shape(expr["a_idx"]), order="F")
    b = B.astype(acc_dtype).reshape(shape(expr["b_idx"]), order="F")
    r = np.einsum("%s,%s->%s" % (sub(expr["a_idx"]), sub(expr["b_idx"]), sub(expr["out_idx"])), a, b)
    sign = -1.0 if expr["op"] == "-=" else 1.0
    return Cin.astype(acc_dtype) + sign * r.reshape(-1, order="F")


def rel_error(got, ref):
    """max |got - ref| / max(|ref|, rms(ref)): the stated error measure (element-wise relative
    error with the denominator floored at the tensor's RMS so near-zero outputs do not blow it up)."""
    got = got.astype(np.float64)
    ref = ref.astype(np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    den = np.maximum(np.abs(ref), rms if rms > 0 else 1.0)
    return float(np.max(np.abs(got - ref) / den)) if ref.size else 0.0
