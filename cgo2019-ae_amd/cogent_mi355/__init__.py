"""Python glue over the engine's C ABI (ctypes only; no compute happens here).

Mirrors the way the reference is driven: `HostTools.plan(...)` + `Plan.emit(...)`
stand for `python tc_code_generator.py <n> <input.in> <config#> <pre_computed> <dtype>`
(cogent/tc_code_generator.py:13-59), and `Expression.entry(...)` calls the
per-expression `sd_t_d2_fusion_` exactly as a driver's `main` does
(cogent/drivers/tccg/code_main_tccg_01.c:69), except that the three tensor
arguments are device addresses.

Nothing here falls back to a CPU implementation: a missing shared object raises.
"""
import ctypes
import json
import os

PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_DIR = os.path.join(PKG_DIR, "lib")
EXPR_DIR = os.path.join(PKG_DIR, "expressions")


class CogentError(RuntimeError):
    pass


def _one_hip_runtime():
    """PyTorch ships its own copy of the HIP runtime under the same soname as /opt/rocm's.  A process
    that is going to share device memory with torch must resolve the engine's objects against THAT
    copy, so torch is imported (when installed) before the first HIP-linked object is loaded; a second
    runtime in the same process finds no device."""
    try:
        import torch  # noqa: F401
    except ImportError:
        pass


def _load(path, hip=False):
    if hip:
        _one_hip_runtime()
    if not os.path.exists(path):
        raise CogentError("native library %s is missing: run __graft_entry__.build() (or cgo2019-ae_amd/build.py) first" % path)
    return ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)


def manifest():
    with open(os.path.join(EXPR_DIR, "manifest.json")) as f:
        return json.load(f)["expressions"]


def group_manifest():
    with open(os.path.join(EXPR_DIR, "manifest.json")) as f:
        return json.load(f).get("groups", [])


def manifest_entry(name):
    for e in manifest() + group_manifest():
        if e["name"] == name:
            return e
    raise KeyError(name)


def expression_text(name):
    with open(os.path.join(EXPR_DIR, manifest_entry(name)["file"])) as f:
        return f.read()


class Plan:
    """A parsed expression plus its gfx950 mapping (handle into libcogent_mi355.so)."""

    def __init__(self, tools, handle):
        self._tools = tools
        self._h = handle
        self.info = json.loads(tools.lib.cogent_plan_json(handle).decode())

    def __del__(self):
        try:
            if self._h:
                self._tools.lib.cogent_plan_destroy(self._h)
                self._h = None
        except Exception:
            pass

    @property
    def num_indices(self):
        return self._tools.lib.cogent_plan_num_indices(self._h)

    def _sizes(self, sizes):
        if len(sizes) != self.num_indices:
            raise CogentError("expected %d extents, got %d" % (self.num_indices, len(sizes)))
        return (ctypes.c_int * len(sizes))(*sizes)

    def flops(self, sizes):
        return self._tools.lib.cogent_plan_flops(self._h, self._sizes(sizes))

    def bytes(self, sizes):
        return self._tools.lib.cogent_plan_bytes(self._h, self._sizes(sizes))

    def candidates(self, k):
        return json.loads(self._tools.lib.cogent_plan_candidates_json(self._h, k).decode())

    def emit(self, unique_name, out_path):
        rc = self._tools.lib.cogent_plan_emit(self._h, unique_name.encode(), out_path.encode())
        if rc:
            raise CogentError(self._tools.last_error())


class HostTools:
    """libcogent_mi355.so: parser, mapping pass, emitter, seeded fill."""

    def __init__(self):
        lib = _load(os.path.join(LIB_DIR, "libcogent_mi355.so"))
        lib.cogent_plan_create.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p,
                                           ctypes.POINTER(ctypes.c_void_p)]
        lib.cogent_plan_create.restype = ctypes.c_int
        lib.cogent_plan_destroy.argtypes = [ctypes.c_void_p]
        lib.cogent_plan_destroy.restype = None
        lib.cogent_plan_json.argtypes = [ctypes.c_void_p]
        lib.cogent_plan_json.restype = ctypes.c_char_p
        lib.cogent_plan_candidates_json.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.cogent_plan_candidates_json.restype = ctypes.c_char_p
        lib.cogent_plan_num_indices.argtypes = [ctypes.c_void_p]
        lib.cogent_plan_num_indices.restype = ctypes.c_int
        lib.cogent_plan_flops.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        lib.cogent_plan_flops.restype = ctypes.c_longlong
        lib.cogent_plan_bytes.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        lib.cogent_plan_bytes.restype = ctypes.c_longlong
        lib.cogent_plan_emit.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p]
        lib.cogent_plan_emit.restype = ctypes.c_int
        lib.cogent_host_last_error.restype = ctypes.c_char_p
        lib.cogent_fill_uniform_f64.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_ulonglong]
        lib.cogent_fill_uniform_f64.restype = None
        lib.cogent_fill_uniform_f32.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_ulonglong]
        lib.cogent_fill_uniform_f32.restype = None
        self.lib = lib

    def last_error(self):
        return self.lib.cogent_host_last_error().decode()

    def plan(self, text, dtype="DOUBLE", config_rank=-1, mapping_spec=None):
        h = ctypes.c_void_p()
        rc = self.lib.cogent_plan_create(text.encode(), dtype.encode(), config_rank,
                                         mapping_spec.encode() if mapping_spec else None, ctypes.byref(h))
        if rc:
            err = CogentError(self.last_error())
            err.code = rc
            raise err
        return Plan(self, h)

    def fill_uniform(self, array, seed):
        """Fill a C-contiguous numpy float64/float32 array in place from `seed`."""
        import numpy as np
        if not array.flags["C_CONTIGUOUS"] and not array.flags["F_CONTIGUOUS"]:
            raise CogentError("fill_uniform needs a contiguous array")
        fn = {np.dtype("float64"): self.lib.cogent_fill_uniform_f64,
              np.dtype("float32"): self.lib.cogent_fill_uniform_f32}[array.dtype]
        fn(array.ctypes.data, array.size, seed)
        return array


class Expression:
    """One compiled per-expression object, lib/<name>.so."""

    def __init__(self, name=None, path=None):
        self.path = path or os.path.join(LIB_DIR, name + ".so")
        self.lib = _load(self.path, hip=True)
        self.lib.cogent_num_indices.restype = ctypes.c_int
        self.lib.cogent_last_error.restype = ctypes.c_char_p
        self.lib.cogent_expression.restype = ctypes.c_char_p
        self.lib.cogent_info.restype = ctypes.c_char_p
        self.n = self.lib.cogent_num_indices()
        self.lib.cogent_run.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        self.lib.cogent_run.restype = ctypes.c_int
        self.lib.cogent_run_noalloc.argtypes = self.lib.cogent_run.argtypes
        self.lib.cogent_run_noalloc.restype = ctypes.c_int
        for fn in (self.lib.sd_t_d2_fusion_, self.lib.sd_t_d2_fusion_host_):
            fn.argtypes = [ctypes.c_int] * self.n + [ctypes.c_void_p] * 3 + [ctypes.c_int, ctypes.c_int]
            fn.restype = ctypes.c_int
        self.expression = self.lib.cogent_expression().decode()
        self.info = json.loads(self.lib.cogent_info().decode())
        self.dtype = self.info["dtype"]

    @property
    def resources(self):
        """hipcc's resource report of the object's kernels, written next to it by build.py: {"hot": the instantiation that
        runs at the benchmark extents, "spilling": kernels with scratch use, "kernels": {name: {vgprs, scratch_bytes, ..}}}."""
        path = self.path[:-3] + ".resources.json"
        if not os.path.exists(path):
            raise CogentError("no resource report next to %s (built by hand?)" % self.path)
        with open(path) as f:
            return json.load(f)

    def last_error(self):
        return self.lib.cogent_last_error().decode()

    def last_kernel(self):
        """Kernel launched by this thread's last call: 'none', 'plain', 'tiled', 'stream' or 'valu'."""
        self.lib.cogent_last_kernel.restype = ctypes.c_int
        return ("none", "plain", "tiled", "stream", "valu")[self.lib.cogent_last_kernel()]

    def entry(self, sizes, c_ptr, a_ptr, b_ptr):
        """sd_t_d2_fusion_(size..., C, A, B, 1, -1) on device addresses; returns the status code."""
        if len(sizes) != self.n:
            raise CogentError("expected %d extents, got %d" % (self.n, len(sizes)))
        return self.lib.sd_t_d2_fusion_(*[int(s) for s in sizes], c_ptr, a_ptr, b_ptr, 1, -1)

    def entry_host(self, sizes, c_ptr, a_ptr, b_ptr):
        if len(sizes) != self.n:
            raise CogentError("expected %d extents, got %d" % (self.n, len(sizes)))
        return self.lib.sd_t_d2_fusion_host_(*[int(s) for s in sizes], c_ptr, a_ptr, b_ptr, 1, -1)

    def run(self, sizes, c_ptr, a_ptr, b_ptr, stream=None, variant=0):
        arr = (ctypes.c_int * len(sizes))(*[int(s) for s in sizes])
        return self.lib.cogent_run(arr, len(sizes), c_ptr, a_ptr, b_ptr, stream, variant)

    def run_noalloc(self, sizes, c_ptr, a_ptr, b_ptr, stream=None, variant=0):
        """cogent_run_noalloc: the same call, guaranteed not to allocate (repacked inputs go to the object's static scratch)."""
        arr = (ctypes.c_int * len(sizes))(*[int(s) for s in sizes])
        return self.lib.cogent_run_noalloc(arr, len(sizes), c_ptr, a_ptr, b_ptr, stream, variant)


class Group:
    """One compiled fused-group object: several contractions into one output, one kernel (lib/<name>.so)."""

    def __init__(self, name=None, path=None):
        self.path = path or os.path.join(LIB_DIR, name + ".so")
        self.lib = _load(self.path, hip=True)
        for fn in (self.lib.cogent_num_indices, self.lib.cogent_num_terms):
            fn.restype = ctypes.c_int
        for fn in (self.lib.cogent_last_error, self.lib.cogent_expression, self.lib.cogent_info):
            fn.restype = ctypes.c_char_p
        self.n = self.lib.cogent_num_indices()
        self.n_terms = self.lib.cogent_num_terms()
        for fn in (self.lib.sd_t_d2_fusion_, self.lib.sd_t_d2_fusion_host_):
            fn.argtypes = [ctypes.c_int] * self.n + [ctypes.c_void_p] * (1 + 2 * self.n_terms) + [ctypes.c_int] * (self.n_terms + 1)
            fn.restype = ctypes.c_int
        self.lib.cogent_run_group.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_void_p,
                                              ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.c_void_p]
        self.lib.cogent_run_group.restype = ctypes.c_int
        self.expressions = self.lib.cogent_expression().decode().split("\n")
        self.info = json.loads(self.lib.cogent_info().decode())
        self.dtype = self.info["dtype"]

    def last_error(self):
        return self.lib.cogent_last_error().decode()

    def _check(self, sizes, inputs):
        if len(sizes) != self.n:
            raise CogentError("expected %d extents, got %d" % (self.n, len(sizes)))
        if len(inputs) != 2 * self.n_terms:
            raise CogentError("expected %d input pointers, got %d" % (2 * self.n_terms, len(inputs)))

    def entry(self, sizes, c_ptr, inputs, enabled=None):
        """sd_t_d2_fusion_(size..., C, A1, B1, ..., AN, BN, cond_1..cond_N, -1) on device addresses."""
        self._check(sizes, inputs)
        flags = [1] * self.n_terms if enabled is None else [int(bool(v)) for v in enabled]
        return self.lib.sd_t_d2_fusion_(*[int(s) for s in sizes], c_ptr, *inputs, *flags, -1)

    def entry_host(self, sizes, c_ptr, inputs):
        self._check(sizes, inputs)
        return self.lib.sd_t_d2_fusion_host_(*[int(s) for s in sizes], c_ptr, *inputs, *([1] * self.n_terms), -1)

    def run(self, sizes, c_ptr, inputs, enabled=None, stream=None):
        arr = (ctypes.c_int * len(sizes))(*[int(s) for s in sizes])
        ptrs = (ctypes.c_void_p * len(inputs))(*inputs)
        en = None if enabled is None else (ctypes.c_int * len(enabled))(*[int(bool(v)) for v in enabled])
        return self.lib.cogent_run_group(arr, len(sizes), c_ptr, ptrs, len(inputs), en, stream)


class Driver:
    """libcogent_driver.so: HIP-event timing of a loaded expression object."""

    def __init__(self):
        lib = _load(os.path.join(LIB_DIR, "libcogent_driver.so"), hip=True)
        lib.cogent_driver_time.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.c_int,
                                           ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                           ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
        lib.cogent_driver_time.restype = ctypes.c_int
        lib.cogent_driver_time_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int,
                                                ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
        lib.cogent_driver_time_copy.restype = ctypes.c_int
        lib.cogent_driver_time_rmw.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_longlong, ctypes.c_int,
                                               ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
        lib.cogent_driver_time_rmw.restype = ctypes.c_int
        lib.cogent_driver_last_error.restype = ctypes.c_char_p
        self.lib = lib

    def time(self, expr, sizes, c_ptrs, a_ptr, b_ptr, warmup, iters, variant=0):
        arr = (ctypes.c_int * len(sizes))(*[int(s) for s in sizes])
        cb = (ctypes.c_void_p * len(c_ptrs))(*c_ptrs)
        each = (ctypes.c_float * iters)()
        stats = (ctypes.c_float * 5)()
        rc = self.lib.cogent_driver_time(expr.path.encode(), arr, len(sizes), cb, len(c_ptrs), a_ptr, b_ptr,
                                         warmup, iters, variant, each, stats)
        if rc:
            raise CogentError("timing failed (%d): %s" % (rc, self.lib.cogent_driver_last_error().decode()))
        return {"mean_ms": stats[0], "median_ms": stats[1], "min_ms": stats[2], "max_ms": stats[3], "batch_mean_ms": stats[4], "each_ms": list(each)}

    def time_group(self, group, sizes, c_ptrs, input_ptrs, warmup, iters):
        self.lib.cogent_driver_time_group.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.c_int,
                                                      ctypes.POINTER(ctypes.c_void_p), ctypes.c_int,
                                                      ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                      ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
        self.lib.cogent_driver_time_group.restype = ctypes.c_int
        arr = (ctypes.c_int * len(sizes))(*[int(s) for s in sizes])
        cb = (ctypes.c_void_p * len(c_ptrs))(*c_ptrs)
        ib = (ctypes.c_void_p * len(input_ptrs))(*input_ptrs)
        each = (ctypes.c_float * iters)()
        stats = (ctypes.c_float * 5)()
        rc = self.lib.cogent_driver_time_group(group.path.encode(), arr, len(sizes), cb, len(c_ptrs), ib, len(input_ptrs),
                                               warmup, iters, each, stats)
        if rc:
            raise CogentError("timing failed (%d): %s" % (rc, self.lib.cogent_driver_last_error().decode()))
        return {"mean_ms": stats[0], "median_ms": stats[1], "min_ms": stats[2], "max_ms": stats[3], "batch_mean_ms": stats[4], "each_ms": list(each)}

    def time_rmw(self, buf_ptrs, nbytes, mode, warmup, iters):
        """Mean ms per launch of a bare read-modify-write of nbytes: mode 0 flat, 1 flat non-temporal, 2 / 3 in the tiles of the
        streaming kernel on config 2's output (contiguous / interleaved runs)."""
        bufs = (ctypes.c_void_p * len(buf_ptrs))(*buf_ptrs)
        stats = (ctypes.c_float * 4)()
        rc = self.lib.cogent_driver_time_rmw(bufs, len(buf_ptrs), nbytes, mode, warmup, iters, stats)
        if rc:
            raise CogentError("read-modify-write timing failed (%d)" % rc)
        return stats[0]

    def time_copy(self, src_ptr, dst_ptr, nbytes, warmup, iters):
        stats = (ctypes.c_float * 4)()
        rc = self.lib.cogent_driver_time_copy(src_ptr, dst_ptr, nbytes, warmup, iters, stats)
        if rc:
            raise CogentError("copy timing failed (%d)" % rc)
        return stats[0]
