"""The C-ABI libraries load and export every symbol include/cogent_mi355.h declares (no compute here),
and the command-line generator writes a translation unit whose entry point has the reference's shape."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cgo2019-ae_amd")
HEADER = os.path.join(ROOT, "include", "cogent_mi355.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(cogent_\w+)\s*\(", text)


def test_header_declarations_are_exported():
    names = declared_functions()
    host = ctypes.CDLL(os.path.join(PKG, "lib", "libcogent_mi355.so"))
    host_names = [n for n in names if n.startswith(("cogent_plan_", "cogent_fill_", "cogent_host_", "cogent_group_"))]
    assert len(host_names) >= 12
    for n in host_names:
        assert hasattr(host, n), n
    per_expression = [n for n in names if n not in host_names]
    assert set(per_expression) == {"cogent_run", "cogent_run_noalloc", "cogent_num_indices", "cogent_last_error", "cogent_last_kernel", "cogent_expression", "cogent_info"}


def test_every_expression_object_exports_the_entry_points():
    import cogent_mi355
    for e in cogent_mi355.manifest():
        path = os.path.join(PKG, "lib", e["name"] + ".so")
        assert os.path.exists(path), "%s not built" % path
        out = subprocess.run(["nm", "-D", "--defined-only", path], stdout=subprocess.PIPE, text=True, check=True).stdout
        syms = {l.split()[-1] for l in out.splitlines() if l.strip()}
        for s in ("sd_t_d2_fusion_", "sd_t_d2_fusion_host_", "cogent_run", "cogent_run_noalloc", "cogent_%s_run" % e["name"],
                  "cogent_num_indices", "cogent_last_error", "cogent_last_kernel", "cogent_expression", "cogent_info"):
            assert s in syms, (e["name"], s)


def test_no_benchmark_kernel_spills_registers():
    """build.py keeps hipcc's per-kernel resource report (the counterpart of the reference's `nvcc -Xptxas -v`,
    cogent/Makefile:16) next to every object and fails on a spilling kernel; here: the report exists for every object, names
    the instantiation its benchmark extents run, and that one uses no scratch memory and fits the register file."""
    import cogent_mi355
    for e in cogent_mi355.manifest():
        res = cogent_mi355.Expression.resources.fget(type("P", (), {"path": os.path.join(PKG, "lib", e["name"] + ".so")})())
        hot = res["hot"]
        assert hot in res["kernels"], (e["name"], hot)
        k = res["kernels"][hot]
        assert k["scratch_bytes"] == 0 or e.get("allow_scratch"), (e["name"], hot, k)
        assert 0 < k["vgprs"] + k.get("agprs", 0) <= 512 and k["occupancy"] >= 1
        if e["name"].startswith("cfg"):
            assert hot not in res["spilling"]
        # Kernels for other extents that spill: the one-K-block kernels for ragged tiles are taken out of use by
        # re-emitting the object with ok=0 ("rerouted"); nothing else may spill in a benchmark object.
        in_use = [k for k in res["spilling"] if k not in res.get("rerouted", [])]
        if not e["name"].startswith("var_"):
            assert in_use == [], (e["name"], in_use)
        if res.get("rerouted"):
            assert ";ok=0" in cogent_mi355.Expression(e["name"]).info["spec"]


def test_driver_library_exports():
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(PKG, "lib", "libcogent_driver.so")],
                         stdout=subprocess.PIPE, text=True, check=True).stdout
    for s in ("cogent_driver_time", "cogent_driver_time_group", "cogent_driver_time_copy", "cogent_driver_last_error"):
        assert s in out


def test_cli_takes_the_reference_arguments(tmp_path):
    """cogent_gen <number> <input.in> <config#> <pre_computed> <DOUBLE|FLOAT> writes temp__<number>.hip
    (the reference writes temp__<number>.cu, cogent/src/codes/tc_gen_code.py:27-30)."""
    gen = os.path.join(PKG, "bin", "cogent_gen")
    src = os.path.join(PKG, "expressions", "tccg_01.in")
    r = subprocess.run([gen, "01", src, "-1", "-1", "DOUBLE"], cwd=tmp_path, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stderr
    text = open(tmp_path / "temp__01.hip").read()
    # entry point: one int per index (output order, then summed), three pointers, two ints
    assert re.search(r"int sd_t_d2_fusion_\(int size_a, int size_b, int size_c, int size_d, double\* t3, double\* t2, "
                     r"double\* v2, int cond_kernel_1, int opt_register_transpose\)", text)
    r = subprocess.run([gen, "43", os.path.join(PKG, "expressions", "tccg_43.in"), "0", "-1", "FLOAT", "-o", str(tmp_path / "f.hip")],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stderr
    assert "float* t3, float* t2, float* v2" in open(tmp_path / "f.hip").read()
    # wrong argument count: the reference prints "Please check arguments" and exits (tc_code_generator.py:13-15)
    r = subprocess.run([gen, "01", src], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode != 0 and "Please check arguments" in r.stderr
    r = subprocess.run([gen, "01", src, "-1", "-1", "HALF"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 2


def test_missing_library_fails_loudly():
    import cogent_mi355
    with pytest.raises(cogent_mi355.CogentError):
        cogent_mi355.Expression("no_such_expression")
