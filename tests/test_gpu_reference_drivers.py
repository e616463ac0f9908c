"""The reference's own drivers, unmodified, running against this build (the drop-in demonstration).

oracle/Makefile compiles cogent/drivers/tccg/code_main_tccg_NN.c with its checker switched on
(-DDEBUG_CORRECTNESS), points the object's call to sd_t_d2_fusion_ at the host-pointer entry
sd_t_d2_fusion_host_ of lib/tccg_NN_f64.so, and links.  The driver allocates host tensors, fills them
with rand(), calls the entry point as it would call COGENT's generated code
(cogent/drivers/tccg/code_main_tccg_01.c:69) and checks the result with ITS host loop and ITS
tolerance (1e-8 absolute for fp64, 1e-5 for fp32; :135-157).  The 18 CCSD(T) drivers (cogent/drivers/ccsd_t) are linked
the same way against the single-term objects lib/ccsd_sd<d>_<k>_f64.so.  Skipped where the binaries were not built (the
reference tree is needed to build them, not to run them).
"""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
def n_indices(num):
    """Number of extents driver NN takes on its command line = indices of expressions/tccg_NN.in."""
    text = open(os.path.join(ROOT, "cgo2019-ae_amd", "expressions", "tccg_%02d.in" % num)).read()
    line = [l for l in text.splitlines() if l.strip() and not l.lstrip().startswith("#")][0]
    lhs, rhs = re.split(r"[-+]=", line)
    out = re.search(r"\[(.*?)\]", lhs).group(1).split(",")[0::2]
    summed = re.search(r"sum\((.*?)\)", rhs).group(1).split(",")[0::2]
    return len(out) + len(summed)


RAGGED = [11, 9, 6, 10, 7, 5, 12]
CASES = [
    ("drv_tccg_01", [40, 36, 24, 44]),                 # 3-D output, one contracted index
    ("drv_tccg_13", [37, 29, 31, 23]),                 # 2-D output, two contracted indices
    ("drv_tccg_20", [9, 10, 11, 12, 13, 14]),          # 4-D output, two contracted indices
    ("drv_tccg_31", [12, 8, 6, 12, 8, 6, 12]),         # 6-D output, "-="
    ("drv_tccg_40", [24, 16, 16, 16, 24, 16, 24]),     # 6-D output at the suite's own extents
    ("drv_float_tccg_43", [12, 8, 6, 12, 8, 6, 12]),   # fp32
    ("drv_tccg_01", []),                               # the driver's built-in default extents (16)
]
# ... and every driver of the corpus at ragged extents: 48 fp64, 9 fp32.  Drivers 33 and 34 are left out:
# their check loops ADD (cogent/drivers/tccg/code_main_tccg_33.c, _34.c) although input_tccg_33.in and
# _34.in say "-=", so the reference's own generated code would fail them too.
for _n in range(1, 49):
    if _n not in (33, 34):
        CASES.append(("drv_tccg_%02d" % _n, RAGGED[:n_indices(_n)]))
for _n in range(40, 49):
    CASES.append(("drv_float_tccg_%02d" % _n, RAGGED[:n_indices(_n)]))
# ... and the 18 CCSD(T) drivers (cogent/drivers/ccsd_t/code_main_sd1_1.c .. sd2_9.c): each calls the single-term entry
# point for its own term (code_main_sd2_1.c:112-114) and checks it with the one active line of its loop (tolerance 1e-4,
# :611-625), against lib/ccsd_sd<d>_<k>_f64.so.  Their command line is seven extents and the register-transpose option.
for _fam in ("sd1", "sd2"):
    for _k in range(1, 10):
        CASES.append(("drv_ccsd_%s_%d" % (_fam, _k), RAGGED + [1]))
CASES.append(("drv_ccsd_sd1_1", []))                   # built-in extents: all 16
CASES.append(("drv_ccsd_sd2_9", []))


@pytest.mark.parametrize("binary,sizes", CASES, ids=["%s-%s" % (b, "x".join(map(str, s)) or "default") for b, s in CASES])
def test_reference_driver_passes_its_own_check(binary, sizes):
    path = os.path.join(ROOT, "oracle", "_ref", binary)
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/%s not built" % binary)
    print("[gpu] %s %s" % (binary, sizes), flush=True)
    r = subprocess.run([path] + [str(s) for s in sizes], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-2000:]
    passed = re.search(r"PASSED:\s*([\d,']+)\s+among\s+([\d,']+)", r.stdout)
    errors = re.search(r"ERROR\s*:\s*([\d,']+)\s+among", r.stdout)
    assert passed and errors, r.stdout[-2000:]
    num = lambda s: int(re.sub(r"[,']", "", s))
    assert num(errors.group(1)) == 0, r.stdout[-2000:]
    assert num(passed.group(1)) == num(passed.group(2)) > 0
