"""The C-ABI library loads and exports every symbol that include/pto_amd.h declares (no GPU needed)."""
import os
import re

from pto_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "pto_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(pto_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    lib = capi.load()
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert declared == set(capi.SYMBOLS), declared ^ set(capi.SYMBOLS)


def test_product_library_holds_no_test_entry_points():
    """Single-tile test programs and tuning hooks live in libpto_st.so (include/pto_amd_st.h) only."""
    import subprocess
    names = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = set(re.findall(r"\b(pto_[a-z0-9_]+)$", names, flags=re.M))
    assert exported == set(capi.SYMBOLS), exported ^ set(capi.SYMBOLS)


def test_test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "pto_amd_st.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(pto_[a-z0-9_]+)\s*\(", header))
    lib = capi.load_st()
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert declared == set(capi.ST_SYMBOLS), declared ^ set(capi.ST_SYMBOLS)


def test_argument_validation_needs_no_gpu():
    lib = capi.load()
    assert lib.pto_gemm_f16f32(0, 0, 0, 0, 128, 256, 64) == capi.ERR_BAD_ARG
    assert lib.pto_tcvt_f32_f16(0, 0, 0, 0, capi.CAST_RINT) == capi.OK          # empty input: nothing to do
    assert lib.pto_gather_rows(0, 0, 0, 0, 0, 0, 0, 2) == capi.OK
    assert lib.pto_version().startswith(b"pto-amd")
