"""Cases for running the reference's own per-instruction NPU test kernels (tests/npu/a2a3/src/st/testcase/<op>/<op>_kernel.cpp,
compiled unchanged through pto-isa_amd/port_ascend_source.py into build/ported/st/<op>.so by pto-isa_amd/build.py) on the
GPU.  Every explicit instantiation of a launcher that a kernel source exports is one case; its template arguments, read
from the demangled symbol, give the element type, the tile shapes and the valid region; launchers that are numbered cases
(`launch<OP>TestCase<N>`) take them from the case table that the build reads from the kernel source (manifest.json).  What
the launcher expects in memory is restated per test from the kernel source (cited), the expected result from the test's
generator (<op>/gen_data.py: plain numpy formulas)."""
import ctypes as C
import json
import os
import re
from types import SimpleNamespace

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ST_DIR = os.path.join(ROOT, "build", "ported", "st")

CTYPE = {"float": (np.float32, C.c_float), "int": (np.int32, C.c_int32), "short": (np.int16, C.c_int16),
         "unsigned short": (np.uint16, C.c_uint16), "signed char": (np.int8, C.c_int8), "unsigned char": (np.uint8, C.c_uint8),
         "unsigned int": (np.uint32, C.c_uint32), "long": (np.int64, C.c_int64),
         "_Float16": (np.float16, C.c_uint16), "unsigned long": (np.uint64, C.c_uint64)}
CTYPE.update({"int32_t": CTYPE["int"], "int16_t": CTYPE["short"], "uint16_t": CTYPE["unsigned short"], "uint32_t": CTYPE["unsigned int"],
              "int8_t": CTYPE["signed char"], "uint8_t": CTYPE["unsigned char"]})


def _ints(m, names):
    return {n: int(m.group(n).rstrip("u")) for n in names}


# ---- families: how the template arguments map to buffers -------------------------------------------------------------
# Every family returns (buffers, valid) with buffers = [(rows, leading dimension), ...] in argument order, output first,
# and valid = (rows, cols) of the region that is computed and stored.

def fam_g_t(p):        # <T, gRows, gCols, tRows, tCols, ...>: memory [gRows, gCols] contiguous (e.g. tabs_kernel.cpp:20-22)
    return (p.g0, p.g1), (p.g0, p.g1)


def fam_t_v_ld_tile(p):  # <T, tRows, tCols, vRows, vCols>, row stride tCols (tadd_kernel.cpp:20-21)
    return (p.v0, p.t1), (p.v0, p.v1)


def fam_t_v_ld_valid(p):  # <T, tRows, tCols, vRows, vCols>, row stride vCols (tor_kernel.cpp:20-21)
    return (p.v0, p.v1), (p.v0, p.v1)


UNARY = r"<(?P<T>[a-z ]+), (?P<g0>\d+), (?P<g1>\d+), (?P<t0>\d+), (?P<t1>\d+)(?:, (?P<flag>true|false))?>\((?:[a-z ]+\*, ){2}void\*\)"
BINARY5 = r"<(?P<T>[a-z ]+), (?P<a>\d+), (?P<b>\d+), (?P<c>\d+), (?P<d>\d+)>\((?:[a-z ]+\*, ){3}void\*\)"
BINARY9 = (r"<(?P<T>[a-z ]+), (?P<dH>\d+), (?P<dW>\d+), (?P<aH>\d+), (?P<aW>\d+), (?P<bH>\d+), (?P<bW>\d+), (?P<vR>\d+), (?P<vC>\d+)>"
           r"\((?:[a-z ]+\*, ){3}void\*\)")
SCALAR7 = (r"<(?P<T>[a-z ]+), (?P<dH>\d+), (?P<dW>\d+), (?P<sH>\d+), (?P<sW>\d+), (?P<vR>\d+), (?P<vC>\d+)>"
           r"\((?:[a-z ]+\*, ){2}[a-z ]+, void\*\)")


def f64(x):
    return x.astype(np.float64)


def _shift_left(a, b):
    return np.left_shift(a, b.astype(a.dtype))


def _shift_right(a, b):
    return np.right_shift(a, b.astype(a.dtype))


def _fmod(a, b):
    if a.dtype.kind == "f":
        return np.fmod(f64(a), f64(b))
    return np.fmod(a, b)


def _remainder(a, b):
    if a.dtype.kind == "f":
        return np.remainder(f64(a), f64(b))
    return np.remainder(a, b)


def _prelu(a, b):
    return np.where(a > 0, a, a * b)


# name -> dict(launcher, regex tail, layout, inputs, expected, half, exact)
#   layout: 'g' (gRows, gCols, tRows, tCols), 'tile_ld' / 'valid_ld' (tRows, tCols, vRows, vCols), 'nine', 'scalar7'
#   inputs: 'any' | 'pos' | 'bits' | 'shift' | 'rem' ; half: `unsigned short` instantiations are fp16 (aclFloat16)
SPECS = {
    # unary, <T, gRows, gCols, tRows, tCols[, inPlace]> (tabs_kernel.cpp:17-44 and alike)
    "tabs": dict(fn="LaunchTAbs", tail=UNARY, layout="g", nin=1, inputs="any", half=True, op=lambda a: np.abs(a)),
    "tneg": dict(fn="LaunchTNeg", tail=UNARY, layout="g", nin=1, inputs="any", half=True, op=lambda a: -a),
    "tnot": dict(fn="LaunchTNot", tail=UNARY, layout="g", nin=1, inputs="bits", half=False, op=lambda a: ~a),
    "texp": dict(fn="LaunchTExp", tail=UNARY, layout="g", nin=1, inputs="any", half=True, op=lambda a: np.exp(f64(a))),
    "tlog": dict(fn="LaunchTLog", tail=UNARY, layout="g", nin=1, inputs="pos", half=True, op=lambda a: np.log(f64(a))),
    "tsqrt": dict(fn="LaunchTSqrt", tail=UNARY, layout="g", nin=1, inputs="pos", half=True, op=lambda a: np.sqrt(f64(a))),
    "trsqrt": dict(fn="LaunchTRsqrt", tail=UNARY, layout="g", nin=1, inputs="pos", half=True, op=lambda a: 1.0 / np.sqrt(f64(a))),
    "trecip": dict(fn="LaunchTRecip", tail=UNARY, layout="g", nin=1, inputs="pos", half=True, op=lambda a: 1.0 / f64(a)),
    "trelu": dict(fn="LaunchTRelu", tail=UNARY, layout="g", nin=1, inputs="any", half=True, op=lambda a: np.maximum(a, 0)),
    "tmov_vect": dict(fn="launchTMOV", tail=UNARY, layout="g", nin=1, inputs="any", half=True, op=lambda a: a),
    # binary, <T, gRows, gCols, tRows, tCols> (tdiv_kernel.cpp:17-45, tmul, tsub)
    "tsub": dict(fn="LaunchTSub", tail=BINARY5, layout="g", nin=2, inputs="any", half=True, op=lambda a, b: a - b),
    "tmul": dict(fn="LaunchTMul", tail=BINARY5, layout="g", nin=2, inputs="any", half=True, op=lambda a, b: a * b),
    "tdiv": dict(fn="LaunchTDiv", tail=BINARY5, layout="g", nin=2, inputs="pos", half=True, op=lambda a, b: f64(a) / f64(b)),
    # binary, <T, tRows, tCols, vRows, vCols>
    "tadd": dict(fn="LaunchTAdd", tail=BINARY5, layout="tile_ld", nin=2, inputs="any", half=True, op=lambda a, b: a + b),
    "tand": dict(fn="LaunchTAnd", tail=BINARY5, layout="valid_ld", nin=2, inputs="bits", half=False, op=lambda a, b: a & b),
    "tor": dict(fn="LaunchTOr", tail=BINARY5, layout="valid_ld", nin=2, inputs="bits", half=False, op=lambda a, b: a | b),
    "tshl": dict(fn="LaunchTShl", tail=BINARY5, layout="valid_ld", nin=2, inputs="shift", half=False, op=_shift_left),
    "tshr": dict(fn="LaunchTShr", tail=BINARY5, layout="valid_ld", nin=2, inputs="shift", half=False, op=_shift_right),
    "tprelu": dict(fn="LaunchTPrelu", tail=BINARY5, layout="valid_ld", nin=2, inputs="any", half=True, op=_prelu),
    # binary on tiles of three different widths, <T, dstH, dstW, src0H, src0W, src1H, src1W, vRows, vCols>: every buffer has
    # its tile's width as row stride (taddplus_kernel.cpp:17-51)
    "taddplus": dict(fn="LaunchTAdd", tail=BINARY9, layout="nine", nin=2, inputs="any", half=True, op=lambda a, b: a + b),
    "tfmod": dict(fn="LaunchTFMOD", tail=BINARY9, layout="nine", nin=2, inputs="rem", half=True, op=_fmod),
    # TREM: the NPU takes the sign of the divisor (a - floor(a / b) b, npu/a2a3/TRem.hpp:22-35; np.remainder in its
    # generator), the CPU simulation that of the dividend (ElementOp.h:145-156: % and fmod).  The test source is built
    # with PTO_TREM_FLOOR_FORM (the NPU's meaning) and runs the generator's range: dividends in [-1000, 1000)
    "trem": dict(fn="LaunchTREM", tail=BINARY9, layout="nine", nin=2, inputs="rem", half=True, op=_remainder),
    "txor": dict(fn="LaunchTXor", tail=BINARY9, layout="nine", nin=2, inputs="bits", half=False, op=lambda a, b: a ^ b),
    # tile (op) scalar, <T, dstH, dstW, srcH, srcW, vRows, vCols>, the scalar by value (tands_kernel.cpp:17-49)
    "tands": dict(fn="LaunchTAndS", tail=SCALAR7, layout="scalar7", nin=1, inputs="bits", half=False, op=lambda a, k: a & k),
    "tors": dict(fn="LaunchTOrS", tail=SCALAR7, layout="scalar7", nin=1, inputs="bits", half=False, op=lambda a, k: a | k),
    "txors": dict(fn="LaunchTXorS", tail=SCALAR7, layout="scalar7", nin=1, inputs="bits", half=False, op=lambda a, k: a ^ k),
    "tshls": dict(fn="LaunchTShlS", tail=SCALAR7, layout="scalar7", nin=1, inputs="shift", half=False, op=lambda a, k: np.left_shift(a, k)),
    "tshrs": dict(fn="LaunchTShrS", tail=SCALAR7, layout="scalar7", nin=1, inputs="shift", half=False, op=lambda a, k: np.right_shift(a, k)),
}


def manifest():
    path = os.path.join(ST_DIR, "manifest.json")
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        return json.load(f)


def _pattern(spec):
    return re.compile(r"^void " + re.escape(spec["fn"]) + spec["tail"] + "$")


def cases():
    """[(test, mangled symbol, demangled symbol)] for every launcher instantiation of every test in SPECS that was built."""
    out = []
    man = manifest()
    for test, spec in SPECS.items():
        pat = _pattern(spec)
        for mangled, demangled in sorted(man.get(spec.get("lib", test), {}).get("launchers", {}).items(), key=lambda kv: kv[1]):
            m = pat.match(demangled)
            if m and ("runnable" not in spec or spec["runnable"](spec, m)):
                out.append((test, mangled, demangled))
    return out


def _elem(tname, half):
    """numpy dtype and ctypes type of a C++ element type name (as demangled, or as written in a kernel source)."""
    dtype, ctype = CTYPE[tname]
    if tname in ("unsigned short", "uint16_t") and half:
        dtype = np.float16
    return np.dtype(dtype), ctype


def plan(test, demangled):
    """-> SimpleNamespace(dtype, outs [(dtype, (rows, ld))], ins [(dtype, (rows, ld))], regions [(rows, cols)] per output,
    scalar None | (ctypes type, value), expect(ins, scalar) -> [array per output], spec)"""
    spec = SPECS[test]
    m = _pattern(spec).match(demangled)
    if "planner" in spec:
        return spec["planner"](test, spec, m)
    dtype, ctype = _elem(m.group("T"), spec["half"])
    lay = spec["layout"]
    if lay == "g":
        p = SimpleNamespace(**_ints(m, ["g0", "g1", "t0", "t1"])) if "g0" in m.groupdict() else \
            SimpleNamespace(g0=int(m.group("a")), g1=int(m.group("b")), t0=int(m.group("c")), t1=int(m.group("d")))
        buf, valid = (p.g0, p.g1), (p.g0, p.g1)
        buffers = [buf] * (1 + spec["nin"])
    elif lay in ("tile_ld", "valid_ld"):
        t0, t1, v0, v1 = (int(m.group(k)) for k in "abcd")
        buf = (v0, t1 if lay == "tile_ld" else v1)
        buffers, valid = [buf] * (1 + spec["nin"]), (v0, v1)
    elif lay == "nine":
        q = _ints(m, ["dH", "dW", "aH", "aW", "bH", "bW", "vR", "vC"])
        buffers, valid = [(q["dH"], q["dW"]), (q["aH"], q["aW"]), (q["bH"], q["bW"])], (q["vR"], q["vC"])
    elif lay == "scalar7":
        q = _ints(m, ["dH", "dW", "sH", "sW", "vR", "vC"])
        buffers, valid = [(q["dH"], q["dW"]), (q["sH"], q["sW"])], (q["vR"], q["vC"])
    else:
        raise AssertionError(lay)
    scalar = None
    if lay == "scalar7":
        scalar = (ctype, 3 if spec["inputs"] == "shift" else 0x5A5A & int(np.iinfo(dtype).max))
    return _elementwise_plan(spec, dtype, buffers, valid, scalar)


def _elementwise_plan(spec, dtype, buffers, valid, scalar, scalar_first=False):
    """One output, spec['nin'] inputs of the same element type, the operation applied to the valid region."""
    vr, vc = valid
    op = spec["op"]

    def expect(ins, k):
        a = ins[0][:vr, :vc]
        if k is not None:
            k = dtype.type(k)
            return [op(k, a) if scalar_first else op(a, k)]
        return [op(a) if len(ins) == 1 else op(a, ins[1][:vr, :vc])]
    return SimpleNamespace(dtype=dtype, outs=[(dtype, buffers[0])], ins=[(dtype, b) for b in buffers[1:]], regions=[valid],
                           scalar=scalar, expect=expect, spec=spec, compare=None, flat_prefix=None, scalar_after_stream=False, ins_after_stream=0)


# ---- numbered cases: launch<OP>TestCase<N>(void *out, void *src, float scalar, stream) -> run<T, dstRows, dstCols, rows,
# validRows, cols, validCols[, srcDivScalar]> (tadds_kernel.cpp:17-45, tdivs_kernel.cpp:17-48): output buffer [dstRows,
# dstCols], input [rows, cols], the scalar converted from float inside the launcher
CASE_SCALAR = r"<(?P<case>\d+)u>\(void\*, void\*, float, ihipStream_t\*\)"
SRC_TYPES = {"float": "float", "half": "unsigned short", "__fp16": "unsigned short", "aclFloat16": "unsigned short", "int32_t": "int", "int16_t": "short",
             "uint16_t": "unsigned short", "uint32_t": "unsigned int", "int8_t": "signed char", "uint8_t": "unsigned char"}


def case_entry(test, m):
    return manifest()[test]["cases"][m.group("case")]


def plan_case_scalar(test, spec, m):
    e = case_entry(test, m)
    t = e["targs"]
    dtype, _ = _elem(SRC_TYPES[t[0]], True)
    dR, dC, rows, vR, cols, vC = (int(x) for x in t[1:7])
    scalar_first = len(t) > 7 and t[7] == "false"
    value = 7.0 if spec["inputs"] in ("rem", "rempos") else (3.0 if dtype.kind != "f" else 1.5)
    return _elementwise_plan(spec, dtype, [(dR, dC), (rows, cols)], (vR, vC), (C.c_float, value), scalar_first)


def _div(a, b):
    if np.asarray(a).dtype.kind == "f":
        return np.asarray(a, np.float64) / np.asarray(b, np.float64)
    return (np.asarray(a, np.int64) // np.asarray(b, np.int64)).astype(np.asarray(a).dtype)      # operands are positive


SPECS.update({
    "tadds": dict(fn="launchTADDSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="any", op=lambda a, k: a + k),
    "tsubs": dict(fn="launchTSUBSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="any", op=lambda a, k: a - k),
    "tmuls": dict(fn="launchTMULSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="any", op=lambda a, k: a * k),
    "tdivs": dict(fn="launchTDIVSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="pos", op=_div),
    "tmaxs": dict(fn="launchTMAXSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="any", op=lambda a, k: np.maximum(a, k)),
    "tfmods": dict(fn="launchTFMODSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="rem", op=_fmod),
    # TREMS: the NPU's meaning (the sign of the divisor), as "trem"
    "trems": dict(fn="launchTREMSTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="rem", op=_remainder),
    "tlrelu": dict(fn="launchTLRELUTestCase", tail=CASE_SCALAR, planner=plan_case_scalar, nin=1, inputs="any", op=_prelu),
})


def TAIL(ints, nptr, suffix="", ptr0=None):
    """Demangled `<T, int..., suffix>(T*, ... nptr pointers ..., void*)`; ptr0: type of the first pointer if it is not T."""
    ptrs = (re.escape(ptr0) + r"\*, " if ptr0 else "") + r"(?:[A-Za-z_0-9 ]+\*, ){%d}" % (nptr - (1 if ptr0 else 0))
    return r"<(?P<T>[A-Za-z_0-9 ]+)" + "".join(r", (?P<%s>-?\d+)u?" % n for n in ints) + suffix + r">\(" + ptrs + r"void\*\)"


def _plan(spec, outs, ins, regions, expect, scalar=None):
    return SimpleNamespace(dtype=ins[0][0] if ins else outs[0][0], outs=outs, ins=ins, regions=regions, scalar=scalar,
                           expect=lambda arrays, k: expect(arrays), spec=spec, compare=None, flat_prefix=None, scalar_after_stream=False, ins_after_stream=0)


# ---- column reductions: launchTCOLSUM<T, cols, srcRows, validRows[, binary]>: [validRows, cols] of a [srcRows, cols] buffer
# reduced to [1, cols] (tcolsum_kernel.cpp:17-50)
def plan_colreduce(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    cols, rows, vr = (int(m.group(k)) for k in ("cols", "rows", "vr"))
    return _plan(spec, [(dt, (1, cols))], [(dt, (rows, cols))], [(1, cols)], lambda a: [spec["op"](a[0][:vr])[None, :]])


def _sum0(a):
    return np.sum(a, axis=0, dtype=np.float64 if a.dtype.kind == "f" else a.dtype)


def _prod0(a):
    return np.prod(a, axis=0, dtype=np.float64 if a.dtype.kind == "f" else a.dtype)


# ---- TROWEXPAND: launchTROWEXPAND<T, rows, srcCols, srcValidCols, dstCols, dstValidCols>: column 0 of the source across
# the valid columns of the destination (trowexpand_kernel.cpp:19-43; the 32-byte-row form :45-72 has srcCols == 1)
def plan_rowexpand(test, spec, m):
    dt, _ = _elem(m.group("T"), False)
    rows, sc, svc, dc, dvc = (int(m.group(k)) for k in ("rows", "sc", "svc", "dc", "dvc"))
    return _plan(spec, [(dt, (rows, dc))], [(dt, (rows, sc))], [(rows, dvc)], lambda a: [np.repeat(a[0][:, :1], dvc, axis=1)])


# ---- dst = matrix (op) per-row operand: launchTRowExpandAdd[2]<T, validRows, validCols, rows, cols, matrixFirst>: the
# per-row operand is a [rows32, 1] column (first form) or [rows32, 32 bytes] rows of which element (r, c mod K) is used
# (second form), rows32 = validRows rounded up to 32 bytes of elements (trowexpandadd_kernel.cpp:17-88)
def plan_rowexpand_bin(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    vr, vc, rows, cols = (int(m.group(k)) for k in ("vr", "vc", "rows", "cols"))
    per = 32 // dt.itemsize
    r32 = -(-vr // per) * per
    K = per if m.group("two") else 1
    mat_first = m.group("flag") == "true"
    op = spec["op"]

    def expect(a):
        mat, row = a[0][:vr, :vc], a[1][:vr][:, np.arange(vc) % K]
        return [op(mat, row) if mat_first else op(row, mat)]
    return _plan(spec, [(dt, (rows, cols))], [(dt, (rows, cols)), (dt, (r32, K))], [(vr, vc)], expect)


# ---- dst = matrix (op) per-column operand: launchTColExpandAdd<T, dstRows, dstCols, 1, cols> (tcolexpandadd_kernel.cpp:17-56)
def plan_colexpand_bin(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    dr, dc, sr, sc = (int(m.group(k)) for k in ("dr", "dc", "sr", "sc"))
    return _plan(spec, [(dt, (dr, dc))], [(dt, (dr, dc)), (dt, (sr, sc))], [(dr, dc)], lambda a: [spec["op"](a[0], a[1][:1, :dc])])


def _expdif(a, b):
    return np.exp(f64(a - b))          # the difference in the tile's element type, as the instruction forms it


ROWBIN = r"(?P<two>2)?" + TAIL(["vr", "vc", "rows", "cols"], 3, r", (?P<flag>true|false)")
COLBIN = TAIL(["dr", "dc", "sr", "sc"], 3)
_ROWCOL_OPS = {"Add": ("any", lambda a, b: a + b), "Sub": ("any", lambda a, b: a - b), "Mul": ("any", lambda a, b: a * b),
               "Div": ("pos", lambda a, b: f64(a) / f64(b)), "Max": ("any", np.maximum), "Min": ("any", np.minimum),
               "Expdif": ("any", _expdif)}
for _name, (_kind, _op) in _ROWCOL_OPS.items():
    SPECS["trowexpand" + _name.lower()] = dict(fn="launchTRowExpand" + _name, tail=ROWBIN, planner=plan_rowexpand_bin, inputs=_kind, op=_op)
    SPECS["tcolexpand" + _name.lower()] = dict(fn="TColExpand%sTest::launchTColExpand%s" % (_name, _name), tail=COLBIN,
                                               planner=plan_colexpand_bin, inputs=_kind, op=_op)

COLRED = TAIL(["cols", "rows", "vr"], 2)
REDUCE_TOL = {"float32": 1e-5, "float16": 4e-3}            # the order of a reduction is the implementation's
REDUCE_ATOL = {"float32": 2e-5, "float16": 2e-2}           # sums of up to 31 values of magnitude up to 4 that may cancel
SPECS.update({
    "tcolsum": dict(fn="launchTCOLSUM", tail=TAIL(["cols", "rows", "vr"], 2, r", (?:true|false)"), planner=plan_colreduce, inputs="any",
                    op=_sum0, tol=REDUCE_TOL, atol=REDUCE_ATOL),
    "tcolmax": dict(fn="launchTCOLMAX", tail=COLRED, planner=plan_colreduce, inputs="any", op=lambda a: np.max(a, axis=0)),
    "tcolmin": dict(fn="launchTCOLMIN", tail=COLRED, planner=plan_colreduce, inputs="any", op=lambda a: np.min(a, axis=0)),
    "tcolprod": dict(fn="launchTCOLPROD", tail=COLRED, planner=plan_colreduce, inputs="small", op=_prod0, tol=REDUCE_TOL),
    "trowexpand": dict(fn="launchTROWEXPAND", tail=TAIL(["rows", "sc", "svc", "dc", "dvc"], 2), planner=plan_rowexpand, inputs="bits"),
})


# ---- comparisons into bit masks: LaunchTCmp<T, gRows, gCols, tRows, tCols, mode>(uint8 *out, T *src0, T *src1): the
# [tRows, tCols] corner of [gRows, gCols] buffers; byte b of an output row holds columns 8b .. 8b+7, lowest bit first
# (tcmp_kernel.cpp:17-48, gen_data.py:49-56).  LaunchTCmps compares with the scalar src1[0] (tcmps_kernel.cpp:17-42).
CMP = [np.equal, np.not_equal, np.less, np.less_equal, np.greater, np.greater_equal]       # pto::CmpMode 0..5


def plan_cmp(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    gr, gc, tr, tc, mode = (int(m.group(k)) for k in ("gr", "gc", "tr", "tc", "mode"))
    scalar_form = spec["scalar_form"]
    u8 = np.dtype(np.uint8)

    def expect(a):
        lhs, rhs = a[0][:tr, :tc], (a[1][0, 0] if scalar_form else a[1][:tr, :tc])
        return [np.packbits(CMP[mode](lhs, rhs), axis=1, bitorder="little")]
    return _plan(spec, [(u8, (gr, gc))], [(dt, (gr, gc)), (dt, (1, 8) if scalar_form else (gr, gc))], [(tr, tc // 8)], expect)


# ---- TSEL: LaunchTSel<T, rows, cols, validRows, validCols>(T *out, uint8 *mask, T *src0, T *src1): bit (r, c) set takes
# src0, clear takes src1; mask rows of ceil(validCols / 8) bytes (tsel_kernel.cpp:17-66, gen_data.py:31-47)
def plan_sel(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    vr, vc = int(m.group("vr")), int(m.group("vc"))
    mc = (vc + 7) // 8

    def expect(a):
        bits = np.unpackbits(a[0], axis=1, bitorder="little")[:, :vc].astype(bool)
        return [np.where(bits, a[1], a[2])]
    return _plan(spec, [(dt, (vr, vc))], [(np.dtype(np.uint8), (vr, mc), "bits"), (dt, (vr, vc)), (dt, (vr, vc))], [(vr, vc)], expect)


# ---- TTRI: LaunchTTri<T, upper, diagonal, tileRows, tileCols, validRows, validCols>(T *out): ones on and above (upper) or
# on and below (lower) the diagonal-th diagonal (ttri_kernel.cpp:17-33, gen_data.py:26-29)
def plan_tri(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    upper, diag, vr, vc = (int(m.group(k)) for k in ("upper", "diag", "vr", "vc"))
    ones = np.ones((vr, vc), dtype=dt)
    return _plan(spec, [(dt, (vr, vc))], [], [(vr, vc)], lambda a: [np.triu(ones, k=diag) if upper else np.tril(ones, k=diag)])


SPECS.update({
    "tcmp": dict(fn="LaunchTCmp", tail=TAIL(["gr", "gc", "tr", "tc"], 3, r", \(pto::CmpMode\)(?P<mode>\d)", ptr0="unsigned char"),
                 planner=plan_cmp, inputs="small", scalar_form=False),
    "tcmps": dict(fn="LaunchTCmps", tail=TAIL(["gr", "gc", "tr", "tc", "mode"], 3, ptr0="unsigned char"), planner=plan_cmp, inputs="small",
                  scalar_form=True),
    "tsel": dict(fn="LaunchTSel", tail=r"<(?P<T>[a-z ]+), (?P<r>\d+), (?P<c>\d+), (?P<vr>\d+), (?P<vc>\d+)>\([a-z ]+\*, unsigned char\*, [a-z ]+\*, [a-z ]+\*, void\*\)",
                 planner=plan_sel, inputs="any"),
    "ttri": dict(fn="LaunchTTri", tail=TAIL(["upper", "diag", "tr", "tc", "vr", "vc"], 1), planner=plan_tri, inputs="any"),
})


# ---- row reductions, numbered cases: launchTROWSUMTestCase<N>(void *out, void *src, stream) -> run<T, rows, validRows,
# srcCols, srcValidCols, 1>: out[r] = reduction of row r over the valid columns, as a vector of validRows elements
# (trowsum_kernel.cpp:17-45; :47-80 stores the same vector from a column-major [rows, 1] tile viewed as [1, rows])
CASE_UNARY = r"<(?P<case>\d+)u>\(void\*, void\*, ihipStream_t\*\)"


def plan_rowreduce(test, spec, m):
    t = case_entry(test, m)["targs"]
    dt, _ = _elem(SRC_TYPES[t[0]], True)
    rows, vr, sc, svc = (int(x) for x in t[1:5])
    return _plan(spec, [(dt, (1, rows))], [(dt, (rows, sc))], [(1, vr)], lambda a: [spec["op"](a[0][:vr, :svc])[None, :]])


SPECS.update({
    "trowsum": dict(fn="launchTROWSUMTestCase", tail=CASE_UNARY, planner=plan_rowreduce, inputs="any", tol=REDUCE_TOL,
                    atol={"float32": 2e-4, "float16": 5e-2}, op=lambda a: np.sum(a, axis=1, dtype=np.float64)),
    "trowmax": dict(fn="launchTROWMAXTestCase", tail=CASE_UNARY, planner=plan_rowreduce, inputs="any", op=lambda a: np.max(a, axis=1)),
    "trowmin": dict(fn="launchTROWMINTestCase", tail=CASE_UNARY, planner=plan_rowreduce, inputs="any", op=lambda a: np.min(a, axis=1)),
})


# ---- TCVT: launchTCVT<D, S, gRows, gCols, tRows, tCols>(D *dst, S *src): round to nearest even (CAST_RINT), values inside
# the destination's range (tcvt_kernel.cpp:19-66; gen_data.py draws [-100, 100] and [-10000, 10000])
def plan_cvt(test, spec, m):
    dd, _ = _elem(m.group("D"), True)
    sd, _ = _elem(m.group("T"), True)
    gr, gc = int(m.group("gr")), int(m.group("gc"))
    narrow = min(dd.itemsize, sd.itemsize) == 1
    kind = "cvt_u" if dd.kind == "u" else ("cvt_narrow" if narrow else "cvt")

    def expect(a):
        x = a[0]
        if sd.kind == "f" and dd.kind != "f":
            return [np.rint(x.astype(np.float64)).astype(dd)]
        return [x.astype(dd)]
    return _plan(spec, [(dd, (gr, gc))], [(sd, (gr, gc), kind)], [(gr, gc)], expect)


EXACT = {"float32": 0.0, "float16": 0.0}
SPECS["tcvt"] = dict(fn="launchTCVT", tail=r"<(?P<D>[a-z ]+), (?P<T>[a-z ]+), (?P<gr>\d+), (?P<gc>\d+), (?P<tr>\d+), (?P<tc>\d+)>\([a-z ]+\*, [a-z ]+\*, void\*\)",
                     planner=plan_cvt, inputs="cvt", tol=EXACT, atol=EXACT)


# ---- matmul: LaunchTMATMUL<N>(uint8 *out, uint8 *src0, uint8 *src1, stream) and LaunchTMATMULBIAS<N>(out, src0, src1, src2,
# stream) -> Run...<OutT, AT, BT, BiasT, m, k, n, bias | round mode>: [m, k] x [k, n] (+ bias[n]), every matrix dense and
# row-major in memory (tmatmul_kernel.cpp:113-197 and the split-k, GEMV and TF32 variants after it; :547-613 the cases)
def _bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _bf16_value(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def plan_matmul(test, spec, m):
    e = manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]
    t = e["targs"]
    names = {"half": np.float16, "float": np.float32, "int8_t": np.int8, "int32_t": np.int32, "bfloat16_t": np.uint16}
    out_dt, a_dt, bias_dt = np.dtype(names[t[0]]), np.dtype(names[t[1]]), np.dtype(names[t[3]])
    vm, vk, vn = (int(x) for x in t[4:7])
    bf16 = t[1] == "bfloat16_t"
    kind = "bf16" if bf16 else ("bits" if a_dt.kind == "i" else "unit")
    ins = [(a_dt, (vm, vk), kind), (a_dt, (vk, vn), kind)]
    if spec["bias"]:
        ins.append((bias_dt, (1, vn), "any" if bias_dt.kind == "i" else "unit"))

    def values(arrays):
        conv = (lambda x: _bf16_value(x).astype(np.float64)) if bf16 else (lambda x: x.astype(np.int64 if a_dt.kind == "i" else np.float64))
        return conv(arrays[0]), conv(arrays[1])

    def expect(arrays):
        a, b = values(arrays)
        c = a @ b
        if spec["bias"]:
            c = c + arrays[2].astype(c.dtype)
        return [c]
    pl = _plan(spec, [(out_dt, (vm, vn))], ins, [(vm, vn)], expect)
    # an fp32 accumulation over k against the exact product: relative to the magnitude of the row-by-column sum
    pl.compare = None if out_dt.kind == "i" else (
        lambda got, want, arrays: np.max(np.abs(got.astype(np.float64) - want) / (np.abs(values(arrays)[0]) @ np.abs(values(arrays)[1]) + 1.0)) < 2e-3)
    return pl


CASE_MATMUL = r"<(?P<case>\d+)>\((?:unsigned char\*, ){%d}void\*\)"
SPECS["tmatmul"] = dict(fn="LaunchTMATMUL", lib="tmatmul", tail=CASE_MATMUL % 3, planner=plan_matmul, inputs="unit", bias=False)
SPECS["tmatmul:bias"] = dict(fn="LaunchTMATMULBIAS", lib="tmatmul", tail=CASE_MATMUL % 4, planner=plan_matmul, inputs="unit", bias=True)


# ---- TMOV / TEXTRACT windows: launchTMOV<N> / launchTEXTRACT<N> / launchTEXTRACT_COMPACT<N>(uint8 *out, uint8 *src0,
# uint8 *src1, stream): out[M - iM, N - iN] = A[iM:M, iK:K] x B[iK:K, iN:N] with A [baseM, baseK] and B [baseK, baseN] in
# memory (base = M, K, N where the case names none), each row-major or, "transposed", column-major (textract_kernel.cpp:
# 17-74 runTMOV, :76-148 unaligned, :150-220 runTEXTRACT, :222-294 unaligned, :296-364 run-time valid, :366-442 compact)
def _extract_case(spec, m):
    return manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]


def _extract_dims(e):
    c = e["consts"]
    M, N, K = int(c["M"]), int(c["N"]), int(c["K"])
    return dict(M=M, N=N, K=K, iM=int(c.get("indexM", 0)), iN=int(c.get("indexN", 0)), iK=int(c.get("indexK", 0)),
                bM=int(c.get("baseM", M)), bN=int(c.get("baseN", N)), bK=int(c.get("baseK", K)),
                ta=c["isAtranspose"] == "true", tb=c["isBtranspose"] == "true")


def extract_runnable(spec, m):
    """False for the cases whose L1 tiles need more than a compute unit's 160 KiB of LDS (A at 0, B at 64 KiB)"""
    e = _extract_case(spec, m)
    d = _extract_dims(e)
    size = {"half": 2, "bfloat16_t": 2, "float": 4, "int8_t": 1}[e["targs"][1]]
    return 64 * 1024 + d["bK"] * d["bN"] * size <= 160 * 1024 and d["bM"] * d["bK"] * size <= 64 * 1024


def plan_extract(test, spec, m):
    e = _extract_case(spec, m)
    d = _extract_dims(e)
    names = {"half": np.float16, "float": np.float32, "int8_t": np.int8, "int32_t": np.int32, "bfloat16_t": np.uint16}
    out_dt, a_dt = np.dtype(names[e["targs"][0]]), np.dtype(names[e["targs"][1]])
    bf16 = e["targs"][1] == "bfloat16_t"
    kind = "bf16" if bf16 else ("bits" if a_dt.kind == "i" else "unit")
    shape_a = (d["bK"], d["bM"]) if d["ta"] else (d["bM"], d["bK"])
    shape_b = (d["bN"], d["bK"]) if d["tb"] else (d["bK"], d["bN"])
    vm, vn = d["M"] - d["iM"], d["N"] - d["iN"]

    def values(arrays):
        conv = (lambda x: _bf16_value(x).astype(np.float64)) if bf16 else (lambda x: x.astype(np.int64 if a_dt.kind == "i" else np.float64))
        a, b = conv(arrays[0]), conv(arrays[1])
        a = a.T if d["ta"] else a
        b = b.T if d["tb"] else b
        return a[d["iM"]:d["M"], d["iK"]:d["K"]], b[d["iK"]:d["K"], d["iN"]:d["N"]]

    def expect(arrays):
        a, b = values(arrays)
        return [a @ b]
    pl = _plan(spec, [(out_dt, (vm, vn))], [(a_dt, shape_a, kind), (a_dt, shape_b, kind)], [(vm, vn)], expect)
    pl.compare = None if out_dt.kind == "i" else (
        lambda got, want, arrays: np.max(np.abs(got.astype(np.float64) - want) / (np.abs(values(arrays)[0]) @ np.abs(values(arrays)[1]) + 1.0)) < 2e-3)
    return pl


for _fn in ("launchTMOV", "launchTEXTRACT", "launchTEXTRACT_COMPACT"):
    SPECS["textract:" + _fn] = dict(fn=_fn, lib="textract", tail=CASE_MATMUL % 3, planner=plan_extract, inputs="unit", runnable=extract_runnable)


# ---- TMAX / TMIN: LaunchTMax<T, gRows, gCols, tileRows, tileCols, validRows, validCols, pad>: the valid corner of
# [gRows, gCols] buffers (tmax_kernel.cpp:39-66); LaunchTMins (TMIN on tiles of three widths, tmins_kernel.cpp:39-75) is the
# nine-argument form with the pad value as a tenth
def plan_g_valid(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    gr, gc, vr, vc = (int(m.group(k)) for k in ("gr", "gc", "vr", "vc"))
    return _elementwise_plan(spec, dt, [(gr, gc)] * 3, (vr, vc), None)


def plan_nine_pad(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    q = _ints(m, ["dH", "dW", "aH", "aW", "bH", "bW", "vR", "vC"])
    return _elementwise_plan(spec, dt, [(q["dH"], q["dW"]), (q["aH"], q["aW"]), (q["bH"], q["bW"])], (q["vR"], q["vC"]), None)


# ---- TEXPANDS: LaunchTExpandS<T, gRows, gCols, tileRows, tileCols, validRows, validCols, pad>(void *out, float scalar):
# the scalar, converted to T, over the valid corner (texpands_kernel.cpp:38-58)
def plan_expands(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    gr, gc, vr, vc = (int(m.group(k)) for k in ("gr", "gc", "vr", "vc"))
    value = 2.5 if dt.kind == "f" else 7.0
    return _plan(spec, [(dt, (gr, gc))], [], [(vr, vc)], lambda a: [np.full((vr, vc), dt.type(value))], scalar=(C.c_float, value))


# ---- TSELS: LaunchTSels<T, TMask, dstH, dstW, maskH, maskW, srcH, srcW, validRows, validCols>(T *out, TMask *mask, T *src,
# T scalar): bit (r, c) of mask row r, read as bytes, takes src, a clear bit the scalar (tsels_kernel.cpp:17-60,
# gen_data.py:38-45); LaunchTSelsHalf the same on fp16 with the scalar's bit pattern by value
def plan_sels(test, spec, m):
    half = m.group("half") is not None
    dt, ct = _elem("unsigned short" if half else m.group("T"), half)
    mdt, _ = _elem(m.group("M"), False)
    q = _ints(m, ["dH", "dW", "mH", "mW", "sH", "sW", "vR", "vC"])
    vr, vc = q["vR"], q["vC"]
    value = 1.5 if dt.kind == "f" else 12345
    if half:
        scalar = (C.c_uint16, int(np.float16(value).view(np.uint16)))
    else:
        scalar = (ct, value)

    def expect(a):
        bits = np.unpackbits(np.ascontiguousarray(a[0]).view(np.uint8).reshape(a[0].shape[0], -1), axis=1, bitorder="little")[:vr, :vc].astype(bool)
        return [np.where(bits, a[1][:vr, :vc], dt.type(value))]
    return _plan(spec, [(dt, (q["dH"], q["dW"]))], [(mdt, (q["mH"], q["mW"]), "bits"), (dt, (q["sH"], q["sW"]), "any")], [(vr, vc)],
                 expect, scalar=scalar)


GVALID = TAIL(["gr", "gc", "tr", "tc", "vr", "vc", "pad"], 3)
SPECS.update({
    "tmax": dict(fn="LaunchTMax", tail=GVALID, planner=plan_g_valid, nin=2, inputs="any", op=np.maximum),
    "tmin": dict(fn="LaunchTMin", tail=GVALID, planner=plan_g_valid, nin=2, inputs="any", op=np.minimum),
    "tmins": dict(fn="LaunchTMins", tail=TAIL(["dH", "dW", "aH", "aW", "bH", "bW", "vR", "vC", "pad"], 3), planner=plan_nine_pad, nin=2,
                  inputs="any", op=np.minimum),
    "texpands": dict(fn="LaunchTExpandS", tail=r"<(?P<T>[a-z ]+), (?P<gr>\d+), (?P<gc>\d+), (?P<tr>\d+), (?P<tc>\d+), (?P<vr>\d+), (?P<vc>\d+), -?\d+>\(void\*, float, void\*\)",
                     planner=plan_expands, inputs="any"),
    "tsels": dict(fn="LaunchTSels", inputs="any", planner=plan_sels,
                  tail=r"(?P<half>Half)?<(?:(?P<T>[a-z ]+), )?(?P<M>unsigned [a-z]+), (?P<dH>\d+), (?P<dW>\d+), (?P<mH>\d+), (?P<mW>\d+), (?P<sH>\d+), "
                       r"(?P<sW>\d+), (?P<vR>\d+), (?P<vC>\d+)>\([a-z ]+\*, [a-z ]+\*, [a-z ]+\*, [a-z ]+, void\*\)"),
})


# ---- TGATHER, mask form: LaunchTGATHER<T, gRows, gCols, tileRows, tileCols, pattern>(T *out, T *src): the selected columns
# of every row (every 2nd or 4th from a phase, or all), packed in running order from the start of the output
# (tgather_kernel.cpp:21-46, gen_data.py:98-116); what follows the packed elements in the output is not defined
def plan_gather_mask(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    gr, gc, p = int(m.group("gr")), int(m.group("gc")), int(m.group("pattern"))
    step, phase = (1, 0) if p == 7 else ((2, p - 1) if p <= 2 else (4, p - 3))
    n = gr * len(range(phase, gc, step))
    pl = _plan(spec, [(dt, (gr, gc))], [(dt, (gr, gc), "pos")], [(gr, gc)], lambda a: [a[0][:, phase::step].reshape(-1)])
    pl.flat_prefix = n
    return pl


# ---- TSORT32: launchTSORT32<N>(uint64 *out, uint64 *src, uint32 *idx, uint64 *tmp) -> runTSORT32<T, rows, cols, validRows,
# validCols, alignedCols>: every group of 32 valid columns of a row in descending order of score, as (score, index)
# structures of 8 bytes (tsort32_kernel.cpp:22-75; the oracle's tsort32 is the expectation)
def _const_value(expr, consts):
    expr = expr.replace("sizeof(float)", "4").replace("sizeof(half)", "2").replace("/", "//")
    if not re.fullmatch(r"[\w\s+\-*/()]+", expr):
        raise ValueError(expr)
    names = {k: _const_value(v, consts) for k, v in consts.items() if re.search(r"\b%s\b" % k, expr)}
    return int(eval(expr, {"__builtins__": {}}, names))


def plan_sort32(test, spec, m):
    e = manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]
    c = e["consts"]
    rows, cols, vr, vc, ac = (_const_value(c[k], c) for k in ("ROWS", "COLS", "VALID_R", "VALID_C", "ALIGN_C"))
    dt = np.dtype(np.float32 if e["targs"][0] == "float" else np.float16)
    per = 8 // dt.itemsize

    def expect(a):
        import sys
        sys.path.insert(0, ROOT)
        from oracle import oracle
        dst = np.zeros((rows, per * cols), dtype=dt)
        return [oracle.tsort32(dst, a[0], a[1], vr, vc)[:vr, :per * vc]]
    pl = _plan(spec, [(dt, (rows, per * cols))], [(dt, (rows, cols), "scores"), (np.dtype(np.uint32), (rows, cols), "index"), (dt, (1, ac), "any")],
               [(vr, per * vc)], expect)
    bits = {2: np.uint16, 4: np.uint32}[dt.itemsize]
    pl.compare = lambda got, want, arrays: np.array_equal(np.ascontiguousarray(got).view(bits), np.ascontiguousarray(want).view(bits))
    return pl


SPECS["tgather"] = dict(fn="LaunchTGATHER", tail=TAIL(["gr", "gc", "tr", "tc"], 2, r", \(pto::MaskPattern\)(?P<pattern>\d)"), planner=plan_gather_mask, inputs="pos")
SPECS["tsort32"] = dict(fn="launchTSORT32", lib="tsort32", planner=plan_sort32, inputs="any",
                        tail=r"<(?P<case>\d+)>\(unsigned long\*, unsigned long\*, unsigned int\*, unsigned long\*, void\*\)")


# ---- TMRGSORT (tmrgsort_kernel.cpp): every launcher takes float pointers; T = uint16_t runs the half kernels with all column
# counts doubled (:261-297), so a "column" below is 4 bytes and a structure (score, index) two of them.
#   LanchTMrgsortMulti<T, gRows, gCols, rows, cols0, cols1, cols2, cols3, topk, lists, exhausted>: 2-4 sorted lists merged (:65-114)
#   LanchTMrgsortSingle<T, gRows, gCols, rows, cols, blockLen>: every four blocks of one source merged (:116-148)
#   LanchTMrgsortTopK<T, gRows, gCols, rows, cols, topk>: sorted blocks of 64 columns merged all the way, first topk kept (:194-258)
def _sort_struct_lists(rng, half, counts, distinct=False):
    """sorted lists of `counts` structures each, as arrays of the kernel's element type"""
    import sort_cases as SC
    out = []
    for tag, n in enumerate(counts):
        l = SC.sorted_list_16(rng, n, "f16", tag) if half else SC.sorted_list(rng, n, tag=tag)
        out.append(np.ascontiguousarray(l).reshape(1, -1))
    return out


def _oracle():
    import sys
    if ROOT not in sys.path:
        sys.path.insert(0, ROOT)
    from oracle import oracle
    return oracle


def plan_mrgsort(test, spec, m):
    half = m.group("T") == "unsigned short"
    dt = np.dtype(np.float16 if half else np.float32)
    coef = 2 if half else 1                     # elements of T per 4-byte column
    bits = np.uint16 if half else np.uint32
    form = spec["form"]
    exact = lambda got, want, arrays: np.array_equal(np.ascontiguousarray(got).view(bits), np.ascontiguousarray(want).view(bits))
    if form == "multi":
        gc, c0, c1, c2, c3, topk, nl = (int(m.group(k)) for k in ("gc", "c0", "c1", "c2", "c3", "topk", "lists"))
        exhausted = m.group("exh") == "true"
        cols = [c0, c1, c2, c3][:nl]
        ins = [(dt, (1, max(c, 8) * coef), ("sorted", c // 2, j)) for j, c in enumerate([c0, c1, c2, c3])]

        def expect(a):
            dst0 = np.zeros(topk * coef, dtype=dt)
            dst, counts = _oracle().tmrgsort_lists(dst0, [a[j][0, :cols[j] * coef] for j in range(nl)], [c * coef for c in cols], topk * coef, exhausted)
            n = int(sum(counts)) * 2 * coef
            return [dst[:n]]
        pl = _plan(spec, [(dt, (1, max(topk, gc * nl) * coef))], ins, [(1, topk * coef)], expect)
        pl.flat_prefix, pl.compare = -1, exact          # -1: as long as the expectation
        return pl
    gc, tc = int(m.group("gc")), int(m.group("tc"))
    if form == "single":
        block = int(m.group("block"))
        ins = [(dt, (1, gc * coef), ("blocks", block // 2, tc // 2))]
        pl = _plan(spec, [(dt, (1, gc * coef))], ins, [(1, tc * coef)],
                   lambda a: [_oracle().tmrgsort_blocks(np.zeros(tc * coef, dtype=dt), a[0][0, :tc * coef], tc * coef, block * coef)[None, :]])
        pl.compare = exact
        return pl
    topk = int(m.group("topk"))
    ins = [(dt, (1, gc * coef), ("blocks_distinct", 32, tc // 2))]

    def expect_topk(a):
        per = 2 * coef
        structs = a[0][0, :tc * coef].reshape(-1, per)
        order = np.argsort(-structs[:, 0].astype(np.float64), kind="stable")
        return [structs[order][:topk // 2].reshape(-1)]
    pl = _plan(spec, [(dt, (1, gc * coef))], ins, [(1, topk * coef)], expect_topk)
    pl.flat_prefix, pl.compare = -1, exact
    return pl


def _sorted_inputs(rng, dt, shape, kind):
    """kind = ("sorted", structures, tag) | ("blocks", structures per block, structures) | ("blocks_distinct", ...)"""
    import sort_cases as SC
    half = dt == np.float16
    per = 4 if half else 2
    buf = np.zeros(shape, dtype=dt)
    if kind[0] == "sorted":
        n, tag = kind[1], kind[2]
        if n:
            l = SC.sorted_list_16(rng, n, "f16", tag) if half else SC.sorted_list(rng, n, tag=tag)
            buf[0, :n * per] = np.ascontiguousarray(l).reshape(-1)
        return buf
    blk, total = kind[1], kind[2]
    parts = []
    if kind[0] == "blocks":
        for b in range(total // blk):
            l = SC.sorted_list_16(rng, blk, "f16", b) if half else SC.sorted_list(rng, blk, tag=b)
            parts.append(np.ascontiguousarray(l).reshape(-1))
    else:                                      # all scores different, so that the merged order does not depend on how ties fall
        scores = rng.permutation(total).astype(np.float64) - total // 2
        for b in range(total // blk):
            sc = np.sort(scores[b * blk:(b + 1) * blk])[::-1]
            st = np.zeros((blk, per), dtype=dt)
            st[:, 0] = sc.astype(dt)
            ids = np.arange(b * blk, (b + 1) * blk, dtype=np.uint32)
            if half:
                st.view(np.uint16)[:, 2], st.view(np.uint16)[:, 3] = ids & 0xFFFF, ids >> 16
            else:
                st.view(np.uint32)[:, 1] = ids
            parts.append(st.reshape(-1))
    flat = np.concatenate(parts)
    buf[0, :flat.size] = flat
    return buf


_MRG_T = r"<(?P<T>float|unsigned short), \d+, (?P<gc>\d+), \d+, "
SPECS["tmrgsort:multi"] = dict(fn="LanchTMrgsortMulti", lib="tmrgsort", form="multi", planner=plan_mrgsort, inputs="any",
                               tail=_MRG_T + r"(?P<c0>\d+), (?P<c1>\d+), (?P<c2>\d+), (?P<c3>\d+), (?P<topk>\d+), (?P<lists>\d), (?P<exh>true|false)>\((?:float\*, ){5}void\*\)")
SPECS["tmrgsort:single"] = dict(fn="LanchTMrgsortSingle", lib="tmrgsort", form="single", planner=plan_mrgsort, inputs="any",
                                tail=_MRG_T + r"(?P<tc>\d+), (?P<block>\d+)u>\((?:float\*, ){2}void\*\)")
SPECS["tmrgsort:topk"] = dict(fn="LanchTMrgsortTopK", lib="tmrgsort", form="topk", planner=plan_mrgsort, inputs="any",
                              tail=_MRG_T + r"(?P<tc>\d+), (?P<topk>\d+)>\((?:float\*, ){2}void\*\)")


# ---- TSTORE (with the TLOAD in front of it): LaunchTStore<format, T, g0..g4, w0..w4>(T *out, T *src): the [g0..g4] corner of
# a dense [w0..w4] array goes through a Vec tile and back to the same places of out; format 0 = ND (rows stacked), 1 = DN
# (column-major tile, the last two dimensions swapped in memory), 2 = NZ (boxed tile) (tstore_kernel.cpp:19-117)
def plan_store(test, spec, m):
    dt, _ = _elem(m.group("T"), False)
    fmt = int(m.group("fmt"))
    g = [int(m.group("g%d" % k)) for k in range(5)]
    w = [int(m.group("w%d" % k)) for k in range(5)]
    total = int(np.prod(w))
    strides = [w[1] * w[2] * w[3] * w[4], w[2] * w[3] * w[4], w[3] * w[4], w[4], 1]
    if fmt == 1:
        strides[3], strides[4] = 1, w[3]
    idx = np.indices(g).reshape(5, -1)
    offsets = (idx * np.array(strides)[:, None]).sum(axis=0)

    def expect(a):
        out = np.full(total, 77, dtype=dt)
        out[offsets] = a[0].reshape(-1)[offsets]
        return [out[None, :]]
    return _plan(spec, [(dt, (1, total))], [(dt, (1, total), "bits")], [(1, total)], expect)


SPECS["tstore"] = dict(fn="LaunchTStore", planner=plan_store, inputs="bits",
                       tail=r"<(?P<fmt>\d), (?P<T>[a-z ]+)" + "".join(r", (?P<g%d>\d+)" % k for k in range(5)) + "".join(r", (?P<w%d>\d+)" % k for k in range(5)) +
                            r">\((?:[a-z ]+\*, ){2}void\*\)")


# ---- TCOLEXPAND: launchTCOLEXPAND<T, srcRows, srcCols, srcValidCols, dstRows, dstCols, dstValidRows, dstValidCols>: row 0 of
# the source down the valid rows of the destination (tcolexpand_kernel.cpp:17-46)
def plan_colexpand(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    sr, sc, dr, dc, dvr, dvc = (int(m.group(k)) for k in ("sr", "sc", "dr", "dc", "dvr", "dvc"))
    return _plan(spec, [(dt, (dr, dc))], [(dt, (sr, sc))], [(dvr, dvc)], lambda a: [np.repeat(a[0][:1, :dvc], dvr, axis=0)])


# ---- TTRANS: LaunchTTRANS<T, tileRows, tileCols, validRows, validCols>: out [tileCols, tileRows] gets the transpose of the
# valid corner of src [tileRows, tileCols] (ttrans_kernel.cpp:17-66)
def plan_trans(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    tr, tc, vr, vc = (int(m.group(k)) for k in ("tr", "tc", "vr", "vc"))
    return _plan(spec, [(dt, (tc, tr))], [(dt, (tr, tc))], [(vc, vr)], lambda a: [a[0][:vr, :vc].T])


# ---- TROWPROD, numbered cases -> run<T, dstRows, srcRows, validRows, srcCols, srcValidCols>: the product of every valid row as
# a vector (trowprod_kernel.cpp:17-48)
def plan_rowprod(test, spec, m):
    t = case_entry(test, m)["targs"]
    dt, _ = _elem(SRC_TYPES[t[0]], True)
    drows, srows, vr, sc, svc = (int(x) for x in t[1:6])
    return _plan(spec, [(dt, (1, drows))], [(dt, (srows, sc), "near1")], [(1, vr)],
                 lambda a: [np.prod(a[0][:vr, :svc].astype(np.float64), axis=1)[None, :]])


# ---- TPARTADD / TPARTMUL: LaunchTPartAdd<T, dstRows, dstCols, src0Rows, src0Cols, src1Rows, src1Cols> (dense buffers of
# exactly those extents, tpartadd_kernel.cpp:17-47); TPARTMAX / TPARTMIN: the same six extents followed by the six tile
# extents (tpartmax_kernel.cpp:17-52).  Where both sources have an element the operation, where one has it that element.
def plan_part(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    dr, dc, ar, ac, br, bc = (int(m.group(k)) for k in ("dr", "dc", "ar", "ac", "br", "bc"))
    op = spec["op"]

    def expect(a):
        out = np.zeros((dr, dc), dtype=np.float64 if dt.kind == "f" else dt)
        in0 = np.zeros((dr, dc), dtype=bool)
        in1 = np.zeros((dr, dc), dtype=bool)
        in0[:ar, :ac] = True
        in1[:br, :bc] = True
        x0 = np.zeros((dr, dc), dtype=out.dtype)
        x1 = np.zeros((dr, dc), dtype=out.dtype)
        x0[:min(ar, dr), :min(ac, dc)] = a[0][:dr, :dc]
        x1[:min(br, dr), :min(bc, dc)] = a[1][:dr, :dc]
        out = np.where(in0 & in1, op(x0, x1), np.where(in0, x0, np.where(in1, x1, 0)))
        return [out]
    return _plan(spec, [(dt, (dr, dc))], [(dt, (ar, ac)), (dt, (br, bc))], [(dr, dc)], expect)


PART6 = TAIL(["dr", "dc", "ar", "ac", "br", "bc"], 3)
PART12 = TAIL(["dr", "dc", "ar", "ac", "br", "bc", "t0", "t1", "t2", "t3", "t4", "t5"], 3)[:-len(r"void\*\)")] + r"ihipStream_t\*\)"
SPECS.update({
    "tcolexpand": dict(fn="launchTCOLEXPAND", tail=TAIL(["sr", "sc", "svc", "dr", "dc", "dvr", "dvc"], 2), planner=plan_colexpand, inputs="any"),
    "ttrans": dict(fn="LaunchTTRANS", tail=TAIL(["tr", "tc", "vr", "vc"], 2), planner=plan_trans, inputs="any"),
    "trowprod": dict(fn="launchTROWPRODTestCase", tail=CASE_UNARY, planner=plan_rowprod, inputs="near1", tol=REDUCE_TOL),
    "tpartadd": dict(fn="LaunchTPartAdd", tail=PART6, planner=plan_part, inputs="any", op=lambda a, b: a + b),
    "tpartmul": dict(fn="LaunchTPartMul", tail=PART6, planner=plan_part, inputs="any", op=lambda a, b: a * b),
    "tpartmax": dict(fn="LaunchTPartMax", tail=PART12, planner=plan_part, inputs="any", op=np.maximum),
    "tpartmin": dict(fn="LaunchTPartMin", tail=PART12, planner=plan_part, inputs="any", op=np.minimum),
})


# ---- the accumulator's way out with a conversion (the fix pipe): tmov_acc2mat (Acc -> Mat by TMOV / TEXTRACT / TINSERT,
# then Mat -> NZ memory) and tstore_acc2gm (Acc -> ND or NZ memory), plain, with one quantisation word, with one per column.
# The numpy model restates the generators' decoding of the word (tmov_acc2mat/gen_data.py:27-100, tstore_acc2gm/gen_data.py):
# bits 31..13 a float scale cut to 10 mantissa bits, 35..32 the int16 shift - 1, 45..37 an offset, 46 signed 8-bit result.
_FIX_NAMES = {"half": np.float16, "float": np.float32, "int8_t": np.int8, "uint8_t": np.uint8, "int16_t": np.int16, "int32_t": np.int32,
              "bfloat16_t": np.uint16, "uint64_t": np.uint64}


def fix_quant_model(acc, words, out_name):
    """acc [m, n] (float32 or int32), words: one uint64 or [n] of them -> the converted matrix (bf16 as its bits)"""
    q = np.broadcast_to(np.asarray(words, dtype=np.uint64), (acc.shape[1],))
    if out_name == "int16_t":
        shift = ((q >> np.uint64(32)) & np.uint64(0xF)).astype(np.int64) + 1
        return np.clip(acc.astype(np.int64) >> shift[None, :], -32768, 32767).astype(np.int16)
    scale = (q & np.uint64(0xFFFFE000)).astype(np.uint32).view(np.float32)
    y = acc.astype(np.float32) * scale[None, :]
    if out_name in ("int8_t", "uint8_t"):
        t = np.clip(np.rint(y), -256, 255).astype(np.int64) + ((q >> np.uint64(37)) & np.uint64(0x1FF)).astype(np.int64)[None, :]
        signed = ((q >> np.uint64(46)) & np.uint64(1)).astype(bool)[None, :]
        return np.where(signed, np.clip(t, -128, 127), np.clip(t, 0, 255)).astype(_FIX_NAMES[out_name])
    if out_name == "half":
        return np.clip(y, -65504, 65504).astype(np.float16)
    return _bf16_bits(y.astype(np.float64))


def fix_plain_model(acc, out_name):
    if out_name == "bfloat16_t":
        return _bf16_bits(acc.astype(np.float64))
    return acc.astype(_FIX_NAMES[out_name])


def fix_scalar_word(scalar, out_name):
    """the word the test kernels build from their float argument (tmov_acc2mat_kernel.cpp:270-283, tstore_acc2gm_kernel.cpp:230-234)"""
    if out_name == "int16_t":
        return np.uint64(((int(scalar) - 1) & 0xF) << 32)
    w = int(np.float32(scalar).view(np.uint32))
    if out_name in ("int8_t", "uint8_t"):
        w |= int(out_name == "int8_t") << 46
    return np.uint64(w)


def _nz(mat, block_cols):
    """[R, C] -> the NZ image [C / bc][R / 16][16][bc] as rows of bc"""
    r, c = mat.shape
    return mat.reshape(r // 16, 16, c // block_cols, block_cols).transpose(2, 0, 1, 3).reshape(-1, block_cols)


def _acc_of(arrays, a_name, vm, vk, vn):
    """the accumulator of the valid product (inputs are zero outside it): int32 for int8 operands, else float32 (exact: small integers)"""
    conv = (lambda x: _bf16_value(x).astype(np.int64)) if a_name == "bfloat16_t" else (lambda x: x.astype(np.int64))
    a, b = conv(arrays[0]), conv(arrays[1])
    c = a @ b
    return c.astype(np.int32 if a_name == "int8_t" else np.float32)


def plan_acc2mat(test, spec, m):
    e = manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]
    t = list(e["targs"])
    form = spec["form"]
    out_name, a_name = t[0], t[1]
    if form == "vector":
        del t[3]
    M, K, N, vm, vk, vn = (int(x) for x in t[3:9])
    opt = t[9:] + ["false", "0", "0", "false", "0", "0"][len(t) - 9:]
    relu, ir, ic, insert, drow, dcol = opt[0] == "true", int(opt[1]), int(opt[2]), opt[3] == "true", int(opt[4]), int(opt[5])
    out_dt, a_dt = np.dtype(_FIX_NAMES[out_name]), np.dtype(_FIX_NAMES[a_name])
    bc = 512 // (16 * out_dt.itemsize)
    rows, cols = (drow, dcol) if insert else (M - ir, N - ic)
    ins = [(a_dt, (M, K), ("corner", vm, vk)), (a_dt, (K, N), ("corner", vk, vn))]
    if form == "vector":
        ins.append((np.dtype(np.uint64), (1, N), ("words", out_name)))
    init_dt = out_dt if out_dt.kind != "f" and out_dt != np.uint16 else out_dt
    ins.append((init_dt, (rows, cols) if insert else (1, 16), "bits" if out_dt.kind in "iu" else "unit"))
    scalar = float(e["args"].rsplit(",", 1)[1]) if form == "scalar" else None

    def expect(arrays):
        acc = _acc_of(arrays, a_name, vm, vk, vn)
        if relu:
            acc = np.maximum(acc, 0)
        if form == "plain":
            g = fix_plain_model(acc, out_name)
        else:
            g = fix_quant_model(acc, arrays[2].reshape(-1) if form == "vector" else fix_scalar_word(scalar, out_name), out_name)
        if insert:
            full = arrays[-1].copy()
            full[ir:ir + M, ic:ic + N] = g
            g = full
        else:
            g = g[ir:, ic:]
        return [_nz(g, bc)]
    pl = _plan(spec, [(out_dt, (rows * cols // bc, bc))], ins, [(rows * cols // bc, bc)], expect)
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(want.dtype), want)
    return pl


for _fn, _form, _n in (("launchTMOVAcc2MatNZ2NZ", "plain", 4), ("launchTMOVAcc2MatSCQuantNz", "scalar", 4), ("launchTMOVAcc2MatFBQuantNz", "vector", 5)):
    SPECS["tmov_acc2mat:" + _fn] = dict(fn=_fn, lib="tmov_acc2mat", tail=CASE_MATMUL % _n, planner=plan_acc2mat, inputs="small", form=_form)


def plan_acc2gm(test, spec, m):
    e = manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]
    t = e["targs"]
    form, nz = spec["form"], spec["nz"]
    atomic, out_name, a_name = t[0] == "1", t[2], t[3]
    g = [int(x) for x in t[4:9]]
    w = [int(x) for x in t[9:14]]
    vm, vn, vk = (int(x) for x in t[14:17])
    relu = len(t) > 17 and t[17] == "1"
    out_dt, a_dt = np.dtype(_FIX_NAMES[out_name]), np.dtype(_FIX_NAMES[a_name])
    kind = ("corner", vm, vk, "bf16") if a_name == "bfloat16_t" else "small"
    ins = [(a_dt, (vm, vk), kind), (a_dt, (vk, vn), ("corner", vk, vn, "bf16") if a_name == "bfloat16_t" else "small")]
    if form == "vector":
        align = (vn * 8 + 127) // 128 * 128 // 8
        ins.append((np.dtype(np.uint64), (1, align), ("words", out_name)))
    scalar = 2.0 if form == "scalar" else None
    if nz:
        assert g == w
        rows, cols = g[2] * g[3], g[0] * g[1] * g[4]
        shape = region = (g[0] * g[1] * g[2] * g[3], g[4])
    else:
        assert g[:3] == [1, 1, 1] and w[:3] == [1, 1, 1]
        rows, cols = g[3], g[4]
        shape, region = (w[3], w[4]), (rows, cols)

    def expect(arrays):
        acc = _acc_of(arrays, a_name, vm, vk, vn)[:rows, :cols]
        if relu:
            acc = np.maximum(acc, 0)
        if form == "plain":
            r = fix_plain_model(acc, out_name)
        else:
            r = fix_quant_model(acc, arrays[2].reshape(-1)[:cols] if form == "vector" else fix_scalar_word(scalar, out_name), out_name)
        if atomic and out_name == "bfloat16_t":
            # the harness fills the output with the bits 77, a bf16 denormal of 7e-39: it is what is left where 0 is added
            # to it and vanishes in the rounding of every other sum
            r = np.where(_bf16_value(r) == 0, np.uint16(77), r)
        elif atomic:    # the harness fills the output with 77 before the launch
            r = (r.astype(np.float64 if out_dt.kind == "f" else np.int64) + 77).astype(out_dt)
        if nz:          # [col blocks][row blocks][rows of a block][columns of a block]
            r = r.reshape(rows, cols // g[4], g[4]).transpose(1, 0, 2).reshape(-1, g[4])
        return [r]
    pl = _plan(spec, [(out_dt, shape)], ins, [region], expect, scalar=(C.c_float, scalar) if form == "scalar" else None)
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(want.dtype), want)
    pl.scalar_after_stream = True
    return pl


for _fn, _form, _nzflag, _n in (("LaunchTStoreAcc2gmNz2nd", "plain", False, 3), ("LaunchTStoreAcc2gmNz2nz", "plain", True, 3),
                               ("LaunchTStoreAcc2gmVectorNz2nd", "vector", False, 4), ("LaunchTStoreAcc2gmVectorNz2nz", "vector", True, 4)):
    SPECS["tstore_acc2gm:" + _fn] = dict(fn=_fn, lib="tstore_acc2gm", tail=CASE_MATMUL % _n, planner=plan_acc2gm, inputs="small", form=_form, nz=_nzflag)
for _fn, _nzflag in (("LaunchTStoreAcc2gmScalarNz2nd", False), ("LaunchTStoreAcc2gmScalarNz2nz", True)):
    SPECS["tstore_acc2gm:" + _fn] = dict(fn=_fn, lib="tstore_acc2gm", tail=r"<(?P<case>\d+)>\((?:unsigned char\*, ){3}void\*, float\)", planner=plan_acc2gm,
                                         inputs="small", form="scalar", nz=_nzflag)


# ---- TFILLPAD / TFILLPAD_INPLACE / TFILLPAD_EXPAND: launchTFILLPAD<N>(out, src, log, stream); kernel N fixes
# <T, 1, 1, 1, rows, cols, tileRows, tileCols, dyn, load pad, fill pad[, inplace[, expand]]>: a [rows, cols] matrix in the
# corner of a [tileRows, tileCols] tile, the fill pad value around it (tfillpad_kernel.cpp:113-194; golden :316-363).  The
# kernel also writes three time stamps into `log`.
def _pad_value(dt, which):
    if dt.kind == "f":
        return dt.type(np.inf if which == "Max" else -np.inf)
    info = np.iinfo(dt)
    return dt.type(info.max if which == "Max" else info.min)


def plan_fillpad(test, spec, m):
    e = manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]
    t = e["targs"]
    dt = np.dtype({"float": np.float32, "uint16_t": np.uint16, "int16_t": np.int16, "int8_t": np.int8, "int32_t": np.int32}[t[0]])
    rows, cols, trows, tcols = (int(x) for x in t[4:8])
    pad = _pad_value(dt, t[10].split("::")[1])

    def expect(arrays):
        out = np.full((trows, tcols), pad, dtype=dt)
        out[:rows, :cols] = arrays[0]
        return [out]
    pl = _plan(spec, [(dt, (trows, tcols))], [(dt, (rows, cols), "any"), (np.dtype(np.uint64), (1, 128), "any")], [(trows, tcols)], expect)
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(np.uint8), want.view(np.uint8))
    return pl


SPECS["tfillpad"] = dict(fn="launchTFILLPAD", lib="tfillpad", tail=r"<(?P<case>\d+)>\(unsigned char\*, unsigned char\*, unsigned long\*, void\*\)", planner=plan_fillpad, inputs="any")


# ---- TQUANT, the a2a3 form: TQuantTest::LaunchTQuantInt8<rows, cols, mode, type>(dst, src, scale, stream, offset):
# int8 = clamp(rint(src * scale[row])), uint8 = clamp(rint(src * scale[row] + offset[row])), each step rounded to fp32
# (tquant_kernel.cpp:24-95, tquant/gen_data.py:22-60)
def plan_quant(test, spec, m):
    rows, cols, asym = int(m.group("r")), int(m.group("c")), m.group("q") == "1"
    dt = np.dtype(np.uint8 if asym else np.int8)

    def expect(arrays):
        y = arrays[0] * arrays[1]
        if asym:
            y = y + arrays[2]
        return [np.clip(np.rint(y), 0 if asym else -128, 255 if asym else 127).astype(dt)]
    f32 = np.dtype(np.float32)
    pl = _plan(spec, [(dt, (rows, cols))], [(f32, (rows, cols), ("range", -2.0, 2.0)), (f32, (rows, 1), ("range", 20.0, 90.0)),
                                             (f32, (rows, 1), ("range", 60.0, 160.0))], [(rows, cols)], expect)
    pl.ins_after_stream = 1
    return pl


SPECS["tquant"] = dict(fn="TQuantTest::LaunchTQuantInt8", planner=plan_quant, inputs="any",
                       tail=r"<(?P<r>\d+), (?P<c>\d+), 0, \(pto::QuantType\)(?P<q>[01])>\(std::conditional<.*>::type\*, float\*, float\*, void\*, float\*\)")


# ---- TDEQUANT: LaunchTDequant<float, S, dstRows, dstCols, srcRows, srcCols, validRows, validCols, paraRows, paraCols>(out, src,
# scale, offset, stream): out = (float(src) - offset[row]) * scale[row] on the valid region; every matrix has the row stride
# dstCols in memory, scale and offset paraCols (tdequant_kernel.cpp:20-57, tdequant/gen_data.py:12-46)
def plan_dequant(test, spec, m):
    src_dt, _ = _elem(m.group("T"), False)
    q = _ints(m, ["dr", "dc", "sr", "sc", "vr", "vc", "pr", "pc"])
    vr, vc = q["vr"], q["vc"]
    f32 = np.dtype(np.float32)

    def expect(arrays):
        return [(arrays[0][:, :vc].astype(np.float32) - arrays[2][:, :1]) * arrays[1][:, :1]]
    return _plan(spec, [(f32, (vr, q["dc"]))], [(src_dt, (vr, q["dc"]), "bits"), (f32, (vr, q["pc"]), ("range", 0.001, 1.0)),
                                                 (f32, (vr, q["pc"]), ("range", -128.0, 127.0))], [(vr, vc)], expect)


SPECS["tdequant"] = dict(fn="LaunchTDequant", planner=plan_dequant, inputs="any",
                         tail=r"<float, (?P<T>[a-z ]+)" + "".join(r", (?P<%s>\d+)" % k for k in ("dr", "dc", "sr", "sc", "vr", "vc", "pr", "pc")) +
                         r">\(float\*, [a-z ]+\*, float\*, float\*, void\*\)")


# ---- TSTORE of Mat tiles: the tstore launcher and cases again, through L1 (tstore_mat2gm_kernel.cpp:17-121); cases whose
# tile is larger than a compute unit's LDS end at their TASSIGN and are not run
def store_mat_runnable(spec, m):
    g = [int(m.group("g%d" % k)) for k in range(5)]
    size = {"long": 8, "float": 4, "short": 2, "signed char": 1, "unsigned short": 2}[m.group("T")]
    block = 32 // size
    up = lambda x: (x + block - 1) // block * block
    fmt = int(m.group("fmt"))
    if fmt == 0:
        numel = g[0] * g[1] * g[2] * g[3] * up(g[4])
    elif fmt == 1:
        numel = up(g[3]) * g[0] * g[1] * g[2] * g[4]
    else:
        numel = g[2] * g[3] * g[0] * g[1] * g[4]
    return numel * size <= 160 * 1024


SPECS["tstore_mat2gm"] = dict(SPECS["tstore"], lib="tstore_mat2gm", runnable=store_mat_runnable)


# ---- TSCATTER, the NPU form: launchTScatterTestCase<N>(out, src, indexes, stream); kernel N fixes <T, TI, rows, cols, idxRows,
# idxCols, ...>: out.flat[indexes[i, j]] = src[i, j] in row-major order of (i, j); what no index names is not defined
# (tscatter_kernel.cpp:17-57, tscatter/gen_data.py:11-22)
def plan_scatter_flat(test, spec, m):
    t = manifest()[spec["lib"]]["cases"][m.group("case")]["targs"]
    dt = np.dtype({"int16_t": np.int16, "half": np.float16, "int32_t": np.int32, "float": np.float32, "int8_t": np.int8}[t[0]])
    it = np.dtype({"uint16_t": np.uint16, "int16_t": np.int16, "uint32_t": np.uint32, "int32_t": np.int32}[t[1]])
    r0, c0, r1, c1 = (int(x) for x in t[2:6])

    def scatter(arrays):
        out = np.zeros(r0 * c0, dtype=dt)
        written = np.zeros(r0 * c0, dtype=bool)
        src, idx = arrays[0], arrays[1]
        for i in range(r1):
            for j in range(c1):
                out[int(idx[i, j])] = src[i, j]
                written[int(idx[i, j])] = True
        return out.reshape(r0, c0), written.reshape(r0, c0)

    pl = _plan(spec, [(dt, (r0, c0))], [(dt, (r0, c0), "any"), (it, (r1, c1), ("below", r0 * c0))], [(r0, c0)], lambda a: [scatter(a)[0]])
    pl.compare = lambda got, want, arrays: np.array_equal(got[scatter(arrays)[1]].view(np.uint8), want[scatter(arrays)[1]].view(np.uint8))
    return pl


SPECS["tscatter"] = dict(fn="launchTScatterTestCase", lib="tscatter", planner=plan_scatter_flat, inputs="any",
                         tail=r"<(?P<case>\d+)u>\(void\*, void\*, void\*, (?:ihipStream_t|void)\*\)")


# ---- TGATHERB: LaunchTGatherB<T, dstRows, dstCols, offRows, offCols, srcRows, srcCols>(out, src, offset, stream): every 32-byte
# block of out = the 32 bytes at byte offset[r, block] of src (tgatherb_kernel.cpp:17-60, tgatherb/gen_data.py:12-40)
def plan_gatherb(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    q = _ints(m, ["dr", "dc", "orr", "oc", "sr", "sc"])
    per = 32 // dt.itemsize
    src_bytes = q["sr"] * q["sc"] * dt.itemsize

    def expect(arrays):
        raw = arrays[0].reshape(-1).view(np.uint8)
        off = arrays[1].astype(np.int64)
        blocks = raw[(off[:, :, None] + np.arange(32)[None, None, :])]          # [rows, blocks, 32]
        return [blocks.reshape(q["dr"], -1).view(dt)[:, :q["dc"]]]
    pl = _plan(spec, [(dt, (q["dr"], q["dc"]))], [(dt, (q["sr"], q["sc"]), "bits" if dt.kind in "iu" else "any"),
                                                   (np.dtype(np.uint32), (q["orr"], q["oc"]), ("block_offsets", src_bytes))], [(q["dr"], q["dc"])], expect)
    assert q["oc"] * per == q["dc"] and q["orr"] == q["dr"]
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(np.uint8), want.view(np.uint8))
    return pl


SPECS["tgatherb"] = dict(fn="LaunchTGatherB", planner=plan_gatherb, inputs="any",
                         tail=r"<(?P<T>[A-Za-z_0-9 ]+)" + "".join(r", (?P<%s>\d+)ul?" % k for k in ("dr", "dc", "orr", "oc", "sr", "sc")) +
                         r">\([A-Za-z_0-9 ]+\*, [A-Za-z_0-9 ]+\*, unsigned int\*, void\*\)")


# ---- pairs of instructions from the a5 tree: Launch<A>_<B><T, tileRows, tileCols, validRows, validCols>(out, src0, src1[, src2],
# stream): all tiles [tileRows, tileCols], memory rows tileCols apart; every instruction rounds to T on its own
# (tests/npu/a5/src/st/testcase/tadd_tdiv/tadd_tdiv_kernel.cpp:20-55 and its seven siblings, and their gen_data.py)
def plan_pair(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    tr, tc, vr, vc = (int(m.group(k)) for k in ("tr", "tc", "vr", "vc"))
    rnd = (lambda x: x.astype(dt)) if dt.kind == "f" else (lambda x: x.astype(np.int64).astype(dt))
    wide = (lambda x: x.astype(np.float64)) if dt.kind == "f" else (lambda x: x.astype(np.int64))
    f = spec["formula"]

    def expect(arrays):
        return [f(*[wide(a[:, :vc]) for a in arrays], rnd=lambda x: wide(rnd(x)), vc=vc)]
    region = (vr, 1) if spec["col0"] else (vr, vc)
    return _plan(spec, [(dt, (vr, tc))], [(dt, (vr, tc))] * spec["nin"], [region], expect)


_PAIRS = {
    "tadd_tdiv": ("LaunchTADD_TDIV", 3, False, lambda a, b, c, rnd, vc: rnd(a + b) / c),
    "tmul_tadds": ("LaunchTMUL_TADDS", 3, False, lambda a, b, c, rnd, vc: rnd(a * b) + c[0, 0]),
    "tmuls_trowsum": ("LaunchTMULS_TROWSUM", 3, True, lambda a, b, c, rnd, vc: rnd(a * b[0, 0]).sum(axis=1, keepdims=True)),
    "trowsum_trowexpand": ("LaunchTROWSUM_TROWEXPAND", 2, False, lambda a, b, rnd, vc: np.repeat(rnd(a.sum(axis=1, keepdims=True)), vc, axis=1)),
    "trowexpand_tdiv": ("LaunchTROWEXPAND_TDIV", 2, False, lambda a, b, rnd, vc: a[:, :1] / b),
    "trowexpand_tsqrt": ("LaunchTROWEXPAND_TSQRT", 2, False, lambda a, b, rnd, vc: np.repeat(np.sqrt(a[:, :1]), vc, axis=1)),
    "trowexpand_trowsum": ("LaunchTROWEXPAND_TROWSUM", 2, True, lambda a, b, rnd, vc: a[:, :1] * vc),
    "tsub_texp": ("LaunchTSUB_TEXP", 2, False, lambda a, b, rnd, vc: np.exp(rnd(a - b))),
}
for _name, (_fn, _nin, _col0, _formula) in _PAIRS.items():
    SPECS["a5_" + _name] = dict(fn=_fn, lib="a5_" + _name, planner=plan_pair, inputs="pos", nin=_nin, col0=_col0, formula=_formula,
                                tail=TAIL(["tr", "tc", "vr", "vc"], _nin + 1), tol=REDUCE_TOL, atol=REDUCE_ATOL)


# ---- TCI: launchTCI_demo_b32_case<N><d>(out, stream) / ..._b16_...: out[0, j] = START +- j; the kernels fix columns and
# direction through macros (tci_common.h:11-26: START 0; b32 columns 128, 600, 32, 2000, b16 256, 800, 64, 5120;
# tci_kernel.cpp:36-67: b32 cases 3 and 4, b16 cases 2 and 4 count down); the launcher's template argument is not used
_TCI = {("b32", 1): (128, 0), ("b32", 2): (600, 0), ("b32", 3): (32, 1), ("b32", 4): (2000, 1),
        ("b16", 1): (256, 0), ("b16", 2): (800, 1), ("b16", 3): (64, 0), ("b16", 4): (5120, 1)}


def plan_ci(test, spec, m):
    cols, down = _TCI[(m.group("w"), int(m.group("case")))]
    dt = np.dtype(np.int32 if m.group("w") == "b32" else np.int16)
    return _plan(spec, [(dt, (1, cols))], [], [(1, cols)], lambda a: [((-1 if down else 1) * np.arange(cols)).astype(dt)[None, :]])


SPECS["tci"] = dict(fn="launchTCI_demo_", lib="tci", planner=plan_ci, inputs="any", tail=r"(?P<w>b32|b16)_case(?P<case>\d)<[01]u>\((?:int|short)\*, void\*\)")


# ---- TLOAD: launchTLOAD<N>(out, src, log, stream); kernel N fixes <T, s0, s1, s2, s3, s4, tileRows, tileCols, dyn, pad>: the
# [s0, s1, s2, s3, s4] tensor, in as many blocks as the launcher asks for, each loading its rows of every slab into one
# tile and storing it through a second tile object at the same address; out is [s0, s1, s2, s3, s4 rounded up to 32 bytes]
# with the pad value in the added columns (tload_kernel.cpp:97-150; golden :253-300)
def plan_load(test, spec, m):
    t = manifest()[spec["lib"]]["cases"]["%s:%s" % (spec["fn"], m.group("case"))]["targs"]
    dt = np.dtype({"float": np.float32, "int16_t": np.int16, "uint8_t": np.uint8, "int64_t": np.int64, "uint64_t": np.uint64}[t[0]])
    s = [int(x) for x in t[1:6]]
    per = 32 // dt.itemsize
    aligned = (s[4] + per - 1) // per * per
    which = t[9].split("::")[1]
    pad = _pad_value(dt, which) if which in ("Max", "Min") else dt.type(0)
    rows = s[0] * s[1] * s[2] * s[3]

    def expect(arrays):
        out = np.full((rows, aligned), pad, dtype=dt)
        out[:, :s[4]] = arrays[0]
        return [out]
    pl = _plan(spec, [(dt, (rows, aligned))], [(dt, (rows, s[4]), "bits" if dt.kind in "iu" else "any"), (np.dtype(np.uint64), (1, 128 * 32), "any")],
               [(rows, aligned)], expect)
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(np.uint8), want.view(np.uint8))
    return pl


SPECS["tload"] = dict(fn="launchTLOAD", lib="tload", tail=r"<(?P<case>\d+)>\(unsigned char\*, unsigned char\*, unsigned long\*, void\*\)", planner=plan_load, inputs="any")


# ---- MGATHER / MSCATTER (a5 tree): LaunchMGATHER<T, TIdx, tableRows, tableCols, outRows, outCols>(out, table, indices, stream),
# out[i, j] = table.flat[indices[i, j]]; LaunchMSCATTER<T, TIdx, srcRows, srcCols, outSize>(out, src, indices, stream),
# out[indices[i, j]] = src[i, j], the rest of out untouched; the Half launchers take fp16 as uint16
# (tests/npu/a5/src/st/testcase/mgather/mgather_kernel.cpp:17-46, mscatter/mscatter_kernel.cpp:19-60 and their gen_data.py)
def plan_mgather(test, spec, m):
    dt = np.dtype(np.float16) if spec["half"] else _elem(m.group("T"), False)[0]
    tr, tc, orr, oc = (int(m.group(k)) for k in ("tr", "tc", "orr", "oc"))
    pl = _plan(spec, [(dt, (orr, oc))], [(dt, (tr, tc), "bits" if dt.kind in "iu" else "any"), (np.dtype(np.int32), (orr, oc), ("below", tr * tc))],
               [(orr, oc)], lambda a: [a[0].reshape(-1)[a[1]]])
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8))
    return pl


def plan_mscatter(test, spec, m):
    dt = np.dtype(np.float16) if spec["half"] else _elem(m.group("T"), False)[0]
    sr, sc, n = (int(m.group(k)) for k in ("sr", "sc", "n"))

    def expect(a):
        out = np.full(n, 77, dtype=dt)
        out[a[1].reshape(-1)] = a[0].reshape(-1)
        return [out[None, :]]
    pl = _plan(spec, [(dt, (1, n))], [(dt, (sr, sc), "bits" if dt.kind in "iu" else "any"), (np.dtype(np.int32), (sr, sc), ("distinct", n))], [(1, n)], expect)
    pl.compare = lambda got, want, arrays: np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8))
    return pl


_G4 = "".join(r", (?P<%s>\d+)" % k for k in ("tr", "tc", "orr", "oc"))
_S3 = "".join(r", (?P<%s>\d+)" % k for k in ("sr", "sc", "n"))
SPECS["a5_mgather"] = dict(fn="LaunchMGATHER", lib="a5_mgather", planner=plan_mgather, inputs="any", half=False,
                           tail=r"<(?P<T>[a-z ]+), int" + _G4 + r">\((?:[a-z ]+\*, ){2}int\*, void\*\)")
SPECS["a5_mgather:half"] = dict(fn="LaunchMGATHERHalf", lib="a5_mgather", planner=plan_mgather, inputs="any", half=True,
                                tail=r"<" + _G4[2:] + r">\((?:unsigned short\*, ){2}int\*, void\*\)")
SPECS["a5_mscatter"] = dict(fn="LaunchMSCATTER", lib="a5_mscatter", planner=plan_mscatter, inputs="any", half=False,
                            tail=r"<(?P<T>[a-z ]+), int" + _S3 + r">\((?:[a-z ]+\*, ){2}int\*, void\*\)")
SPECS["a5_mscatter:half"] = dict(fn="LaunchMSCATTERHalf", lib="a5_mscatter", planner=plan_mscatter, inputs="any", half=True,
                                 tail=r"<" + _S3[2:] + r">\((?:unsigned short\*, ){2}int\*, void\*\)")


# ---- TPACK (a5 tree): TPackTest::LaunchTPack<rows, cols, Src, Dst>(dst, src, stream): the low bytes of every element
# (tests/npu/a5/src/st/testcase/tpack/tpack_kernel.cpp:20-50, tpack/gen_data.py:10-38)
def plan_pack(test, spec, m):
    rows, cols = int(m.group("r")), int(m.group("c"))
    sdt, ddt = _elem(m.group("S"), False)[0], _elem(m.group("D"), False)[0]
    return _plan(spec, [(ddt, (rows, cols))], [(sdt, (rows, cols), "bits")], [(rows, cols)],
                 lambda a: [(a[0].astype(np.uint64) & np.uint64((1 << (8 * ddt.itemsize)) - 1)).astype(ddt)])


SPECS["a5_tpack"] = dict(fn="TPackTest::LaunchTPack", lib="a5_tpack", planner=plan_pack, inputs="bits",
                         tail=r"<(?P<r>\d+), (?P<c>\d+), (?P<S>[a-z ]+), (?P<D>[a-z ]+)>\([a-z ]+\*, [a-z ]+\*, void\*\)")


# ---- TROWEXPAND from a column tile (a5 tree): TRowExpandTest::launchTROWEXPAND<T, rows, cols>(out, src, stream):
# out[r, c] = src[r] (tests/npu/a5/src/st/testcase/trowexpandbrcb/trowexpandbrcb_kernel.cpp:16-45)
def plan_rowexpand_col(test, spec, m):
    dt, _ = _elem(m.group("T"), True)
    rows, cols = int(m.group("r")), int(m.group("c"))
    return _plan(spec, [(dt, (rows, cols))], [(dt, (rows, 1), "any")], [(rows, cols)], lambda a: [np.repeat(a[0], cols, axis=1)])


SPECS["a5_trowexpandbrcb"] = dict(fn="TRowExpandTest::launchTROWEXPAND", lib="a5_trowexpandbrcb", planner=plan_rowexpand_col, inputs="any",
                                  tail=r"<(?P<T>[a-z ]+), (?P<r>\d+)u, (?P<c>\d+)u>\([a-z ]+\*, [a-z ]+\*, void\*\)", tol=EXACT)


# ---- sources of the a5 tree whose launchers have the form of their a2a3 namesakes: the same planners
for _name in ("tpartmul", "tfmods", "tmov_vect"):
    SPECS["a5_" + _name] = dict(SPECS[_name], lib="a5_" + _name)


def lib_of(test):
    """name of the library (build/ported/st/<name>.so, and of the manifest entry) that holds a test's launchers"""
    return SPECS[test].get("lib", test)


def draw(rng, dt, shape, kind, j):
    """Operand j of a test whose operation is of the given kind."""
    if isinstance(kind, tuple) and kind[0] == "distinct":    # distinct indices below kind[1]
        return rng.permutation(kind[1])[:int(np.prod(shape))].reshape(shape).astype(dt)
    if isinstance(kind, tuple) and kind[0] == "below":       # indices below kind[1]
        return rng.integers(0, kind[1], size=shape).astype(dt)
    if isinstance(kind, tuple) and kind[0] == "block_offsets":      # byte offsets of whole 32-byte blocks inside kind[1] bytes
        return (rng.integers(0, kind[1] // 32, size=shape) * 32).astype(dt)
    if isinstance(kind, tuple) and kind[0] == "range":
        return rng.uniform(kind[1], kind[2], size=shape).astype(dt)
    if isinstance(kind, tuple) and kind[0] == "corner":      # small integers in the [vr, vc] corner, zeros around it
        x = np.zeros(shape, dtype=dt)
        v = rng.integers(-1, 2, size=(kind[1], kind[2]), endpoint=True)
        x[:kind[1], :kind[2]] = _bf16_bits(v.astype(np.float64)) if len(kind) > 3 and kind[3] == "bf16" else v.astype(dt)
        return x
    if isinstance(kind, tuple) and kind[0] == "words":       # quantisation words for results of type kind[1]
        n = int(np.prod(shape))
        if kind[1] == "int16_t":
            return (rng.integers(0, 7, size=n, endpoint=True).astype(np.uint64) << np.uint64(32)).reshape(shape)
        w = rng.choice(np.array([0.5, 1.0, 1.5, 2.0], dtype=np.float32), size=n).view(np.uint32).astype(np.uint64)
        if kind[1] in ("int8_t", "uint8_t"):
            w |= rng.integers(0, 3, size=n, endpoint=True).astype(np.uint64) << np.uint64(37)
            w |= np.uint64(int(kind[1] == "int8_t")) << np.uint64(46)
        return w.reshape(shape)
    if isinstance(kind, tuple):
        return _sorted_inputs(rng, dt, shape, kind)
    bits = dt.itemsize * 8
    if kind.startswith("cvt"):                # inside the range of every destination type of the conversion tests
        lo, hi = (0, 100) if kind == "cvt_u" else (-100, 100)
        if dt.kind == "f":
            return rng.uniform(lo, hi, size=shape).astype(dt)
        if kind == "cvt":
            lo, hi = -10000, 10000
        return rng.integers(lo, hi, size=shape, endpoint=True).astype(dt)
    if kind == "unit":
        return rng.uniform(-1.0, 1.0, size=shape).astype(dt)
    if kind == "near1":
        return rng.uniform(0.9, 1.1, size=shape).astype(dt)
    if kind == "scores":                      # few distinct values: many equal scores, whose order the index decides
        return (rng.integers(-20, 20, size=shape) * 0.5).astype(dt)
    if kind == "index":
        return rng.permutation(int(np.prod(shape))).reshape(shape).astype(dt)
    if kind == "bf16":
        return _bf16_bits(rng.uniform(-1.0, 1.0, size=shape))
    if kind == "small":                       # few distinct values: equal pairs occur, products stay small
        return rng.integers(-3 if dt.kind != "u" else 0, 3, size=shape, endpoint=True).astype(dt)
    if dt.kind == "f":
        if kind == "pos":
            x = rng.uniform(0.5, 4.0, size=shape)
        elif kind in ("rem", "rempos") and j == 1:
            x = rng.integers(3, 100, size=shape).astype(np.float64)
        elif kind in ("rem", "rempos"):
            x = rng.integers(0 if kind == "rempos" else -1000, 1000, size=shape).astype(np.float64)
        else:
            x = rng.uniform(-4.0, 4.0, size=shape)
        return x.astype(dt)
    info = np.iinfo(dt)
    if kind == "shift" and j == 1:
        x = rng.integers(0, bits - 1, size=shape)
    elif kind == "shift":
        x = rng.integers(0, min(info.max, 1 << (bits - 2)) >> 3, size=shape)      # room to shift without sign trouble
    elif kind in ("rem", "rempos") and j == 1:
        x = rng.integers(3, 100, size=shape)
    elif kind in ("rem", "rempos"):
        x = rng.integers(0 if kind == "rempos" else max(info.min, -1000), min(info.max, 1000), size=shape)
    elif kind == "bits":
        if dt.itemsize == 8:
            return rng.integers(0, 2**63 - 1, size=shape, dtype=np.int64).view(dt) ^ dt.type(0x5A5A)
        x = rng.integers(info.min, info.max, size=shape, endpoint=True)
    elif kind == "pos":
        x = rng.integers(1, 100, size=shape)
    else:
        x = rng.integers(max(info.min, -100), min(info.max, 100), size=shape)
    return x.astype(dt)


def make_inputs(pl, seed):
    """Input buffers (whole, with their leading dimensions), drawn for the test's kind of operation."""
    rng = np.random.default_rng(seed)
    return [draw(rng, dt, shape, pl.spec["inputs"] if len(entry) == 2 else entry[2], j)
            for j, entry in enumerate(pl.ins) for dt, shape in [entry[:2]]]


def expected(pl, ins):
    """Per output, the valid region, in float64 for floating-point tiles (the caller rounds / compares)."""
    return pl.expect(ins, pl.scalar[1] if pl.scalar else None)
