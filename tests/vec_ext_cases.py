"""Seeded inputs shared by the oracle tests, the golden generator and the GPU tests of the further Vec instructions."""
import numpy as np

UNARY = ["ABS", "NEG", "RELU", "SQRT", "RSQRT", "LOG", "RECIP", "EXP"]
BINARY = ["ADD", "SUB", "MUL", "DIV", "MAX", "MIN", "PRELU", "CMP_EQ", "CMP_NE", "CMP_LT", "CMP_LE", "CMP_GT", "CMP_GE", "SELS"]
SCALAR = ["ADDS", "SUBS", "MULS", "DIVS", "MAXS", "MINS", "LRELU"]
ROWOPS = ["ROWEXPAND", "ROWEXPANDSUB", "ROWEXPANDMUL", "ROWEXPANDDIV", "ROWEXPANDADD", "ROWEXPANDMAX", "ROWEXPANDMIN", "ROWEXPANDEXPDIF"]
COLOPS = ["COLEXPAND", "COLEXPANDSUB", "COLEXPANDMUL", "COLEXPANDDIV", "COLEXPANDADD", "COLEXPANDMAX", "COLEXPANDMIN", "COLEXPANDEXPDIF"]
ALL_OPS = UNARY + BINARY + SCALAR + ROWOPS + COLOPS
POSITIVE = {"SQRT", "RSQRT", "LOG"}          # defined for positive inputs only
NONZERO_B = {"DIV", "DIVS", "ROWEXPANDDIV", "COLEXPANDDIV", "RECIP"}


def vec_inputs(op, seed=0):
    """a, b [64,128], vec [64] or [128] (or None), scalar for one op."""
    rng = np.random.default_rng(1000 + seed + sum(map(ord, op)))
    a = (rng.standard_normal((64, 128)) * 3).astype(np.float32)
    b = (rng.standard_normal((64, 128)) * 3).astype(np.float32)
    if op in POSITIVE:
        a = (np.abs(a) + np.float32(0.01)).astype(np.float32)
    if op == "RECIP":
        a = np.where(np.abs(a) < 0.05, np.float32(0.5), a).astype(np.float32)
    if op in ("EXP", "ROWEXPANDEXPDIF", "COLEXPANDEXPDIF"):
        a = (a * np.float32(2.0)).astype(np.float32)
    if op.startswith("CMP"):        # plenty of equal pairs
        eq = rng.random((64, 128)) < 0.3
        b = np.where(eq, a, b).astype(np.float32)
    if op in NONZERO_B:
        b = np.where(np.abs(b) < 0.05, np.float32(0.7), b).astype(np.float32)
    vec = None
    if op in ROWOPS:
        vec = (rng.standard_normal(64) * 2).astype(np.float32)
    if op in COLOPS:
        vec = (rng.standard_normal(128) * 2).astype(np.float32)
    if vec is not None and op in NONZERO_B:
        vec = np.where(np.abs(vec) < 0.05, np.float32(0.7), vec).astype(np.float32)
    scalar = np.float32(1.0) if op == "SELS" else np.float32(-1.375)
    return a, b, vec, scalar


def numpy_vec_op(op, a, b, vec, k):
    """Closed forms (fp32 arithmetic; sqrt / log / exp evaluated in double and cast, as the CPU simulation does)."""
    f32, f64 = np.float32, np.float64
    with np.errstate(all="ignore"):
        r = vec[:, None] if vec is not None and vec.size == 64 else None
        c = vec[None, :] if vec is not None and vec.size == 128 else None
        table = {
            "ABS": lambda: np.abs(a), "NEG": lambda: -a, "RELU": lambda: np.maximum(a, f32(0)),
            "SQRT": lambda: np.sqrt(a.astype(f64)), "RSQRT": lambda: 1.0 / np.sqrt(a.astype(f64)),
            "LOG": lambda: np.log(a.astype(f64)), "RECIP": lambda: f32(1) / a, "EXP": lambda: np.exp(a.astype(f64)),
            "ADD": lambda: a + b, "SUB": lambda: a - b, "MUL": lambda: a * b, "DIV": lambda: a / b,
            "MAX": lambda: np.maximum(a, b), "MIN": lambda: np.minimum(a, b), "PRELU": lambda: np.where(a > 0, a, a * b),
            "CMP_EQ": lambda: a == b, "CMP_NE": lambda: a != b, "CMP_LT": lambda: a < b, "CMP_LE": lambda: a <= b,
            "CMP_GT": lambda: a > b, "CMP_GE": lambda: a >= b, "SELS": lambda: a if k == 1 else b,
            "ADDS": lambda: a + k, "SUBS": lambda: a - k, "MULS": lambda: a * k, "DIVS": lambda: a / k,
            "MAXS": lambda: np.maximum(a, k), "MINS": lambda: np.minimum(a, k), "LRELU": lambda: np.where(a > 0, a, a * k),
            "ROWEXPAND": lambda: np.broadcast_to(r, a.shape), "ROWEXPANDSUB": lambda: a - r, "ROWEXPANDMUL": lambda: a * r,
            "ROWEXPANDDIV": lambda: a / r, "ROWEXPANDADD": lambda: a + r, "ROWEXPANDMAX": lambda: np.maximum(a, r),
            "ROWEXPANDMIN": lambda: np.minimum(a, r), "ROWEXPANDEXPDIF": lambda: np.exp((a - r).astype(f64)),
            "COLEXPAND": lambda: np.broadcast_to(c, a.shape), "COLEXPANDSUB": lambda: a - c, "COLEXPANDMUL": lambda: a * c,
            "COLEXPANDDIV": lambda: a / c, "COLEXPANDADD": lambda: a + c, "COLEXPANDMAX": lambda: np.maximum(a, c),
            "COLEXPANDMIN": lambda: np.minimum(a, c), "COLEXPANDEXPDIF": lambda: np.exp((a - c).astype(f64)),
        }
        return np.asarray(table[op]()).astype(f32)


def reduce_inputs(seed=0):
    rng = np.random.default_rng(77 + seed)
    return (rng.standard_normal((64, 128)) * 5).astype(np.float32)


REDUCE_SHAPES = [(64, 128), (37, 128), (64, 88), (5, 24), (1, 128), (64, 8)]
