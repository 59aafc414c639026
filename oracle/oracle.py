"""ctypes view of the CPU oracle (``libscn_oracle.so``).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this
module; the product never does.  Each function forwards to the C restatement
in ``scn_oracle.c`` whose header cites the reference code it follows.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libscn_oracle.so")

# reference ActivationFunction numbering (types.h:11-20)
NOSIGMOID, RELU, VLEAKYRELU, LEAKYRELU, TANH, SOFTMAX, PRELU, SIGMOID = range(8)


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s", "-B"])


def _load():
    # SCN_ORACLE_LIB: another build of the same source (bench.py's cpu_baseline
    # times the -march=native one; checkers never set it)
    path = os.environ.get("SCN_ORACLE_LIB") or _LIB_PATH
    if path == _LIB_PATH and not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(path)
    vp, i32, i64, f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float
    sig = {
        "orc_grids_create": (vp, [C.c_int]),
        "orc_grids_destroy": (None, [vp]),
        "orc_grids_set": (None, [vp, C.c_int, i64, vp, vp, i32]),
        "orc_grids_size": (i64, [vp, C.c_int]),
        "orc_grids_background": (i32, [vp, C.c_int]),
        "orc_grids_get": (None, [vp, C.c_int, vp, vp]),
        "orc_ivec_create": (vp, []),
        "orc_ivec_destroy": (None, [vp]),
        "orc_ivec_size": (i64, [vp]),
        "orc_ivec_data": (vp, [vp]),
        "orc_sq_inputL": (C.c_int, [C.c_int] * 3),
        "orc_sq_inputR": (C.c_int, [C.c_int] * 3),
        "orc_sq_outputL": (C.c_int, [C.c_int] * 3),
        "orc_sq_outputR": (C.c_int, [C.c_int] * 4),
        "orc_ipow": (C.c_int, [C.c_int] * 2),
        "orc_triangle_size": (C.c_int, [C.c_int] * 2),
        "orc_tri_ord": (C.c_int, [C.c_int, C.c_int, vp]),
        "orc_rules_square": (i64, [vp, vp] + [C.c_int] * 6 + [vp]),
        "orc_rules_triangular": (i64, [vp, vp] + [C.c_int] * 6 + [vp]),
        "orc_rules_terminal": (i64, [vp, vp, vp]),
        "orc_gather_rows": (None, [vp, vp, vp, i64, C.c_int]),
        "orc_nin_forward": (None, [vp] * 5 + [i64, C.c_int, C.c_int, f32, C.c_int]),
        "orc_nin_forward_f64": (None, [vp] * 5 + [i64, C.c_int, C.c_int, f32, C.c_int]),
        "orc_softmax_rows": (None, [vp, vp, i64, C.c_int]),
        "orc_maxpool": (None, [vp, vp, vp, i64, C.c_int, C.c_int, vp]),
        "orc_terminal_pool": (None, [vp, vp, vp, i64, C.c_int, C.c_int]),
        "orc_top_indices": (None, [vp, C.c_int, C.c_int, vp]),
        "orc_softmax_classifier": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, vp, vp]),
        "orc_fmp_ticks_po": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_double, vp, vp]),
        "orc_fmp_ticks_pd": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_double, vp, vp]),
        "orc_fmp_increments": (C.c_int, [C.c_int, C.c_int, C.c_int, vp]),
        "orc_fmp_ticks_ro": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp]),
        "orc_fmp_ticks_rd": (C.c_int, [C.c_int, C.c_int, vp, vp, vp]),
        "orc_rules_fmp": (i64, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, vp, C.c_int, vp]),
        "orc_softmax_grad": (None, [vp, vp, vp, i64, C.c_int]),
        "orc_activation_backward": (None, [vp, vp, i64, C.c_int, C.c_int, vp, vp, vp]),
        "orc_sgemm_AtB": (None, [vp, vp, vp, i64, C.c_int, C.c_int]),
        "orc_sgemm_ABt": (None, [vp, vp, vp, i64, C.c_int, C.c_int]),
        "orc_nag_update": (None, [vp, vp, vp, i64, f32, f32, C.c_int]),
        "orc_gather_rows_backward": (None, [vp, vp, vp, i64, C.c_int]),
        "orc_maxpool_backward": (None, [vp, vp, i64, C.c_int, vp]),
        "orc_terminal_pool_backward": (None, [vp, vp, vp, i64, C.c_int, C.c_int]),
        "orc_set_threads": (None, [C.c_int]),
        "orc_get_threads": (C.c_int, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def set_threads(n):
    lib.orc_set_threads(int(n))


class Grids:
    """A batch of per-sample SparseGrids (key -> row, backgroundCol)."""

    def __init__(self, batch):
        self.batch = int(batch)
        self.h = lib.orc_grids_create(self.batch)

    def __del__(self):
        if getattr(self, "h", None):
            lib.orc_grids_destroy(self.h)
            self.h = None

    def set(self, item, keys, rows, background):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        rows = _i32(rows)
        assert keys.shape == rows.shape
        lib.orc_grids_set(self.h, item, keys.size, _p(keys), _p(rows), int(background))

    def size(self, item):
        return lib.orc_grids_size(self.h, item)

    def background(self, item):
        return lib.orc_grids_background(self.h, item)

    def get(self, item):
        n = self.size(item)
        keys = np.empty(n, np.int64)
        rows = np.empty(n, np.int32)
        lib.orc_grids_get(self.h, item, _p(keys), _p(rows))
        return keys, rows

    def flat(self):
        """(sample, key, row) of every entry in iteration order, and bg[batch]."""
        s, k, r = [], [], []
        for i in range(self.batch):
            kk, rr = self.get(i)
            s.append(np.full(kk.size, i, np.int32))
            k.append(kk)
            r.append(rr)
        bg = np.array([self.background(i) for i in range(self.batch)], np.int32)
        cat = lambda xs, dt: np.concatenate(xs).astype(dt) if xs else np.zeros(0, dt)
        return cat(s, np.int32), cat(k, np.int64), cat(r, np.int32), bg

    @staticmethod
    def from_flat(batch, sample, key, row, bg):
        g = Grids(batch)
        sample = np.asarray(sample)
        for i in range(batch):
            m = sample == i
            g.set(i, np.asarray(key)[m], np.asarray(row)[m], int(bg[i]))
        return g


def _ivec_take(v):
    n = lib.orc_ivec_size(v)
    out = np.empty(n, np.int32)
    if n:
        C.memmove(_p(out), lib.orc_ivec_data(v), n * 4)
    lib.orc_ivec_destroy(v)
    return out


def rules_square(grids, dimension, nIn, nOut, size, stride, minActive=1):
    out = Grids(grids.batch)
    v = lib.orc_ivec_create()
    n = lib.orc_rules_square(grids.h, out.h, dimension, nIn, nOut, size, stride, minActive, v)
    rules = _ivec_take(v)
    if n < 0:
        raise ValueError("orc_rules_square: bad arguments")
    return out, rules, int(n)


def rules_triangular(grids, dimension, nIn, nOut, size, stride, minActive=1):
    out = Grids(grids.batch)
    v = lib.orc_ivec_create()
    n = lib.orc_rules_triangular(grids.h, out.h, dimension, nIn, nOut, size, stride, minActive, v)
    rules = _ivec_take(v)
    if n < 0:
        raise ValueError("orc_rules_triangular: bad arguments")
    return out, rules, int(n)


def fmp_ticks(kind, nIn, nOut, poolSize, draw):
    """(inputL, inputR) of one axis.  kind: "po" / "pd" (pseudorandom overlapping / disjoint; draw = u in [0, 1))
    or "ro" / "rd" (random; draw = the shuffled increments, see fmp_increments).  None when the reference asserts."""
    L, R = np.empty(nOut, np.int32), np.empty(nOut, np.int32)
    if kind == "po":
        rc = lib.orc_fmp_ticks_po(nIn, nOut, poolSize, float(draw), _p(L), _p(R))
    elif kind == "pd":
        rc = lib.orc_fmp_ticks_pd(nIn, nOut, poolSize, float(draw), _p(L), _p(R))
    elif kind == "ro":
        rc = lib.orc_fmp_ticks_ro(nIn, nOut, poolSize, _p(_i32(draw)), _p(L), _p(R))
    else:
        rc = lib.orc_fmp_ticks_rd(nIn, nOut, _p(_i32(draw)), _p(L), _p(R))
    return (L, R) if rc == 0 else None


def fmp_increments(nIn, nOut, overlapping):
    inc = np.empty(nOut, np.int32)
    n = lib.orc_fmp_increments(nIn, nOut, int(overlapping), _p(inc))
    return inc[:n].copy()


def rules_fmp(grids, dimension, nIn, nOut, poolSize, inputL, inputR, uniform):
    """inputL / inputR: [batch, dimension, nOut] int32"""
    inputL, inputR = _i32(inputL), _i32(inputR)
    assert inputL.shape == (grids.batch, dimension, nOut) == inputR.shape
    out = Grids(grids.batch)
    v = lib.orc_ivec_create()
    n = lib.orc_rules_fmp(grids.h, out.h, dimension, nIn, nOut, poolSize, _p(inputL), _p(inputR), int(uniform), v)
    rules = _ivec_take(v)
    if n < 0:
        raise ValueError("orc_rules_fmp: bad arguments")
    return out, rules, int(n)


def rules_terminal(grids):
    out = Grids(grids.batch)
    v = lib.orc_ivec_create()
    S = lib.orc_rules_terminal(grids.h, out.h, v)
    return out, _ivec_take(v), int(S)


def tri_ord(s, d):
    ord_ = np.empty(s ** d, np.int32)
    S = lib.orc_tri_ord(s, d, _p(ord_))
    return ord_, S


def gather_rows(inp, rules, nIn):
    inp, rules = _f32(inp), _i32(rules)
    out = np.empty((rules.size, nIn), np.float32)
    lib.orc_gather_rows(_p(inp), _p(out), _p(rules), rules.size, nIn)
    return out


def nin_forward(A, W, B, prelu, p, act, f64=False):
    A, W, B = _f32(A), _f32(W), _f32(B)
    M, K = A.shape
    N = W.shape[1]
    assert W.shape[0] == K and B.size == N
    pr = _f32(prelu) if prelu is not None else None
    out = np.empty((M, N), np.float64 if f64 else np.float32)
    fn = lib.orc_nin_forward_f64 if f64 else lib.orc_nin_forward
    fn(_p(A), _p(W), _p(B), _p(pr) if pr is not None else None, _p(out), M, K, N, float(p), int(act))
    return out


def softmax_rows(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib.orc_softmax_rows(_p(x), _p(out), x.shape[0], x.shape[1])
    return out


def maxpool(inp, rules, nOutSites, ps, Cn):
    inp, rules = _f32(inp), _i32(rules)
    out = np.empty((nOutSites, Cn), np.float32)
    choice = np.empty((nOutSites, Cn), np.int32)
    lib.orc_maxpool(_p(inp), _p(out), _p(rules), nOutSites, ps, Cn, _p(choice))
    return out, choice


def terminal_pool(inp, rules, count, S, Cn):
    inp, rules = _f32(inp), _i32(rules)
    out = np.empty((count, Cn), np.float32)
    with np.errstate(all="ignore"):
        lib.orc_terminal_pool(_p(inp), _p(out), _p(rules), count, S, Cn)
    return out


def top_indices(v, k):
    v = _f32(v)
    idx = np.empty(k, np.int32)
    lib.orc_top_indices(_p(v), v.size, k, _p(idx))
    return idx


def softmax_classifier(probs, labels, nTop):
    probs, labels = _f32(probs), _i32(labels)
    batch, nClasses = probs.shape
    pred = np.empty((batch, nTop), np.int32)
    nll = C.c_float(0.0)
    mistakes = lib.orc_softmax_classifier(_p(probs), _p(labels), batch, nClasses, nTop, _p(pred), C.byref(nll))
    return pred, int(mistakes), float(nll.value)


# ---- backward pass -------------------------------------------------------
def softmax_grad(probs, labels):
    probs, labels = _f32(probs), _i32(labels)
    out = np.empty_like(probs)
    lib.orc_softmax_grad(_p(probs), _p(labels), _p(out), probs.shape[0], probs.shape[1])
    return out


def activation_backward(out, delta, act, prelu=None):
    """(delta multiplied by the activation's derivative, bias gradient, PReLU slope gradient or None)"""
    out, delta = _f32(out), np.array(delta, np.float32, order="C")
    M, N = out.shape
    db = np.empty(N, np.float32)
    pr = _f32(prelu) if prelu is not None else None
    dpr = np.empty(N, np.float32) if prelu is not None else None
    lib.orc_activation_backward(_p(out), _p(delta), M, N, int(act), _p(pr) if pr is not None else None, _p(db),
                                _p(dpr) if dpr is not None else None)
    return delta, db, dpr


def sgemm_AtB(A, D):
    A, D = _f32(A), _f32(D)
    out = np.empty((A.shape[1], D.shape[1]), np.float32)
    lib.orc_sgemm_AtB(_p(A), _p(D), _p(out), A.shape[0], A.shape[1], D.shape[1])
    return out


def sgemm_ABt(D, W):
    D, W = _f32(D), _f32(W)
    out = np.empty((D.shape[0], W.shape[0]), np.float32)
    lib.orc_sgemm_ABt(_p(D), _p(W), _p(out), D.shape[0], D.shape[1], W.shape[0])
    return out


def nag_update(delta, mom, wts, learningRate, momentum, keepPositive=False):
    """updates mom and wts (float32 arrays) in place"""
    delta = _f32(delta)
    assert mom.dtype == np.float32 and wts.dtype == np.float32 and mom.flags.c_contiguous and wts.flags.c_contiguous
    lib.orc_nag_update(_p(delta), _p(mom), _p(wts), wts.size, float(learningRate), float(momentum), int(keepPositive))


def gather_rows_backward(dconv, rules, nRowsIn, nIn):
    dconv, rules = _f32(dconv), _i32(rules)
    din = np.zeros((nRowsIn, nIn), np.float32)
    lib.orc_gather_rows_backward(_p(din), _p(dconv), _p(rules), rules.size, nIn)
    return din


def maxpool_backward(dout, choice, nRowsIn):
    dout, choice = _f32(dout), _i32(choice)
    count, Cn = dout.shape
    din = np.zeros((nRowsIn, Cn), np.float32)
    lib.orc_maxpool_backward(_p(din), _p(dout), count, Cn, _p(choice))
    return din


def terminal_pool_backward(dout, rules, S, nRowsIn):
    dout, rules = _f32(dout), _i32(rules)
    count, Cn = dout.shape
    din = np.zeros((nRowsIn, Cn), np.float32)
    lib.orc_terminal_pool_backward(_p(din), _p(dout), _p(rules), count, Cn, S)
    return din
