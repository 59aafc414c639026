"""csrc/scn_pyr_dev.h on the CPU: the per-lane bodies of the kernels that build a whole net's rule books from the
output side (k_pyr_masks / k_pyr_rules), compiled for the host and run lane after lane by tests/chain_cpu_harness.cpp,
against the oracle's gridRules (Regions.cu:528-653) layer by layer and its terminal rules
(TerminalPoolingLayer.cu:8-20).  Every buffer the harness writes is allocated with guard words that must come back
untouched."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "chain_cpu_harness.cpp")
LIB = os.path.join(HERE, "libchain_cpu.so")
GUARD = 64
REGIONS, TERMINAL = 0, 1


def build(force=False):
    hdr = os.path.join(ROOT, "sparseconvnet-archived_amd", "csrc", "scn_pyr_dev.h")
    stale = not os.path.exists(LIB) or os.path.getmtime(LIB) < max(os.path.getmtime(SRC), os.path.getmtime(hdr))
    if force or stale:
        subprocess.check_call(["g++", "-O1", "-g", "-std=c++17", "-shared", "-fPIC", "-Wall", "-fsanitize=undefined",
                               "-fno-sanitize-recover=undefined", "-static-libubsan",
                               "-I", os.path.dirname(hdr), SRC, "-o", LIB])


@pytest.fixture(scope="module")
def harness():
    build()
    lib = C.CDLL(LIB)
    lib.pyr_cpu_chain.restype = C.c_int
    return lib


def guarded(n, dtype, fill):
    a = np.full(n + 2 * GUARD, fill, dtype)
    a[:GUARD] = 0x5A5A5A5A
    a[n + GUARD:] = 0x5A5A5A5A
    return a


def intact(a, n):
    return np.all(a[:GUARD] == 0x5A5A5A5A) and np.all(a[n + GUARD:] == 0x5A5A5A5A)


def random_batch(rng, d, n, batch, fill):
    """source grids: (sample, key, row in insertion order, background row per sample, number of rows)"""
    S, K, R, bg = [], [], [], []
    row = 0
    vol = n ** d
    for b in range(batch):
        mode = rng.integers(0, 6)
        if mode == 0:
            keys = np.zeros(0, np.int64)  # an empty sample
        elif mode == 1 and vol <= 4096:
            keys = np.arange(vol, dtype=np.int64)  # a full one (a small field: it has to fit the LDS)
        else:
            keys = np.flatnonzero(rng.random(vol) < fill * rng.uniform(0.2, 2.0)).astype(np.int64)
        full = len(keys) == vol
        if not full and rng.random() < 0.8:
            bg.append(row)
            row += 1
        else:
            bg.append(-1 if full else row)
            row += 0 if full else 1
        rng.shuffle(keys)  # rows in insertion order, not key order
        S.append(np.full(len(keys), b, np.int32))
        K.append(keys)
        R.append(np.arange(row, row + len(keys), dtype=np.int32))
        row += len(keys)
    return (np.concatenate(S), np.concatenate(K), np.concatenate(R), np.array(bg, np.int32), row)


def run_chain(lib, d, n0, layers, batch, seed, fill=0.08, lds=152 * 1024, T=64, tight_bounds=False):
    """layers: list of ("c", size, stride) / ("t",) from the input side; the field sizes follow from n0."""
    rng = np.random.default_rng(seed)
    S, K, R, bg, nRows = random_batch(rng, d, n0, batch, fill)
    grids = orc.Grids.from_flat(batch, S, K, R, bg)
    geo, want = [], []
    n, cur = n0, grids
    for lay in layers:
        if lay[0] == "t":
            og, rules, width = orc.rules_terminal(cur)
            geo.append((TERMINAL, n, 1, 1, 1))
            want.append(dict(kind="t", grids=og, rules=rules, nSites=batch, width=width))
            cur, n = og, 1
        else:
            _, size, stride = lay
            assert (n - size) % stride == 0
            nOut = (n - size) // stride + 1
            og, rules, nSites = orc.rules_square(cur, d, n, nOut, size, stride, 1)
            geo.append((REGIONS, n, nOut, size, stride))
            want.append(dict(kind="c", grids=og, rules=rules, nSites=nSites, width=size ** d, volOut=nOut ** d))
            cur, n = og, nOut
    nL = len(layers)
    geo = np.array(geo, np.int32)
    rules, ekey, erow, bgo, caps, bounds = [], [], [], [], [], []
    for w in want:
        cap = max(w["rules"].size, 1)
        nAct = w["grids"].flat()[0].size
        rules.append(guarded(cap, np.int32, -99))
        ekey.append(guarded(nAct + 1, np.int64, -99))
        erow.append(guarded(nAct + 1, np.int32, -99))
        bgo.append(guarded(batch, np.int32, -99))
        caps.append(cap)
        if w["kind"] == "t":
            bounds += [w["width"] - (1 if tight_bounds else 0), batch]
        else:
            bounds += [w["nSites"] - (1 if tight_bounds else 0), nAct]
    ptr = lambda arrs, ct: (C.POINTER(ct) * nL)(*[C.cast(a[GUARD:].ctypes.data, C.POINTER(ct)) for a in arrs])
    report = np.zeros((nL + 1, 4), np.int64)
    caps = np.array(caps, np.int64)
    bounds = np.array(bounds, np.int64)
    S, K, R = np.ascontiguousarray(S, np.int32), np.ascontiguousarray(K, np.int64), np.ascontiguousarray(R, np.int32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    rc = lib.pyr_cpu_chain(d, batch, n0, nL, p(geo), p(S), p(K), p(R), C.c_longlong(len(K)), p(bg),
                           ptr(rules, C.c_int), p(caps), ptr(ekey, C.c_longlong), ptr(erow, C.c_int),
                           ptr(bgo, C.c_int), p(bounds), p(report), int(lds), int(T))
    for a, w in zip(rules, want):
        assert intact(a, max(w["rules"].size, 1))
    for a, b_, c, w in zip(ekey, erow, bgo, want):
        nAct = w["grids"].flat()[0].size
        assert intact(a, nAct + 1) and intact(b_, nAct + 1) and intact(c, batch)
    return rc, want, report, rules, ekey, erow, bgo


def check(lib, d, n0, layers, batch, seed, **kw):
    rc, want, report, rules, ekey, erow, bgo = run_chain(lib, d, n0, layers, batch, seed, **kw)
    assert rc == 0
    for l, w in enumerate(want):
        s, k, r, b = w["grids"].flat()
        nAct = s.size
        assert report[l + 1, 2] == 0
        assert report[l + 1, 0] == w["nSites"] and report[l + 1, 1] == (len(b) if w["kind"] == "t" else nAct)
        got = rules[l][GUARD:GUARD + w["rules"].size]
        assert np.array_equal(got, w["rules"]), "rule book of layer %d" % l
        assert np.array_equal(bgo[l][GUARD:GUARD + len(b)], b)
        if w["kind"] == "t":
            assert report[l + 1, 3] == w["width"]
            assert np.array_equal(ekey[l][GUARD:GUARD + len(b)], np.arange(len(b)))
            assert np.array_equal(erow[l][GUARD:GUARD + len(b)], np.arange(len(b)))
            continue
        # the entry list is in row order within a sample here, in key order in the oracle: compare as maps
        gk, gr = ekey[l][GUARD:GUARD + nAct], erow[l][GUARD:GUARD + nAct]
        mine = sorted(zip(gk.tolist(), gr.tolist()))
        theirs = sorted(zip((s.astype(np.int64) * w["volOut"] + k).tolist(), r.tolist()))
        assert mine == theirs, "entry list of layer %d" % l


CHAINS = [
    (2, 14, [("c", 2, 1), ("c", 3, 2), ("c", 2, 1), ("c", 3, 2), ("t",)]),
    (2, 30, [("c", 3, 1), ("c", 2, 2), ("c", 2, 1), ("c", 3, 2), ("c", 4, 2), ("t",)]),
    (2, 126, [("c", 2, 1), ("c", 3, 2), ("c", 2, 1), ("c", 3, 2), ("c", 2, 1), ("c", 3, 2), ("c", 2, 1), ("c", 3, 2),
              ("c", 2, 1), ("c", 3, 2), ("t",)]),
    (3, 11, [("c", 2, 1), ("c", 2, 2), ("c", 2, 1), ("c", 2, 2), ("t",)]),
    (3, 23, [("c", 2, 1), ("c", 2, 2), ("c", 2, 1), ("c", 2, 2), ("c", 2, 1), ("c", 2, 2)]),
    (1, 70, [("c", 3, 1), ("c", 2, 2), ("c", 16, 1), ("c", 1, 1), ("c", 4, 3), ("t",)]),
    (2, 9, [("t",)]),
    (2, 65, [("c", 3, 2)]),
    (2, 67, [("c", 4, 3), ("c", 1, 1), ("c", 2, 2)]),
]


@pytest.mark.parametrize("case", range(len(CHAINS)))
def test_output_side_chain_against_oracle(harness, case):
    d, n0, layers = CHAINS[case]
    fill = 0.08 if n0 ** d <= 8192 else 0.025  # (a sample has to fit the LDS: ten bytes a site over all layers)
    for seed, batch, T in ((1, 7, 64), (2, 1, 32), (3, 12, 512)):
        check(harness, d, n0, layers, batch, 100 * case + seed, T=T, fill=fill)


def test_dense_and_sparse_extremes(harness):
    check(harness, 2, 30, CHAINS[1][2], 5, 901, fill=0.9)
    check(harness, 2, 30, CHAINS[1][2], 5, 902, fill=0.002)
    check(harness, 3, 11, CHAINS[3][2], 4, 903, fill=0.7)


WINDOWED = [
    (2, 70, [("c", 2, 1)] * 5 + [("c", 3, 2), ("c", 2, 1), ("t",)], 0.05),
    (2, 70, [("c", 1, 1), ("c", 2, 1), ("c", 1, 1), ("c", 3, 1), ("c", 3, 2), ("c", 2, 1)], 0.05),
    (3, 17, [("c", 2, 1), ("c", 1, 1), ("c", 2, 1), ("c", 2, 1), ("c", 2, 2), ("c", 2, 1), ("t",)], 0.03),
    (1, 300, [("c", 3, 1), ("c", 2, 1), ("c", 5, 1), ("c", 3, 2), ("c", 3, 1), ("t",)], 0.2),
]


@pytest.mark.parametrize("case", range(len(WINDOWED)))
def test_levels_taken_a_window_at_a_time(harness, case):
    """With little LDS pass B builds a sample's layers in several windows of levels, the rows of a window's last
    level carried into the next one; the rule books are the same."""
    d, n0, layers, fill = WINDOWED[case]
    seen = set()
    for kb in list(range(7, 40)) + list(range(40, 153, 4)):
        rc, want, report, *_ = run_chain(harness, d, n0, layers, 5, 700 + case, fill=fill, lds=kb * 1024, T=64)
        if rc != 0:
            continue  # (not even one layer of some sample fits: reported, nothing written)
        w = int(report[0, 0])
        if w not in seen:
            check(harness, d, n0, layers, 5, 700 + case, fill=fill, lds=kb * 1024, T=64)
            check(harness, d, n0, layers, 5, 700 + case, fill=fill, lds=kb * 1024, T=512)
        seen.add(w)
    assert max(seen) >= 3, seen


def test_a_sample_that_outgrows_the_lds_is_reported(harness):
    d, n0, layers = CHAINS[1]
    rc, want, report, rules, *_ = run_chain(harness, d, n0, layers, 6, 5, fill=0.6, lds=8 * 1024)
    assert rc & 1 and np.all(report[1:, 2] == 1)
    for a, w in zip(rules, want):  # nothing was written
        assert np.all(a[GUARD:GUARD + max(w["rules"].size, 1)] == -99)


def test_a_layer_that_outgrows_its_bounds_is_reported(harness):
    d, n0, layers = CHAINS[0]
    rc, want, report, rules, *_ = run_chain(harness, d, n0, layers, 6, 6, tight_bounds=True)
    assert rc & 2 and np.all(report[1:, 2] == 1)
    for a, w in zip(rules, want):
        assert np.all(a[GUARD:GUARD + max(w["rules"].size, 1)] == -99)
