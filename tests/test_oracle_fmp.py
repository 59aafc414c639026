"""Fractional max-pooling: the oracle's tick tables against closed forms and invariants, its rule books against a
brute-force builder over explicit windows."""
import numpy as np
import pytest

import brute
import oracle as orc
from test_oracle_rules import grids_as_dicts, to_grids


def draws(kind, nIn, nOut, rng):
    if kind in ("po", "pd"):
        return float(np.float32(rng.random()))
    inc = orc.fmp_increments(nIn, nOut, kind == "ro")
    rng.shuffle(inc)
    return inc


def test_pseudorandom_ticks_closed_forms():
    # u = 0: inputL[j] = floor(j alpha) exactly
    L, R = orc.fmp_ticks("po", 25, 18, 2, 0.0)
    alpha = (25 - 2) / 17
    assert L.tolist() == [int(j * alpha) for j in range(18)] and (R - L).tolist() == [2] * 18 and R[-1] == 25
    L, R = orc.fmp_ticks("pd", 10, 7, 2, 0.0)
    assert L.tolist() == [int(j * 10 / 7) for j in range(7)] and R.tolist() == [int(j * 10 / 7) for j in range(1, 8)]
    # the reference's asserts: nIn too small; ceil(alpha) != poolSize
    assert orc.fmp_ticks("po", 5, 5, 2, 0.5) is None
    assert orc.fmp_ticks("pd", 10, 7, 3, 0.5) is None
    assert orc.fmp_ticks("ro", 7, 7, 2, np.ones(6, np.int32)) is None


@pytest.mark.parametrize("kind", ["po", "pd", "ro", "rd"])
def test_tick_invariants(kind):
    rng = np.random.default_rng(sum(map(ord, kind)))
    for nOut in (2, 3, 7, 20, 41):
        for ratio in (1.2, 1.414, 1.6, 1.9):
            nIn = int(nOut * ratio + 0.5)
            if nIn == nOut:
                nIn += 1
            for trial in range(5):
                t = orc.fmp_ticks(kind, nIn, nOut, 2, draws(kind, nIn, nOut, rng))
                assert t is not None, (kind, nIn, nOut)
                L, R = t
                assert L[0] == 0 and R[-1] == nIn
                assert np.all(np.diff(L) >= 1) and np.all(np.diff(L) <= 2)  # steps of floor / ceil of a ratio in (1, 2)
                if kind in ("po", "ro"):
                    assert np.all(R - L == 2)
                else:  # a partition of the input axis
                    assert np.array_equal(R[:-1], L[1:]) and np.all((R - L >= 1) & (R - L <= 2))
                covered = np.zeros(nIn, int)
                for l, r in zip(L, R):
                    covered[l:r] += 1
                assert covered.min() >= 1  # every input cell is pooled by someone


def test_random_increments():
    inc = orc.fmp_increments(10, 7, False)
    assert inc.tolist() == [1, 1, 1, 1, 2, 2, 2] and inc.sum() == 10
    inc = orc.fmp_increments(10, 7, True)  # one fewer: the last region ends at nIn through its pool size
    assert inc.tolist() == [1, 1, 1, 1, 2, 2] and inc.sum() + 2 == 10


@pytest.mark.parametrize("kind", ["po", "pd", "ro", "rd"])
@pytest.mark.parametrize("d,nOut,nIn", [(1, 5, 7), (2, 4, 6), (2, 7, 10), (3, 3, 5)])
def test_fmp_rules_vs_brute_force(kind, d, nOut, nIn):
    rng = np.random.default_rng(d * 100 + nOut + len(kind) + ord(kind[1]))
    s = 2
    for trial in range(10):
        density = [0.05, 0.2, 0.5, 0.9, 1.0, 0.0][trial % 6]
        batch = 1 + trial % 3
        samples, _ = brute.random_samples(rng, batch, d, nIn, density)
        inL = np.empty((batch, d, nOut), np.int32)
        inR = np.empty((batch, d, nOut), np.int32)
        for b in range(batch):
            for a in range(d):
                inL[b, a], inR[b, a] = orc.fmp_ticks(kind, nIn, nOut, s, draws(kind, nIn, nOut, rng))
        uniform = kind in ("po", "ro")
        want_rules, want_n, want_out = brute.rules_windows(samples, d, nIn, nOut, s, inL, inR, uniform)
        out, rules, n = orc.rules_fmp(to_grids(samples), d, nIn, nOut, s, inL, inR, uniform)
        assert n == want_n
        assert np.array_equal(rules, want_rules)
        assert grids_as_dicts(out) == want_out


def test_regular_regions_are_a_special_case():
    """ticks inputL = j * stride, inputR = inputL + size reproduce the square rule book."""
    rng = np.random.default_rng(3)
    d, size, stride, nOut = 2, 3, 2, 4
    nIn = size + (nOut - 1) * stride
    samples, _ = brute.random_samples(rng, 3, d, nIn, 0.3)
    L = np.tile(np.arange(nOut, dtype=np.int32) * stride, (3, d, 1))
    out, rules, n = orc.rules_fmp(to_grids(samples), d, nIn, nOut, size, L, L + size, True)
    out2, rules2, n2 = orc.rules_square(to_grids(samples), d, nIn, nOut, size, stride, 1)
    assert n == n2 and np.array_equal(rules, rules2) and grids_as_dicts(out) == grids_as_dicts(out2)
