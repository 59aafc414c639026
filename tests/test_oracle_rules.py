"""Pins for the oracle's rulebook generators (CPU only)."""
import itertools
import json
import os

import numpy as np
import pytest

import brute
import oracle as orc

GOLD = os.path.join(os.path.dirname(__file__), "golden", "rulebook_kats.json")


def to_grids(samples):
    g = orc.Grids(len(samples))
    for i, (bg, mp) in enumerate(samples):
        g.set(i, list(mp.keys()), list(mp.values()), bg)
    return g


def grids_as_dicts(g):
    out = []
    for i in range(g.batch):
        k, r = g.get(i)
        out.append((g.background(i), dict(zip(k.tolist(), r.tolist()))))
    return out


@pytest.mark.parametrize("case", json.load(open(GOLD))["cases"], ids=lambda c: c["name"])
def test_reference_executed_vectors(case):
    samples = [(s["bg"], dict(zip(s["keys"], s["rows"]))) for s in case["samples"]]
    g = to_grids(samples)
    fn = orc.rules_square if case["kind"] == "square" else orc.rules_triangular
    out, rules, n = fn(g, case["dimension"], case["nIn"], case["nOut"], case["size"], case["stride"], case["minActive"])
    assert n == case["nOutSites"]
    assert rules.tolist() == case["rules"]
    got = grids_as_dicts(out)
    for (bg, mp), exp in zip(got, case["out"]):
        assert bg == exp["bg"]
        assert mp == {int(k): v for k, v in exp["grid"].items()}
    if case["kind"] == "triangular":
        ordv, S = orc.tri_ord(case["size"], case["dimension"])
        assert ordv.tolist() == case["ord"] and S == case["S"]


def test_region_arithmetic_brute_force():
    # j in [outputL(i), outputR(i))  <=>  inputL(j) <= i < inputR(j)
    for size, stride, nOut in itertools.product(range(1, 6), range(1, 5), range(1, 7)):
        nIn = size + (nOut - 1) * stride
        for i in range(nIn):
            lo = orc.lib.orc_sq_outputL(size, stride, i)
            hi = orc.lib.orc_sq_outputR(size, stride, nOut, i)
            want = [j for j in range(nOut) if j * stride <= i < j * stride + size]
            assert list(range(lo, hi)) == want, (size, stride, nOut, i)
        for j in range(nOut):
            assert orc.lib.orc_sq_inputL(size, stride, j) == j * stride
            assert orc.lib.orc_sq_inputR(size, stride, j) == j * stride + size


def test_ipow_triangle_size_ord():
    for b, e in itertools.product(range(1, 7), range(0, 5)):
        assert orc.lib.orc_ipow(b, e) == b ** e
    for n, d in itertools.product(range(1, 7), range(1, 4)):
        assert orc.lib.orc_triangle_size(n, d) == brute.triangle_size(n, d)
    for s, d in itertools.product(range(1, 5), range(1, 4)):
        ordv, S = orc.tri_ord(s, d)
        bo, bS = brute.tri_ord(s, d)
        assert ordv.tolist() == bo and S == bS


GEOMS = [
    # d, size, stride, nOut
    (1, 2, 1, 6), (1, 3, 2, 4), (2, 2, 1, 5), (2, 3, 1, 4), (2, 3, 2, 3), (2, 2, 2, 4),
    (2, 2, 3, 3), (3, 2, 1, 3), (3, 3, 1, 2), (3, 2, 2, 2), (3, 3, 2, 2),
]


@pytest.mark.parametrize("d,size,stride,nOut", GEOMS)
@pytest.mark.parametrize("minActive", [1, 2, 3])
def test_square_rules_vs_brute_force(d, size, stride, nOut, minActive):
    rng = np.random.default_rng(1000 * d + 100 * size + 10 * stride + nOut + minActive)
    nIn = size + (nOut - 1) * stride
    for trial in range(12):
        density = [0.05, 0.2, 0.5, 0.9, 1.0, 0.0][trial % 6]
        samples, _ = brute.random_samples(rng, 1 + trial % 3, d, nIn, density)
        want_rules, want_n, want_out = brute.rules(samples, d, nIn, nOut, size, stride, minActive)
        out, rules, n = orc.rules_square(to_grids(samples), d, nIn, nOut, size, stride, minActive)
        assert n == want_n
        assert np.array_equal(rules, want_rules)
        assert grids_as_dicts(out) == want_out


@pytest.mark.parametrize("d,size,stride,nOut", GEOMS)
def test_whole_array_rule_book_vs_brute_force(d, size, stride, nOut):
    """brute.rules_vectorized (what the full-size GPU tests check against) agrees with the per-site brute force."""
    rng = np.random.default_rng(77 + 1000 * d + 100 * size + 10 * stride + nOut)
    nIn = size + (nOut - 1) * stride
    for trial in range(12):
        density = [0.05, 0.2, 0.5, 0.9, 1.0, 0.0][trial % 6]
        batch = 1 + trial % 3
        samples, _ = brute.random_samples(rng, batch, d, nIn, density)
        want_rules, want_n, want_out = brute.rules(samples, d, nIn, nOut, size, stride, 1)
        flat = to_grids(samples).flat()
        (bs, ks, rows), bgOut, n, rules = brute.rules_vectorized(d, batch, nIn, nOut, size, stride, flat)
        assert n == want_n
        assert np.array_equal(rules.ravel(), want_rules)
        for i, (bg, grid) in enumerate(want_out):
            assert bgOut[i] == bg
            m = bs == i
            assert dict(zip(ks[m].tolist(), rows[m].tolist())) == grid


def test_square_rules_valid_vs_brute_force():
    rng = np.random.default_rng(7)
    for nOut in (1, 2, 4, 7):
        nIn = nOut + 2
        for density in (0.1, 0.5, 1.0):
            samples, _ = brute.random_samples(rng, 2, 2, nIn, density)
            want_rules, want_n, want_out = brute.rules(samples, 2, nIn, nOut, 3, 1, -1)
            out, rules, n = orc.rules_square(to_grids(samples), 2, nIn, nOut, 3, 1, -1)
            assert n == want_n and np.array_equal(rules, want_rules)
            assert grids_as_dicts(out) == want_out


TRI_GEOMS = [(1, 2, 1, 4), (2, 2, 1, 4), (2, 3, 1, 3), (2, 3, 2, 3), (2, 2, 2, 3), (3, 2, 1, 3), (3, 3, 2, 2)]


@pytest.mark.parametrize("d,size,stride,nOut", TRI_GEOMS)
@pytest.mark.parametrize("minActive", [1, 2, 3])
def test_triangular_rules_vs_brute_force(d, size, stride, nOut, minActive):
    rng = np.random.default_rng(50 * d + 7 * size + stride + nOut + 3 * minActive)
    nIn = size + (nOut - 1) * stride
    for trial in range(12):
        density = [0.05, 0.3, 0.7, 1.0][trial % 4]
        samples, _ = brute.random_samples(rng, 1 + trial % 2, d, nIn, density)
        # a triangular lattice only has sites with coordinate sum < nIn
        samples = [(bg, {k: r for k, r in mp.items() if sum(brute.decode(k, nIn, d)) < nIn}) for bg, mp in samples]
        want_rules, want_n, want_out = brute.rules(samples, d, nIn, nOut, size, stride, minActive, triangular=True)
        out, rules, n = orc.rules_triangular(to_grids(samples), d, nIn, nOut, size, stride, minActive)
        assert n == want_n
        assert np.array_equal(rules, want_rules)
        assert grids_as_dicts(out) == want_out


def test_terminal_rules():
    rng = np.random.default_rng(3)
    samples, _ = brute.random_samples(rng, 4, 2, 3, 0.5)
    samples.append((99, {}))  # a sample with no active site pools its background row
    g = to_grids(samples)
    out, rules, S = orc.rules_terminal(g)
    want_S = max(1, max(len(mp) for _, mp in samples))
    assert S == want_S
    rules = rules.reshape(len(samples), S)
    for b, (bg, mp) in enumerate(samples):
        rows = [mp[k] for k in sorted(mp)] or [bg]
        assert rules[b].tolist() == rows + [-1] * (S - len(rows))
        assert grids_as_dicts(out)[b] == (-1, {0: b})


def test_bad_arguments():
    g = orc.Grids(1)
    g.set(0, [0], [1], 0)
    with pytest.raises(ValueError):
        orc.rules_square(g, 2, 6, 4, 2, 1)  # nIn != size + (nOut-1)*stride
    with pytest.raises(ValueError):
        orc.rules_square(g, 4, 3, 2, 2, 1)  # dimension 4 refused
    with pytest.raises(ValueError):
        orc.rules_square(g, 3, 5, 3, 3, 1, -1)  # valid mode is 2-D only
