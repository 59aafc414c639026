"""Fractional max-pooling rule books on the GPU (scn_rules_fmp_plan + scn_rules_fill) against the oracle: bit-exact
rules, row numbering, output grids and background rows; then max-pooling through them."""
import numpy as np
import pytest

import brute
import oracle as orc
from gpu_util import assert_same_grids, device_grids, oracle_grids

pytestmark = pytest.mark.gpu


def draw_ticks(kind, batch, d, nIn, nOut, s, rng):
    inL = np.empty((batch, d, nOut), np.int32)
    inR = np.empty((batch, d, nOut), np.int32)
    for b in range(batch):
        for a in range(d):
            if kind in ("po", "pd"):
                draw = float(np.float32(rng.random()))
            else:
                draw = orc.fmp_increments(nIn, nOut, kind == "ro")
                rng.shuffle(draw)
            inL[b, a], inR[b, a] = orc.fmp_ticks(kind, nIn, nOut, s, draw)
    return inL, inR


@pytest.mark.parametrize("kind", ["po", "pd", "ro", "rd"])
@pytest.mark.parametrize("d,nOut,nIn", [(1, 5, 7), (2, 4, 6), (2, 7, 10), (2, 30, 42), (3, 3, 5), (3, 9, 13), (2, 61, 77)])
def test_fmp_rules(scn, ctx, kind, d, nOut, nIn):
    rng = np.random.default_rng(d * 100 + nOut + ord(kind[0]) + ord(kind[1]))
    s = 2
    for trial in range(6):
        density = [0.05, 0.2, 0.5, 0.9, 1.0, 0.0][trial]
        batch = 1 + trial % 4
        samples, nSites = brute.random_samples(rng, batch, d, nIn, density)
        inL, inR = draw_ticks(kind, batch, d, nIn, nOut, s, rng)
        print("fmp %s d=%d nIn=%d nOut=%d batch=%d density=%.2f" % (kind, d, nIn, nOut, batch, density), flush=True)
        o_out, o_rules, o_n = orc.rules_fmp(oracle_grids(samples), d, nIn, nOut, s, inL, inR, kind in ("po", "ro"))
        g = device_grids(scn, ctx, samples, d, nIn, nSites)
        d_out, d_rules, n, w = scn.rules_fmp(ctx, g, nIn, nOut, s, inL, inR)
        assert n == o_n and n * w == o_rules.size
        assert np.array_equal(d_rules.download()[: n * w], o_rules)
        assert_same_grids(d_out, o_out)


def test_fmp_pool_size_three_and_maxpool(scn, ctx):
    """overlapping regions of side 3 (boxes of up to 27 candidates in 3-D), then the pooling itself."""
    rng = np.random.default_rng(33)
    for d, nOut, nIn in [(2, 10, 16), (3, 5, 9)]:
        s, batch, C = 3, 3, 32
        samples, nSites = brute.random_samples(rng, batch, d, nIn, 0.15)
        inL, inR = draw_ticks("po", batch, d, nIn, nOut, s, rng)
        o_out, o_rules, o_n = orc.rules_fmp(oracle_grids(samples), d, nIn, nOut, s, inL, inR, True)
        g = device_grids(scn, ctx, samples, d, nIn, nSites)
        d_out, d_rules, n, w = scn.rules_fmp(ctx, g, nIn, nOut, s, inL, inR)
        assert n == o_n and np.array_equal(d_rules.download()[: n * w], o_rules)
        assert_same_grids(d_out, o_out)
        feats = rng.standard_normal((nSites, C)).astype(np.float32)
        d_o = ctx.empty((n, C), np.float32)
        d_c = ctx.empty((n, C), np.int32)
        ctx.maxpool(ctx.array(feats), d_o, d_rules, n, w, C, d_c)
        want, choice = orc.maxpool(feats, o_rules, n, w, C)
        assert np.array_equal(d_o.download(), want) and np.array_equal(d_c.download(), choice)


def test_fmp_disjoint_rows_hold_minus_one_and_pool(scn, ctx):
    rng = np.random.default_rng(34)
    d, nOut, nIn, s, batch, C = 2, 7, 10, 2, 4, 8
    samples, nSites = brute.random_samples(rng, batch, d, nIn, 0.4)
    inL, inR = draw_ticks("pd", batch, d, nIn, nOut, s, rng)
    g = device_grids(scn, ctx, samples, d, nIn, nSites)
    d_out, d_rules, n, w = scn.rules_fmp(ctx, g, nIn, nOut, s, inL, inR)
    rules = d_rules.download()[: n * w]
    assert (rules == -1).any()  # regions of one cell in a 2 x 2 row
    feats = rng.standard_normal((nSites, C)).astype(np.float32)
    d_o = ctx.empty((n, C), np.float32)
    d_c = ctx.empty((n, C), np.int32)
    ctx.maxpool(ctx.array(feats), d_o, d_rules, n, w, C, d_c)
    want, choice = orc.maxpool(feats, rules, n, w, C)
    assert np.array_equal(d_o.download(), want) and np.array_equal(d_c.download(), choice)


def test_fmp_regular_ticks_equal_the_square_rule_book(scn, ctx):
    rng = np.random.default_rng(35)
    d, size, stride, nOut = 2, 3, 2, 9
    nIn = size + (nOut - 1) * stride
    samples, nSites = brute.random_samples(rng, 3, d, nIn, 0.3)
    L = np.tile(np.arange(nOut, dtype=np.int32) * stride, (3, d, 1))
    g = device_grids(scn, ctx, samples, d, nIn, nSites)
    a_out, a_rules, n, w = scn.rules_fmp(ctx, g, nIn, nOut, size, L, L + size)
    b_out, b_rules, n2, w2 = scn.rules_square(ctx, g, nIn, nOut, size, stride)
    assert (n, w) == (n2, w2) and np.array_equal(a_rules.download()[: n * w], b_rules.download()[: n * w])


def test_fmp_bad_tables_are_refused(scn, ctx):
    rng = np.random.default_rng(36)
    samples, nSites = brute.random_samples(rng, 1, 2, 6, 0.5)
    g = device_grids(scn, ctx, samples, 2, 6, nSites)
    L = np.zeros((1, 2, 4), np.int32)
    for bad in (L + 7, L - 1):  # outside the grid
        with pytest.raises(scn.ScnError):
            scn.rules_fmp(ctx, g, 6, 4, 2, bad, bad + 2)
    with pytest.raises(scn.ScnError):  # wider than the pool size
        scn.rules_fmp(ctx, g, 6, 4, 2, L, L + 3)
