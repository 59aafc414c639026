"""Rule books built on the GPU against the CPU oracle: bit-exact rules, row
numbering, output grids and background rows (through the C ABI)."""
import json
import os

import numpy as np
import pytest

import brute
import oracle as orc
from gpu_util import assert_same_grids, device_grids, flatten_samples, oracle_grids

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "rulebook_kats.json")


def run_both(scn, ctx, samples, d, nIn, nOut, size, stride, minActive, tri, nSites):
    print("case d=%d nIn=%d nOut=%d size=%d stride=%d min=%d tri=%d batch=%d" %
          (d, nIn, nOut, size, stride, minActive, tri, len(samples)), flush=True)
    fn = orc.rules_triangular if tri else orc.rules_square
    o_out, o_rules, o_n = fn(oracle_grids(samples), d, nIn, nOut, size, stride, minActive)
    g = device_grids(scn, ctx, samples, d, nIn, nSites)
    d_out, d_rules, n, w = scn.rules_square(ctx, g, nIn, nOut, size, stride, minActive, triangular=tri)
    assert n == o_n
    assert n * w == o_rules.size
    got = d_rules.download()[: n * w]
    assert np.array_equal(got, o_rules)
    assert_same_grids(d_out, o_out)
    assert d_out.info()["nSpatialSites"] == o_n
    return d_out, o_out


@pytest.mark.parametrize("case", json.load(open(GOLD))["cases"], ids=lambda c: c["name"])
def test_reference_executed_vectors_on_gpu(scn, ctx, case):
    samples = [(s["bg"], dict(zip(s["keys"], s["rows"]))) for s in case["samples"]]
    nSites = 1 + max([s["bg"] for s in case["samples"]] + [r for s in case["samples"] for r in s["rows"]])
    g = device_grids(scn, ctx, samples, case["dimension"], case["nIn"], nSites)
    out, rules, n, w = scn.rules_square(ctx, g, case["nIn"], case["nOut"], case["size"], case["stride"],
                                        case["minActive"], triangular=case["kind"] == "triangular")
    assert n == case["nOutSites"]
    assert rules.download()[: n * w].tolist() == case["rules"]
    s, k, r, bg = out.download()
    for i, exp in enumerate(case["out"]):
        assert bg[i] == exp["bg"]
        got = {int(kk): int(rr) for ss, kk, rr in zip(s, k, r) if ss == i}
        assert got == {int(kk): v for kk, v in exp["grid"].items()}


GEOMS = [(1, 2, 1, 6), (1, 3, 2, 4), (2, 2, 1, 5), (2, 3, 1, 4), (2, 3, 2, 3), (2, 2, 2, 4), (2, 2, 3, 3),
         (3, 2, 1, 3), (3, 3, 1, 2), (3, 2, 2, 2), (3, 3, 2, 2), (2, 3, 1, 30), (3, 3, 1, 9), (2, 5, 3, 7), (1, 2, 2, 5), (3, 2, 2, 5)]


@pytest.mark.parametrize("d,size,stride,nOut", GEOMS)
@pytest.mark.parametrize("minActive", [1, 2, 3])
def test_square_rules(scn, ctx, d, size, stride, nOut, minActive):
    rng = np.random.default_rng(77 * d + 13 * size + 5 * stride + nOut + minActive)
    nIn = size + (nOut - 1) * stride
    for trial in range(6):
        density = [0.05, 0.2, 0.5, 0.9, 1.0, 0.0][trial]
        samples, nSites = brute.random_samples(rng, 1 + trial % 4, d, nIn, density)
        run_both(scn, ctx, samples, d, nIn, nOut, size, stride, minActive, False, nSites)


WIDE_GEOMS = [(1, 3, 1, 300), (1, 3, 2, 150), (1, 5, 3, 90), (2, 2, 1, 100), (2, 3, 2, 70), (2, 4, 3, 45), (3, 3, 1, 70),
              (3, 2, 2, 40), (1, 2, 2, 100), (2, 2, 2, 50), (3, 2, 2, 33)]


@pytest.mark.parametrize("d,size,stride,nOut", WIDE_GEOMS)
def test_square_rules_rows_longer_than_a_mask_word(scn, ctx, d, size, stride, nOut):
    """Fields whose rows span several 64-bit mask words and do not start on word boundaries (the output mask of these
    rule books is derived from the input mask a word at a time)."""
    rng = np.random.default_rng(1000 * d + 100 * size + 10 * stride + nOut)
    nIn = size + (nOut - 1) * stride
    for density in (0.002, 0.03, 0.6):
        samples, nSites = brute.random_samples(rng, 3, d, nIn, density)
        run_both(scn, ctx, samples, d, nIn, nOut, size, stride, 1, False, nSites)


@pytest.mark.parametrize("d,nIn,size,stride,batch,density", [(2, 1025, 3, 2, 5, 0.02), (3, 130, 2, 1, 3, 0.015),
                                                            (2, 1500, 2, 2, 2, 0.03)])
def test_rule_books_whose_prefix_sums_take_many_tiles(scn, ctx, d, nIn, size, stride, batch, density):
    """Masks of more than 65536 words and more than 65536 active sites: both prefix sums of a plan (set bits of the
    mask, candidates per input) are then made in one pass over many tiles, each workgroup adding up what the tiles
    before it have published."""
    rng = np.random.default_rng(nIn + size)
    nOut = (nIn - size) // stride + 1
    samples, nSites = brute.random_samples(rng, batch, d, nIn, density)
    assert batch * nIn ** d > 64 * 65536 and sum(len(m) for _, m in samples) > 65536
    run_both(scn, ctx, samples, d, nIn, nOut, size, stride, 1, False, nSites)
    # an input with a few very long runs of empty tiles between its sites
    sparse = []
    row = 0
    for b in range(batch):
        keys = rng.choice(nIn ** d, size=37, replace=False)
        sparse.append((row, {int(k): row + 1 + i for i, k in enumerate(keys)}))
        row += 38
    run_both(scn, ctx, sparse, d, nIn, nOut, size, stride, 1, False, row)


def test_find_on_grids_without_a_table(scn, ctx):
    """Look-ups by coordinate on grids whose hash table is only built when asked for: input grids of a batch too large
    for a dense row table, and the output grids of a rule-book plan (which never get either as they are built)."""
    rng = np.random.default_rng(21)
    d, nIn = 3, 210  # 2 x 210^3 sites: beyond the batches that get a dense row table as they are built
    samples = []
    row = 0
    for b in range(2):
        keys = rng.choice(nIn ** d, size=500, replace=False)
        samples.append((-1, {int(k): row + i for i, k in enumerate(keys)}))
        row += 500
    samples = [(row + b, mp) for b, (_, mp) in enumerate(samples)]
    g = device_grids(scn, ctx, samples, d, nIn, row + 2)
    qs = [0] * 300 + [1] * 300
    qk = [int(k) for k in list(samples[0][1])[:150]] + [int(k) for k in rng.integers(0, nIn ** d, 150)] + \
         [int(k) for k in list(samples[1][1])[:150]] + [int(k) for k in rng.integers(0, nIn ** d, 150)]
    want = [samples[b][1].get(k, -1) for b, k in zip(qs, qk)]
    assert g.find(qs, qk).tolist() == want
    # the outputs of a plan, before and after their rules are filled
    o_out, o_rules, o_n = orc.rules_square(oracle_grids(samples), d, nIn, nIn - 2, 3, 1, 1)
    out = scn.Grids(ctx)
    n = g.plan_square(out, nIn, nIn - 2, 3, 1)
    assert n == o_n
    os_, ok, or_, _ = o_out.flat()
    omap = {(int(a), int(b)): int(c) for a, b, c in zip(os_, ok, or_)}
    pick = rng.choice(len(ok), size=200, replace=False)
    assert out.find(os_[pick], ok[pick]).tolist() == or_[pick].tolist()
    rules = ctx.empty(n * 27, np.int32)
    g.fill(out, rules, n * 27)
    assert np.array_equal(rules.download()[: n * 27], o_rules)
    assert out.find([1] * 3, [0, 1, 2]).tolist() == [omap.get((1, k), -1) for k in (0, 1, 2)]


def test_valid_rules(scn, ctx):
    rng = np.random.default_rng(8)
    for nOut in (1, 2, 4, 7, 20):
        for density in (0.1, 0.5, 1.0):
            samples, nSites = brute.random_samples(rng, 3, 2, nOut + 2, density)
            run_both(scn, ctx, samples, 2, nOut + 2, nOut, 3, 1, -1, False, nSites)


TRI_GEOMS = [(1, 2, 1, 4), (2, 2, 1, 4), (2, 3, 1, 3), (2, 3, 2, 3), (2, 2, 2, 3), (3, 2, 1, 3), (3, 3, 2, 2), (2, 3, 1, 12)]


@pytest.mark.parametrize("d,size,stride,nOut", TRI_GEOMS)
@pytest.mark.parametrize("minActive", [1, 2, 3])
def test_triangular_rules(scn, ctx, d, size, stride, nOut, minActive):
    rng = np.random.default_rng(31 * d + 7 * size + stride + nOut + 3 * minActive)
    nIn = size + (nOut - 1) * stride
    for trial in range(4):
        density = [0.05, 0.3, 0.7, 1.0][trial]
        samples, nSites = brute.random_samples(rng, 1 + trial % 3, d, nIn, density)
        samples = [(bg, {k: r for k, r in mp.items() if sum(brute.decode(k, nIn, d)) < nIn}) for bg, mp in samples]
        run_both(scn, ctx, samples, d, nIn, nOut, size, stride, minActive, True, nSites)


def test_terminal_rules(scn, ctx):
    rng = np.random.default_rng(5)
    samples, nSites = brute.random_samples(rng, 5, 2, 3, 0.5)
    samples.append((nSites, {}))
    nSites += 1
    o_out, o_rules, o_S = orc.rules_terminal(oracle_grids(samples))
    g = device_grids(scn, ctx, samples, 2, 3, nSites)
    d_out, d_rules, S = scn.rules_terminal(ctx, g)
    assert S == o_S
    assert np.array_equal(d_rules.download()[: len(samples) * S], o_rules)
    assert_same_grids(d_out, o_out)


def test_chained_layers_2d(scn, ctx):
    """C2 then MP3/2 twice: deeper layers consume grids the library produced."""
    rng = np.random.default_rng(11)
    field = 2 + 0  # placeholder, computed below
    # sizes: 29 -(C2)- 28 -(MP3/2)- 13 ... use out=3: 3 ->(MP3/2) 7 ->(C2) 8 ->(MP3/2) 17 ->(C2) 18
    sizes = [18, 17, 8, 7, 3]
    samples, nSites = brute.random_samples(rng, 6, 2, sizes[0], 0.06)
    og = oracle_grids(samples)
    dg = device_grids(scn, ctx, samples, 2, sizes[0], nSites)
    geoms = [(2, 1), (3, 2), (2, 1), (3, 2)]
    for (size, stride), nIn, nOut in zip(geoms, sizes[:-1], sizes[1:]):
        print("chain", nIn, nOut, size, stride, flush=True)
        og2, o_rules, o_n = orc.rules_square(og, 2, nIn, nOut, size, stride, 1)
        dg2, d_rules, n, w = scn.rules_square(ctx, dg, nIn, nOut, size, stride, 1)
        assert n == o_n and np.array_equal(d_rules.download()[: n * w], o_rules)
        assert_same_grids(dg2, og2)
        og, dg = og2, dg2
    o_out, o_rules, o_S = orc.rules_terminal(og)
    d_out, d_rules, S = scn.rules_terminal(ctx, dg)
    assert S == o_S and np.array_equal(d_rules.download()[: 6 * S], o_rules)


def test_grids_reused_across_batches_with_one_clear(scn, ctx):
    """The same grids objects take three batches in a row (large, small, large)
    with scn_grids_clear_many at the start of each, as the host classes do:
    nothing of an earlier batch may survive in a table or a mask."""
    rng = np.random.default_rng(21)
    sizes = [18, 17, 8]
    geoms = [(2, 1), (3, 2)]
    dg = scn.Grids(ctx)
    outs = [scn.Grids(ctx), scn.Grids(ctx)]
    for batch, density in ((7, 0.08), (2, 0.02), (5, 0.3)):
        samples, nSites = brute.random_samples(rng, batch, 2, sizes[0], density)
        scn.clear_many(ctx, [dg] + outs)
        s, k, r, bg = flatten_samples(samples)
        dg.build(len(samples), 2, sizes[0], s, k, r, bg, nSites)
        og, cur = oracle_grids(samples), dg
        for (size, stride), nIn, nOut, out in zip(geoms, sizes[:-1], sizes[1:], outs):
            og2, o_rules, o_n = orc.rules_square(og, 2, nIn, nOut, size, stride, 1)
            d2, d_rules, n, w = scn.rules_square(ctx, cur, nIn, nOut, size, stride, 1, out=out)
            assert n == o_n and np.array_equal(d_rules.download()[: n * w], o_rules)
            assert_same_grids(d2, og2)
            og, cur = og2, d2


def _chain(scn, ctx, dg, outs, term, samples, sizes, geoms):
    """conv/pool chain + terminal layer into existing grids objects; returns what fill produced."""
    got, cur = [], dg
    for (size, stride), nIn, nOut, out in zip(geoms, sizes[:-1], sizes[1:], outs):
        d2, d_rules, n, w = scn.rules_square(ctx, cur, nIn, nOut, size, stride, 1, out=out)
        got.append((d2, d_rules, n, w))
        cur = d2
    S = cur.plan_terminal(term)
    t_rules = ctx.empty(max(len(samples) * S, 1), np.int32)
    cur.fill(term, t_rules, len(samples) * S)
    got.append((term, t_rules, len(samples), S))
    return got


@pytest.mark.parametrize("sizes,geoms", [([18, 17, 8, 7], [(2, 1), (3, 2), (2, 1)]),
                                         ([19, 18, 9, 7], [(2, 1), (2, 2), (3, 1)])])
def test_deferred_counts(scn, ctx, sizes, geoms):
    """scn_ctx_defer_counts / scn_rules_settle: a batch that fits the bounds of
    the previous one is planned without waiting and gives the same rule books
    and grids; a batch that outgrows them is reported and planned again.  (The
    second chain has windows of side 2 at stride 2, whose owners are read off
    the input mask a word at a time.)"""
    rng = np.random.default_rng(31)
    dg = scn.Grids(ctx)
    outs = [scn.Grids(ctx) for _ in geoms]
    term = scn.Grids(ctx)

    def oracle_chain(samples):
        og, want = oracle_grids(samples), []
        for (size, stride), nIn, nOut in zip(geoms, sizes[:-1], sizes[1:]):
            og2, o_rules, o_n = orc.rules_square(og, 2, nIn, nOut, size, stride, 1)
            want.append((og2, o_rules, o_n))
            og = og2
        o_out, o_rules, o_S = orc.rules_terminal(og)
        want.append((o_out, o_rules, o_S))
        return want

    def check(got, want, batch):
        for (dgr, d_rules, n, w), (ogr, o_rules, o_n) in zip(got[:-1], want[:-1]):
            info = dgr.info()
            assert info["nSpatialSites"] == o_n
            assert np.array_equal(d_rules.download()[: o_n * w], o_rules)
            assert_same_grids(dgr, ogr)
        (dgr, d_rules, _, _), (ogr, o_rules, o_S) = got[-1], want[-1]
        assert dgr.rules_width() == o_S
        assert np.array_equal(d_rules.download()[: batch * o_S], o_rules)

    def build(samples, nSites):
        scn.clear_many(ctx, [dg] + outs + [term])
        s, k, r, bg = flatten_samples(samples)
        dg.build(len(samples), 2, sizes[0], s, k, r, bg, nSites)

    # 1: exact (no history yet), establishes the bounds
    samples, nSites = brute.random_samples(rng, 6, 2, sizes[0], 0.10)
    build(samples, nSites)
    check(_chain(scn, ctx, dg, outs, term, samples, sizes, geoms), oracle_chain(samples), 6)
    # 2: deferred, a little smaller and a little larger than batch 1 (within the 25 % head room)
    for density in (0.07, 0.11):
        samples, nSites = brute.random_samples(rng, 6, 2, sizes[0], density)
        build(samples, nSites)
        scn.defer_counts(ctx, True)
        got = _chain(scn, ctx, dg, outs, term, samples, sizes, geoms)
        with pytest.raises(scn.ScnError):
            got[0][0].info()  # not readable before the counts are settled
        scn.defer_counts(ctx, False)
        assert scn.settle(ctx)
        check(got, oracle_chain(samples), 6)
    # 3: deferred, far denser: outgrows the bounds, is reported, and planned again the exact way
    samples, nSites = brute.random_samples(rng, 6, 2, sizes[0], 0.6)
    build(samples, nSites)
    scn.defer_counts(ctx, True)
    _chain(scn, ctx, dg, outs, term, samples, sizes, geoms)
    scn.defer_counts(ctx, False)
    assert not scn.settle(ctx)
    check(_chain(scn, ctx, dg, outs, term, samples, sizes, geoms), oracle_chain(samples), 6)
    # 4: and the raised bounds now hold for a batch of that size
    samples, nSites = brute.random_samples(rng, 6, 2, sizes[0], 0.55)
    build(samples, nSites)
    scn.defer_counts(ctx, True)
    got = _chain(scn, ctx, dg, outs, term, samples, sizes, geoms)
    scn.defer_counts(ctx, False)
    assert scn.settle(ctx)
    check(got, oracle_chain(samples), 6)


def test_larger_3d_batch(scn, ctx):
    rng = np.random.default_rng(12)
    nOut, size, stride = 22, 3, 1
    nIn = size + (nOut - 1) * stride
    samples, nSites = brute.random_samples(rng, 8, 3, nIn, 0.02)
    d_out, o_out = run_both(scn, ctx, samples, 3, nIn, nOut, size, stride, 1, False, nSites)
    # pool the result 2/2
    o2, o_rules, o_n = orc.rules_square(o_out, 3, nOut, nOut // 2, 2, 2, 1)
    d2, d_rules, n, w = scn.rules_square(ctx, d_out, nOut, nOut // 2, 2, 2, 1)
    assert n == o_n and np.array_equal(d_rules.download()[: n * w], o_rules)
    assert_same_grids(d2, o2)


def test_find_and_errors(scn, ctx):
    samples = [(0, {7: 1, 6: 2, 19: 3})]
    g = device_grids(scn, ctx, samples, 2, 5, 4)
    got = g.find([0, 0, 0, 0, 1], [6, 7, 8, 19, 6])
    assert got.tolist() == [2, 1, -1, 3, -1]
    out = scn.Grids(ctx)
    with pytest.raises(scn.ScnError):
        g.plan_square(out, 6, 4, 2, 1)  # nIn != size + (nOut - 1) * stride
    with pytest.raises(scn.ScnError):
        g.plan_square(out, 5, 3, 3, 1, -1) and g.plan_square(out, 5, 4, 2, 1, -1)
    with pytest.raises(scn.ScnError):
        g.fill(out, ctx.empty(4, np.int32))  # no plan
    n = g.plan_square(out, 5, 4, 2, 1)
    with pytest.raises(scn.ScnError):
        g.fill(out, ctx.empty(4, np.int32), 4)  # capacity
    assert n == 9


def test_sites_outside_the_field_are_reported(scn, ctx):
    g = scn.Grids(ctx)
    # key 30 does not exist in a 5 x 5 field; sample 3 does not exist in a batch of 1
    g.build(1, 2, 5, [0, 0, 3], [7, 30, 2], [1, 2, 3], [0], 4)
    out = scn.Grids(ctx)
    with pytest.raises(scn.ScnError, match="outside the field"):
        g.plan_square(out, 5, 4, 2, 1)
    # the context stays usable
    g.build(1, 2, 5, [0, 0], [7, 6], [1, 2], [0], 3)
    assert g.plan_square(out, 5, 4, 2, 1) == 7


def test_empty_batch_and_empty_samples(scn, ctx):
    samples = [(0, {}), (1, {3: 2}), (3, {})]
    run_both(scn, ctx, samples, 2, 5, 4, 2, 1, 1, False, 4)
    run_both(scn, ctx, [(0, {})], 3, 4, 2, 3, 1, 1, False, 1)
