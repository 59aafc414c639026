"""Fractional max-pooling rule books on the GPU (scn_rules_fmp_plan + scn_rules_fill) against the oracle: bit-exact
rules, row numbering, output grids and background rows; then max-pooling through them."""
import numpy as np
import pytest

import brute
import oracle as orc
from gpu_util import assert_same_grids, device_grids, oracle_grids
from gpu_util import assert_probabilities

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


# ---- whole nets with fractional max-pooling layers through the C++ host classes
def rel_l2(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
@pytest.mark.parametrize("train", [False, True])
def test_net_with_fractional_max_pooling(scn, kind, train):
    """addLeNetLayerPOFMP / PDFMP / ROFMP / RDFMP: the regions the layers drew are read back and handed to the oracle;
    rule books and grids bit-exact, features to 1e-4, and (train) one training step through the pooling choices."""
    import oracle_net
    from sparseconvnet_archived_amd import hostapi, synthetic
    d, nIn, nClasses, batch = 2, 3, 10, 6
    shrink = 1.5
    net = hostapi.Net(d, nIn, nClasses, nTop=1, threads=2)
    ora = oracle_net.Net(d, nIn, nClasses, nTop=1)
    for n_ in (net, ora):
        n_.addLeNetLayerFMP(kind, 32, 2, 1, 2, shrink, synthetic.VLEAKYRELU)
        n_.addLeNetLayerFMP(kind, 64, 2, 1, 2, shrink, synthetic.VLEAKYRELU)
        n_.addLeNetLayerMP(64, 2, 1, 1, 1, synthetic.VLEAKYRELU)
        n_.addTerminalPoolingLayer(2)
        n_.addSoftmaxLayer()
    assert net.layers() == ora.layer_list()
    assert net.inputSpatialSize == ora.inputSpatialSize
    lattice = net.inputSpatialSize
    for i, (W, B, pr) in synthetic.he_normal_weights(net.layers(), 5).items():
        net.set_weights(i, W, B, pr)
        ora.set_weights(i, W, B, pr)
    rng = np.random.default_rng(40 + kind)
    samples = []
    for _ in range(batch):
        pts = np.array([(a, b) for a in range(lattice) for b in range(lattice) if rng.random() < 0.3], np.int32)
        samples.append((pts, rng.uniform(-1, 1, (len(pts), nIn)).astype(np.float32), int(rng.integers(0, nClasses))))
    ds = hostapi.Dataset("fmp", nIn, nClasses, hostapi.TRAINBATCH if train else hostapi.TESTBATCH)
    for pts, f, label in samples:
        ds.add_points(d, lattice, pts, f, label)
    net.set_training(0.01, 0.9, shuffle=False)
    net.begin(ds, batch)
    assert net.next_batch()
    layers = net.layers()
    ticks = {i: net.region_ticks(i + 1) for i, l in enumerate(layers) if l["kind"] == "fmp"}
    assert len(ticks) == 2 and all(t is not None for t in ticks.values())
    S, K, R, bg, feats, n = synthetic.codify(samples, d, lattice, lattice, nIn)
    labels = np.array([s[2] for s in samples], np.int32)
    want = ora.forward(batch, S, K, R, bg, feats, n, labels, ticks=ticks)
    for i, wi in enumerate(want["interfaces"]):
        gi = net.interface(i)
        assert gi["nSpatialSites"] == wi["nSpatialSites"] and gi["spatialSize"] == wi["spatialSize"]
        assert np.array_equal(gi["rules"], wi["rules"])
        s_, k_, r_, b_ = gi["grids"]
        os_, ok, or_, ob = wi["grids"].flat()
        assert np.array_equal(s_, os_) and np.array_equal(k_, ok) and np.array_equal(r_, or_) and np.array_equal(b_, ob)
        assert rel_l2(gi["features"], wi["features"]) <= 1e-4
        if i > 0 and layers[i - 1]["kind"] == "fmp":
            assert np.array_equal(gi["choices"], wi["choices"])
    out = net.batch_outputs()
    assert_probabilities(out["probabilities"], ora.forward64(want))
    if train:
        ora.train_step(want, labels, 0.01, 0.9)
        for i, wi in enumerate(want["interfaces"]):
            if "dfeatures" in wi:
                assert rel_l2(net.dfeatures(i), wi["dfeatures"]) <= 1e-4
        for i, l in enumerate(layers):
            if l["kind"].startswith("nin"):
                MW, MB, _ = net.get_weights(i, momentum=True)
                assert rel_l2(MW, ora.momentum[i][0]) <= 1e-4 and rel_l2(MB, ora.momentum[i][1]) <= 1e-4
    net.end()
    net.close()


def test_host_ticks_satisfy_the_invariants_and_vary(scn):
    """The regions drawn by the host library: partition / coverage invariants per kind, new for every sample."""
    from sparseconvnet_archived_amd import hostapi, synthetic
    for kind in range(4):
        net = hostapi.Net(2, 1, 4, nTop=1, threads=1)
        net.addLeNetLayerFMP(kind, 32, 2, 1, 2, 1.414, synthetic.RELU)
        net.addLeNetLayerFMP(kind, 32, 2, 1, 2, 1.414, synthetic.RELU)
        net.addLeNetLayerFMP(kind, 32, 2, 1, 2, 1.414, synthetic.RELU)
        net.addLeNetLayerMP(32, 2, 1, 1, 1, synthetic.RELU)
        net.addTerminalPoolingLayer(2)
        net.addSoftmaxLayer()
        lattice = net.inputSpatialSize
        ds = hostapi.Dataset("t", 1, 4, hostapi.TESTBATCH)
        for b in range(8):
            ds.add_points(2, lattice, np.array([[b, b], [b + 1, b]], np.int32), np.ones((2, 1), np.float32), 0)
        net.begin(ds, 8)
        assert net.next_batch()
        seen = set()
        for i, l in enumerate(net.layers()):
            if l["kind"] != "fmp":
                continue
            L, R = net.region_ticks(i + 1)
            nInAxis = net.interface(i)["spatialSize"]
            for b in range(8):
                for a in range(2):
                    l_, r_ = L[b, a], R[b, a]
                    assert l_[0] == 0 and r_[-1] == nInAxis and np.all(np.diff(l_) >= 1)
                    if kind in (0, 2):
                        assert np.all(r_ - l_ == 2)
                    else:
                        assert np.array_equal(r_[:-1], l_[1:])
                    seen.add((i, tuple(l_)))
        assert len(seen) > 8  # not one draw repeated everywhere
        net.end()
        net.close()
