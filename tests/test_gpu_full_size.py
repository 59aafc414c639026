"""The headline configurations at their full batch sizes, checked through properties that do not need the oracle:
every rule book is rebuilt here with numpy from the grids alone (which sites exist, which rows they get, what each
rule names), every feature layer is checked against what its definition says of its input (gather = copy through
the rules, max-pool = first maximum, NiN on a sample of rows in float64, soft-max rows sum to one), and a sample's
result must not depend on what else is in the batch."""
import numpy as np
import pytest

from brute import rules_vectorized
from gpu_util import assert_probabilities

pytestmark = pytest.mark.gpu


def layer_geometry(stack):
    """per net layer: ("conv" | "pool", size, stride), ("nin",) or ("terminal",), in the order the builders add them."""
    out = []
    for call in stack:
        if call[0] == "addLeNetLayerMP":
            _, nF, fs, fstride, ps, pstride = call[:6]
            if fs > 1:
                out.append(("conv", fs, fstride))
            out.append(("nin",))
            if ps > 1:
                out.append(("pool", ps, pstride))
        elif call[0] == "addTerminalPoolingLayer":
            out.append(("terminal",))
        elif call[0] == "addSoftmaxLayer":
            out.append(("nin",))
    return out


def check_net(scn, number, batch, seed, nin_rows=1500, fused=False, max_rows=1 << 16, precision=None, tol=1e-4, warm=0,
              chained=None):
    """warm: batches the slot is given before the one that is checked (its first batch is always planned layer by
    layer through HBM; later ones through recorded plans where a sample's masks fit a compute unit's LDS, the second
    with the widest arena, the third with one sized by what the slot has seen -- the path of every batch of a long
    pass); chained: whether the checked batch must or must not have been planned that way."""
    from sparseconvnet_archived_amd import hostapi, synthetic
    cfg = synthetic.config(number, batch=batch)
    d = cfg.dimension
    net = hostapi.Net(d, cfg.nInputFeatures, cfg.nClasses, nTop=1, threads=2)
    cfg.build(net)
    net.setFusedConvolutions(fused)
    if precision is not None:
        net.setPrecision(precision)
    weights = synthetic.he_normal_weights(net.layers(), seed + 1)
    for i, (W, B, pr) in weights.items():
        net.set_weights(i, W, B, pr)
    samples = synthetic.make_samples(cfg, seed)
    ds = hostapi.Dataset(cfg.name, cfg.nInputFeatures, max(cfg.nClasses, 1), hostapi.TESTBATCH)
    for pts, f, label in samples:
        ds.add_points(d, cfg.lattice, pts, f, label)
    for _ in range(warm):
        net.begin(ds, batch)
        assert net.next_batch()
        net.end()
    chains = net.chain_counts()[0]
    net.begin(ds, batch)
    assert net.next_batch()
    if chained is not None:
        assert (net.chain_counts()[0] > chains) == chained
    layers = net.layers()
    geo = layer_geometry(cfg.stack)
    assert len(geo) == len(layers)
    rng = np.random.default_rng(seed)
    prev, before = net.interface(0), None
    for i, (g, l) in enumerate(zip(geo, layers)):
        cur = net.interface(i + 1)
        print("layer", i, l["kind"], g, "rows", cur["nSpatialSites"], flush=True)
        fin, fout = prev["features"], cur["features"]
        assert l["kind"].startswith({"conv": "conv", "pool": "maxpool", "nin": "nin", "terminal": "terminal"}[g[0]])
        if g[0] in ("conv", "pool"):
            (bs, ks, rows), bgOut, nRows, rules = rules_vectorized(
                d, batch, prev["spatialSize"], cur["spatialSize"], g[1], g[2], prev["grids"])
            assert cur["nSpatialSites"] == nRows
            s2, k2, r2, b2 = cur["grids"]
            o = np.lexsort((k2, s2))
            o2 = np.lexsort((ks, bs))
            assert np.array_equal(s2[o], bs[o2]) and np.array_equal(k2[o], ks[o2])  # the same sites exist
            assert np.array_equal(r2[o], rows[o2])  # ... and have the same rows
            assert np.array_equal(b2, bgOut)
            got = cur["rules"].reshape(nRows, -1)
            assert np.array_equal(got, rules)
            pick = np.arange(nRows) if nRows <= max_rows else np.sort(rng.choice(nRows, max_rows, replace=False))
            if g[0] == "conv":
                if fout is None:  # the gather runs inside the next NiN kernel
                    assert fused
                else:
                    assert np.array_equal(fout[pick], fin[got[pick]].reshape(len(pick), -1))  # copy through the rules
            else:
                cand = fin[got[pick]]  # [rows x window x channels]
                assert np.array_equal(fout[pick], cand.max(1))
                C_ = fin.shape[1]
                ch = cur["choices"].reshape(nRows, C_)[pick]
                # dMaxPool keeps the first maximum of the window; the choice is its element index in the input
                assert np.array_equal(ch, np.take_along_axis(got[pick], cand.argmax(1), 1) * C_ + np.arange(C_))
        elif g[0] == "nin":
            W, B, pr = weights[i]
            nR = cur["nSpatialSites"]
            pick = rng.choice(nR, min(nin_rows, nR), replace=False)
            if fin is None:  # rows of the convolution's output, gathered here
                A = before["features"][prev["rules"].reshape(nR, -1)[pick]].reshape(len(pick), -1)
            else:
                A = fin[pick]
            z = A.astype(np.float64) @ W.astype(np.float64) + B
            act = l["act"]
            if act == synthetic.SOFTMAX:
                assert np.allclose(fout.sum(1), 1, atol=1e-4)
                e = np.exp(z - z.max(1, keepdims=True))
                want = e / e.sum(1, keepdims=True)
                assert_probabilities(fout[pick], want, tol)  # each within tol of its row's largest
            else:
                slope = {synthetic.RELU: 0.0, synthetic.PRELU: None}.get(act, 1.0)
                want = np.where(z > 0, z, z * (pr if slope is None else slope))
                scale = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
                assert np.all(np.abs(fout[pick] - want) <= tol * scale)
        else:  # terminal pooling: a sample's row is the mean of its rows (TerminalPoolingLayer.cu:9-30)
            s, k, r, bg = prev["grids"]
            assert cur["nSpatialSites"] == batch
            sums = np.zeros((batch, fin.shape[1]), np.float64)
            np.add.at(sums, s, fin[r].astype(np.float64))
            n = np.bincount(s, minlength=batch)
            want = np.where(n[:, None] > 0, sums / np.maximum(n, 1)[:, None], fin[bg])  # an empty sample: its background
            assert np.allclose(fout, want, rtol=1e-4, atol=1e-6)
        before, prev = prev, cur
    out = net.batch_outputs() if cfg.nClasses > 1 else None
    net.end()
    return net, ds, samples, out


def test_config2_full_batch_rule_books_and_layers(scn):
    net, ds, samples, out = check_net(scn, 2, 100, 2015)
    # a sample's probabilities do not depend on the rest of the batch
    from sparseconvnet_archived_amd import hostapi
    for pickOne in (0, 57, 99):
        one = hostapi.Dataset("one", 3, 100, hostapi.TESTBATCH)
        pts, f, label = samples[pickOne]
        one.add_points(2, 96, pts, f, label)
        net.begin(one, 1)
        assert net.next_batch()
        alone = net.batch_outputs()["probabilities"][0]
        net.end()
        # (other kernels serve a batch of one: equal to rounding, not to the bit)
        assert_probabilities(alone[None], out["probabilities"][pickOne][None])
    net.close()


@pytest.mark.parametrize("number,batch,fused", [(1, 16, False), (3, 32, False), (4, 128, False), (4, 128, True),
                                                (5, 96, True)])
def test_full_batch_rule_books_and_layers(scn, number, batch, fused):
    net, ds, samples, out = check_net(scn, number, batch, 100 * number + 5, fused=fused, chained=False)
    net.close()


@pytest.mark.parametrize("number,batch,fused,warm", [(1, 16, False, 2), (2, 100, True, 1), (2, 100, True, 2),
                                                     (2, 100, False, 2), (3, 32, True, 1), (3, 32, True, 2),
                                                     (3, 32, False, 2), (4, 128, True, 2), (4, 128, False, 2)])
def test_full_batch_rule_books_from_recorded_plans(scn, number, batch, fused, warm):
    """The rule books every batch of a long pass gets -- recorded plans run as k_chain_sample / k_chain_place -- at the
    full field and batch of configs 1-4: the slot's second or third batch, rebuilt from the grids alone
    (gridRules per sample, Regions.cu:528-653, ConvolutionalLayer.cu:114-118), and every feature layer on top."""
    net, ds, samples, out = check_net(scn, number, batch, 100 * number + 7, fused=fused, warm=warm, chained=True)
    net.close()


def test_large_field_third_batch_is_planned_layer_by_layer(scn):
    """Config 5 (128^3: a sample's masks do not fit LDS) never takes the recorded plans; its third batch, planned
    with deferred counts through HBM, is checked like its first."""
    net, ds, samples, out = check_net(scn, 5, 96, 512, fused=True, warm=2, chained=False)
    net.close()


def test_wide_net_full_batch_bf16(scn):
    """The GEMM-bound net at its batch of 128 with bf16 operands: rule books rebuilt from the grids, every NiN layer
    on a sample of rows against float64 within 2e-2 of the row's scale (each layer is checked on the inputs it
    actually had, so the tolerance does not compound), pooling and gather exact."""
    for fused in (False, True):
        net, ds, samples, out = check_net(scn, 4, 128, 405, fused=fused, precision=scn.BF16, tol=2e-2)
        assert np.allclose(out["probabilities"].sum(1), 1, atol=1e-4)
        net.close()


@pytest.mark.parametrize("distinct,inputs_on_host", [(1, False), (1, True), (3, False)])
def test_benchmark_pass_against_oracle(scn, distinct, inputs_on_host):
    """The pass bench.py times, as it runs it: config 2 at batch 100, ten producer threads on two producer streams, two
    forward lanes, fused convolutions, priming batches, then warm-up + timed + tail batches in one
    scnh_forward_stream_timed(_many) pass, inputs resident in HBM or uploaded from pinned memory with every batch.
    Every batch of that pass must have come from recorded plans; the probabilities of all of them are compared with
    the float64 evaluation of the oracle's pass over the same batch, and the rule books, grids and background rows
    the last batch left in its slot with the oracle's, bit for bit."""
    import oracle_net
    from sparseconvnet_archived_amd import hostapi, synthetic
    cfg = synthetic.config(2)
    B, producers, warmup, steps = cfg.batch, 10, 5, 20
    assert B == 100
    net = hostapi.Net(cfg.dimension, cfg.nInputFeatures, cfg.nClasses, threads=producers)
    net.setProducerStreams(2)
    ora = oracle_net.Net(cfg.dimension, cfg.nInputFeatures, cfg.nClasses)
    cfg.build(net)
    cfg.build(ora)
    net.setFusedConvolutions(True)
    for i, (W, Bv, pr) in synthetic.he_normal_weights(net.layers(), 2016).items():
        net.set_weights(i, W, Bv, pr)
        ora.set_weights(i, W, Bv, pr)
    ctx = scn.Context(handle=net.context_handle())

    def pinned(a):
        h = ctx.host_alloc(a.nbytes)
        np.frombuffer(h.buffer(), a.dtype, a.size)[:] = a.reshape(-1)
        return h

    keep, descr, wants, p64 = [], [], [], []
    for i in range(distinct):
        samples = synthetic.make_samples(cfg, 2015 + 100 * i)
        S, K, R, bg, feats, n = synthetic.codify(samples, cfg.dimension, cfg.lattice, net.inputSpatialSize,
                                                 cfg.nInputFeatures)
        arrays = (S.astype(np.int32), K.astype(np.int64), R.astype(np.int32), bg.astype(np.int32),
                  feats.astype(np.float32))
        if inputs_on_host:
            arrs = [pinned(np.ascontiguousarray(x)) for x in arrays]
        else:
            arrs = [ctx.array(x, x.dtype) for x in arrays]
        keep.append(arrs)
        descr.append((B, arrs[0].ptr, arrs[1].ptr, arrs[2].ptr, arrs[3].ptr, int(len(K)), int(n), arrs[4].ptr))
        wants.append(ora.forward(B, S, K, R, bg, feats, n, np.array([s[2] for s in samples], np.int32)))
        p64.append(ora.forward64(wants[-1]))
    probs = np.zeros((B, cfg.nClasses), np.float32)
    priming = 3 * producers + distinct
    if distinct == 1:
        net.forward_stream_timed(0, priming, *descr[0], inputs_on_host=inputs_on_host, h_probs=probs)
    else:
        net.forward_stream_timed_many(0, priming, descr, inputs_on_host=inputs_on_host, h_probs=probs)
    net.setStreamTail(producers)
    nPass = warmup + steps + producers
    everything = np.zeros((nPass, B, cfg.nClasses), np.float32)
    net.collect_probabilities(everything)
    chains = net.chain_counts()[0]
    if distinct == 1:
        dt = net.forward_stream_timed(warmup, steps, *descr[0], inputs_on_host=inputs_on_host, h_probs=probs)
    else:
        dt = net.forward_stream_timed_many(warmup, steps, descr, inputs_on_host=inputs_on_host, h_probs=probs)
    net.collect_probabilities(None)
    print("benchmark pass: %.4f ms per batch, %d batches ready when the clock started"
          % (1e3 * dt / steps, net.streamReadyAtStart()), flush=True)
    # every batch of the pass had its rule books from recorded plans (k_chain_sample / k_chain_place)
    assert net.chain_counts()[0] == chains + nPass
    worst = 0.0
    for i in range(nPass):
        worst = max(worst, assert_probabilities(everything[i], p64[i % distinct]))
        assert np.array_equal(everything[i], everything[i % distinct])  # the same batch gives the same bits every time
    print("probabilities of %d batches: worst %.3g of the row's scale" % (nPass, worst), flush=True)
    # what the last batch of the pass left in its slot
    want = wants[(nPass - 1) % distinct]
    for i, wi in enumerate(want["interfaces"]):
        gi = net.interface(i, want_features=False)
        assert gi["nSpatialSites"] == wi["nSpatialSites"]
        assert np.array_equal(gi["rules"], wi["rules"])
        s, k, r, b = gi["grids"]
        os_, ok, or_, ob = wi["grids"].flat()
        assert np.array_equal(s, os_) and np.array_equal(k, ok) and np.array_equal(r, or_) and np.array_equal(b, ob)
    del keep
    net.close()


def test_ten_producers_several_passes_against_oracle(scn):
    """Ten producer threads, three batches (100, 100, 50) in flight at once on streams of their own, four passes over
    the same dataset: a slot's first batch is planned layer by layer, its second from recorded plans with the widest
    LDS arena, later ones with an arena sized by what the slot has seen -- with the chains of the three batches
    running side by side.  Every batch of every pass: row counts and rule books of all interfaces bit for bit, and
    the probabilities against float64."""
    import oracle_net
    from sparseconvnet_archived_amd import hostapi, synthetic
    cfg = synthetic.config(2)
    net = hostapi.Net(cfg.dimension, cfg.nInputFeatures, cfg.nClasses, threads=10)
    ora = oracle_net.Net(cfg.dimension, cfg.nInputFeatures, cfg.nClasses)
    cfg.build(net)
    cfg.build(ora)
    net.setFusedConvolutions(True)
    for i, (W, Bv, pr) in synthetic.he_normal_weights(net.layers(), 4).items():
        net.set_weights(i, W, Bv, pr)
        ora.set_weights(i, W, Bv, pr)
    samples = synthetic.make_samples(cfg, 11, batch=250)
    ds = hostapi.Dataset("three", cfg.nInputFeatures, cfg.nClasses, hostapi.TESTBATCH)
    for pts, f, label in samples:
        ds.add_points(cfg.dimension, cfg.lattice, pts, f, label)
    wants, p64 = [], []
    for lo in range(0, 250, 100):
        chunk = samples[lo:lo + 100]
        S, K, R, bg, feats, n = synthetic.codify(chunk, cfg.dimension, cfg.lattice, net.inputSpatialSize,
                                                 cfg.nInputFeatures)
        wants.append(ora.forward(len(chunk), S, K, R, bg, feats, n, np.array([s[2] for s in chunk], np.int32)))
        p64.append(ora.forward64(wants[-1]))
    for p in range(4):
        chains = net.chain_counts()[0]
        net.begin(ds, 100)
        for bi, want in enumerate(wants):
            assert net.next_batch()
            for i, wi in enumerate(want["interfaces"]):
                gi = net.interface(i, want_features=False)
                assert gi["nSpatialSites"] == wi["nSpatialSites"], "pass %d batch %d interface %d" % (p, bi, i)
                assert np.array_equal(gi["rules"], wi["rules"]), "pass %d batch %d interface %d" % (p, bi, i)
            assert_probabilities(net.batch_outputs()["probabilities"], p64[bi])
        assert not net.next_batch()
        assert net.chain_counts()[0] == chains + (3 if p else 0)
    net.close()
