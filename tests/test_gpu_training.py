"""Training batches through the C++ host classes (processBatch with a TRAINBATCH: forward, SoftmaxClassifier's
gradient, backwards() of every layer, momentum step) against the net-level oracle, and the sanity property that
training lowers the cost."""
import numpy as np
import pytest

import oracle_net
from gpu_util import assert_nll, assert_probabilities

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = a.astype(np.float64).ravel()
    b = b.astype(np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def pair(cfg, hostapi, seed, triangular=False, fused=False):
    from sparseconvnet_archived_amd import synthetic
    net = hostapi.Net(cfg.dimension, cfg.nInputFeatures, cfg.nClasses, nTop=1, threads=2, triangular=triangular)
    ora = oracle_net.Net(cfg.dimension, cfg.nInputFeatures, cfg.nClasses, nTop=1, triangular=triangular)
    cfg.build(net)
    cfg.build(ora)
    net.setFusedConvolutions(fused)
    for i, (W, B, pr) in synthetic.he_normal_weights(net.layers(), seed).items():
        B = (np.random.default_rng(seed + i).standard_normal(B.shape) * 0.05).astype(np.float32)
        net.set_weights(i, W, B, pr)
        ora.set_weights(i, W, B, pr)
    return net, ora


def train_and_compare(scn, cfg, samples, nBatches, lr=0.01, momentum=0.9, triangular=False, fused=False, tol=1e-4):
    from sparseconvnet_archived_amd import hostapi, synthetic
    net, ora = pair(cfg, hostapi, 77, triangular, fused)
    ds = hostapi.Dataset(cfg.name, cfg.nInputFeatures, cfg.nClasses, hostapi.TRAINBATCH)
    for pts, f, label in samples:
        ds.add_points(cfg.dimension, cfg.lattice, pts, f, label)
    batch = len(samples) // nBatches
    net.set_training(lr, momentum, shuffle=False)
    net.begin(ds, batch)
    layers = net.layers()
    for b in range(nBatches):
        print("training batch", b, flush=True)
        assert net.next_batch()
        mine = samples[b * batch:(b + 1) * batch]
        S, K, R, bg, feats, n = synthetic.codify(mine, cfg.dimension, cfg.lattice, net.inputSpatialSize,
                                                 cfg.nInputFeatures)
        labels = np.array([s[2] for s in mine], np.int32)
        fwd = ora.forward(len(mine), S, K, R, bg, feats, n, labels)
        p64 = ora.forward64(fwd)  # (with the weights the batch saw)
        ora.train_step(fwd, labels, lr, momentum)
        out = net.batch_outputs()
        assert_probabilities(out["probabilities"], p64)
        assert_nll(out["nll"], p64, labels)
        # gradients at every interface the backward pass reaches
        for i, wi in enumerate(fwd["interfaces"]):
            got = net.dfeatures(i)
            if "dfeatures" not in wi:
                continue
            err = rel_l2(got, wi["dfeatures"])
            print("  interface %d: gradient rel-L2 error %.3g (%d values)" % (i, err, got.size), flush=True)
            assert got.size == wi["dfeatures"].size
            assert err <= tol
        # updated weights and momentum of every layer with weights
        for i, l in enumerate(layers):
            if not l["kind"].startswith("nin"):
                continue
            W, B, pr = net.get_weights(i)
            MW, MB, MP = net.get_weights(i, momentum=True)
            oW, oB, opr = ora.weights[i]
            oMW, oMB, oMP = ora.momentum[i]
            eW, eB = rel_l2(MW, oMW), rel_l2(MB, oMB)
            print("  layer %d: momentum rel-L2 error W %.3g B %.3g" % (i, eW, eB), flush=True)
            assert eW <= tol and eB <= tol
            assert np.allclose(W, oW, rtol=1e-4, atol=1e-6) and np.allclose(B, oB, rtol=1e-4, atol=1e-6)
            if pr is not None:
                assert rel_l2(MP, oMP) <= tol and np.allclose(pr, opr, rtol=1e-4, atol=1e-6)
    assert not net.next_batch()
    net.close()


def test_train_config2_two_batches(scn):
    from sparseconvnet_archived_amd import synthetic
    cfg = synthetic.config(2, batch=16)
    train_and_compare(scn, cfg, synthetic.make_samples(cfg, 301), 2)


def test_train_config3_voxels(scn):
    from sparseconvnet_archived_amd import synthetic
    cfg = synthetic.config(3, batch=6)
    train_and_compare(scn, cfg, synthetic.make_samples(cfg, 302), 1)


def test_train_fused_setting_gathers_while_training(scn):
    """setFusedConvolutions(true) must not change a training step: the backward pass needs the gathered matrix."""
    from sparseconvnet_archived_amd import synthetic
    cfg = synthetic.config(2, batch=8)
    train_and_compare(scn, cfg, synthetic.make_samples(cfg, 303), 1, fused=True)


def test_train_triangular_leaky_tanh(scn):
    from sparseconvnet_archived_amd import synthetic
    stack = [("addLeNetLayerMP", 32, 2, 1, 2, 2, synthetic.VLEAKYRELU), ("addLeNetLayerMP", 64, 2, 1, 2, 2, synthetic.TANH),
             ("addLeNetLayerMP", 64, 2, 1, 1, 1, synthetic.LEAKYRELU), ("addTerminalPoolingLayer", 2), ("addSoftmaxLayer",)]
    cfg = synthetic.Config("tri", 2, 3, 10, 8, 13, stack)
    cfg.number = 2
    rng = np.random.default_rng(5)
    samples = []
    for _ in range(8):
        pts = np.array([(a, b) for a in range(13) for b in range(13 - a) if rng.random() < 0.4], np.int32)
        samples.append((pts, rng.uniform(-1, 1, (len(pts), 3)).astype(np.float32), int(rng.integers(0, 10))))
    train_and_compare(scn, cfg, samples, 1, triangular=True)


def test_training_lowers_the_cost(scn):
    """processDataset on a TRAINBATCH dataset, a few epochs: the negative log-likelihood of the training set falls
    well below that of the untrained net."""
    from sparseconvnet_archived_amd import hostapi, synthetic
    stack = [("addLeNetLayerMP", 32, 3, 1, 2, 2, synthetic.VLEAKYRELU), ("addLeNetLayerMP", 64, 2, 1, 2, 2, synthetic.VLEAKYRELU),
             ("addLeNetLayerMP", 64, 2, 1, 1, 1, synthetic.VLEAKYRELU), ("addTerminalPoolingLayer", 2), ("addSoftmaxLayer",)]
    cfg = synthetic.Config("learn", 2, 1, 4, 16, 18, stack)
    cfg.number = 2
    net = hostapi.Net(2, 1, 4, nTop=1, threads=2)
    cfg.build(net)
    rng = np.random.default_rng(11)
    train = hostapi.Dataset("train", 1, 4, hostapi.TRAINBATCH)
    test = hostapi.Dataset("test", 1, 4, hostapi.TESTBATCH)
    for n in range(64):
        label = n % 4
        # four classes of pictures: a bar along one of two axes, a diagonal, or a block, at a random place
        o = rng.integers(0, 8, 2)
        if label == 0:
            pts = [(o[0] + i, o[1]) for i in range(8)]
        elif label == 1:
            pts = [(o[0], o[1] + i) for i in range(8)]
        elif label == 2:
            pts = [(o[0] + i, o[1] + i) for i in range(8)]
        else:
            pts = [(o[0] + i, o[1] + j) for i in range(3) for j in range(3)]
        pts = np.array(pts, np.int32)
        f = np.ones((len(pts), 1), np.float32)
        train.add_points(2, 18, pts, f, label)
        test.add_points(2, 18, pts, f, label)
    before = net.processDataset(test, 16)
    for epoch in range(30):
        net.processDatasetTrain(train, 16, learningRate=0.003, momentum=0.9)
    after = net.processDataset(test, 16)
    print("NLL before %.4f after %.4f" % (before, after), flush=True)
    assert after < 0.5 * before
    net.close()


def test_training_with_dropout(scn):
    """NiN layers with dropout: a training batch keeps a random subset of their output features (read back from the
    host library and handed to the oracle), the layers run on the sub-matrices of their weights, and only the entries
    used take the momentum step.  A PReLU layer without dropout of its own sits above dropped inputs."""
    from sparseconvnet_archived_amd import hostapi, synthetic
    stack = [("addLeNetLayerMP", 64, 2, 1, 3, 2, synthetic.VLEAKYRELU, 0.5),
             ("addLeNetLayerMP", 64, 2, 1, 2, 2, synthetic.RELU, 0.5),
             ("addLeNetLayerMP", 96, 2, 1, 1, 1, synthetic.PRELU, 0.0),
             ("addLeNetLayerMP", 64, 1, 1, 1, 1, synthetic.TANH, 0.5),
             ("addTerminalPoolingLayer", 2), ("addSoftmaxLayer",)]
    cfg = synthetic.Config("dropout", 2, 3, 10, 8, 14, stack)
    cfg.number = 2
    net, ora = pair(cfg, hostapi, 91)
    assert net.inputSpatialSize == ora.inputSpatialSize
    lattice = net.inputSpatialSize
    rng = np.random.default_rng(12)
    samples = []
    for _ in range(16):
        pts = np.array([(a, b) for a in range(lattice) for b in range(lattice) if rng.random() < 0.3], np.int32)
        samples.append((pts, rng.uniform(-1, 1, (len(pts), 3)).astype(np.float32), int(rng.integers(0, 10))))
    ds = hostapi.Dataset("dropout", 3, 10, hostapi.TRAINBATCH)
    for pts, f, label in samples:
        ds.add_points(2, lattice, pts, f, label)
    lr, mu = 0.01, 0.9
    net.set_training(lr, mu, shuffle=False)
    net.begin(ds, 8)
    layers = net.layers()
    before = {i: net.get_weights(i) for i, l in enumerate(layers) if l["kind"].startswith("nin")}
    drawn = []
    for b in range(2):
        assert net.next_batch()
        mine = samples[b * 8:(b + 1) * 8]
        present = {i: net.features_present(i + 1) for i, l in enumerate(layers) if l["kind"].startswith("nin")}
        drawn.append(present)
        kept = {i: len(p) for i, p in present.items()}
        print("batch", b, "features kept per NiN layer:", kept, flush=True)
        for i, p in present.items():
            assert np.all(np.diff(p) > 0) and p[0] >= 0 and p[-1] < layers[i]["nOut"]
        # (the builder rounds the kept features to a multiple of 32, SparseConvNetCUDA.cu:55-58)
        assert kept == {1: 32, 4: 32, 7: 96, 8: 32, 10: 10}
        S, K, R, bg, feats, n = synthetic.codify(mine, 2, lattice, lattice, 3)
        labels = np.array([s[2] for s in mine], np.int32)
        fwd = ora.forward(len(mine), S, K, R, bg, feats, n, labels, present=present)
        ora.train_step(fwd, labels, lr, mu)
        for i, wi in enumerate(fwd["interfaces"]):
            gi = net.interface(i)
            assert gi["features"].shape == wi["features"].shape
            assert rel_l2(gi["features"], wi["features"]) <= 1e-4
            if "dfeatures" in wi:
                assert rel_l2(net.dfeatures(i), wi["dfeatures"]) <= 1e-4
        for i in present:
            W, B, pr = net.get_weights(i)
            MW, MB, MP = net.get_weights(i, momentum=True)
            oW, oB, opr = ora.weights[i]
            assert rel_l2(MW, ora.momentum[i][0]) <= 1e-4 and rel_l2(MB, ora.momentum[i][1]) <= 1e-4
            assert np.allclose(W, oW, rtol=1e-4, atol=1e-6) and np.allclose(B, oB, rtol=1e-4, atol=1e-6)
    # weights that joined no kept pair in either batch have not moved at all
    i = 4
    W0 = before[i][0]
    W1 = net.get_weights(i)[0]
    used = np.zeros_like(W0, bool)
    for present in drawn:
        used[np.ix_(net_in_present(layers, present, i), present[i])] = True
    assert np.array_equal(W1[~used], W0[~used]) and (~used).any() and not np.array_equal(W1[used], W0[used])
    assert drawn[0][4].tolist() != drawn[1][4].tolist()  # a new draw for every batch
    net.close()


def net_in_present(layers, present, i):
    """features present at the input of NiN layer i: the kept outputs of the NiN below, replicated by the
    convolution in between (ConvolutionalLayer.cu:74-80); pooling layers pass them on"""
    below = [j for j in present if j < i]
    if not below:
        return np.arange(layers[i]["nIn"])
    p, nf = present[max(below)], layers[max(below)]["nOut"]
    conv = [l for l in layers[max(below) + 1:i] if l["kind"] == "conv"]
    if not conv:
        return p
    fs = conv[0]["nOut"] // conv[0]["nIn"]
    return np.concatenate([p + nf * q for q in range(fs)])


def test_rescale_batches(scn):
    """RESCALEBATCH passes (scaleWeights after every layer's forward pass): the weights after two passes against
    the oracle's, and the effect they are for: the mean magnitude of every hidden layer's output moves towards 1."""
    from sparseconvnet_archived_amd import hostapi, synthetic
    cfg = synthetic.config(2, batch=12)
    net, ora = pair(cfg, hostapi, 31)
    samples = synthetic.make_samples(cfg, 32)
    ds = hostapi.Dataset("rescale", cfg.nInputFeatures, cfg.nClasses, hostapi.RESCALEBATCH)
    for pts, f, label in samples:
        ds.add_points(cfg.dimension, cfg.lattice, pts, f, label)
    S, K, R, bg, feats, n = synthetic.codify(samples, cfg.dimension, cfg.lattice, net.inputSpatialSize, cfg.nInputFeatures)
    labels = np.array([s[2] for s in samples], np.int32)
    layers = net.layers()
    scales = []
    for rep in range(3):
        net.processDataset(ds, len(samples))
        fwd = ora.forward(len(samples), S, K, R, bg, feats, n, labels, rescale=True)
        scales.append([wi["featureScale"] for wi in fwd["interfaces"] if "featureScale" in wi])
        for i, l in enumerate(layers):
            if l["kind"].startswith("nin"):
                W, B, pr = net.get_weights(i)
                oW, oB, opr = ora.weights[i]
                assert np.allclose(W, oW, rtol=2e-4, atol=1e-7), (rep, i)
                assert np.allclose(B, oB, rtol=2e-4, atol=1e-7)
    first, last = np.array(scales[0][:-1]), np.array(scales[-1][:-1])
    print("feature scales of the hidden layers, first pass:", first, "third pass:", last, flush=True)
    assert np.all(np.abs(np.log(last)) <= np.abs(np.log(first)) + 1e-3)
    net.close()


def test_train_config4_wide_layers(scn):
    """The wide net (contractions of 640..3200 by 160..800): other kernels serve the backward products here."""
    from sparseconvnet_archived_amd import synthetic
    cfg = synthetic.config(4, batch=3)
    train_and_compare(scn, cfg, synthetic.make_samples(cfg, 304), 1)


def test_train_batch_of_one_and_empty_sample(scn):
    """Edge cases: a batch of one sample, then a batch whose second sample has no active site at all."""
    from sparseconvnet_archived_amd import synthetic
    cfg = synthetic.config(2, batch=1)
    train_and_compare(scn, cfg, synthetic.make_samples(cfg, 305), 1)
    cfg = synthetic.config(2, batch=3)
    samples = synthetic.make_samples(cfg, 306)
    pts, f, label = samples[1]
    samples[1] = (pts[:0], f[:0], label)
    train_and_compare(scn, cfg, samples, 1)
