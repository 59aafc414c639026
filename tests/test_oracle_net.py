"""Pins for the net-level oracle (oracle/oracle_net.py), CPU only.

* the dense-equivalence invariant: a sparse net equals the dense valid-convolution net on the full lattice in which
  every inactive site holds that depth's background vector (zero at the input, layer(background) after every layer),
  compared at the active sites and at the background row.  The dense side is plain numpy written here: it shares no
  code with the oracle, so the rule books, the gather, the NiN layers, max-pooling and the way forward() strings them
  together are all checked against an independent computation;
* builder arithmetic against numbers the reference itself holds or that are worked out by hand;
* central finite differences of a float64 loss through train_step() on a whole small net;
"""
import numpy as np
import pytest

import oracle as orc
import oracle_net

RELU, VLEAKY, LEAKY, PRELU, SOFTMAX = orc.RELU, orc.VLEAKYRELU, orc.LEAKYRELU, orc.PRELU, orc.SOFTMAX


# ---------------------------------------------------------------- dense equivalence
def dense_windows(F, n, d, size, stride):
    """F: [n^d, C] dense field, row-major sites.  Returns [nOut^d, size^d, C]: the window of every output site, offsets
    row-major (axis 0 slowest), and nOut."""
    nOut = (n - size) // stride + 1
    grid = F.reshape((n,) * d + (-1,))
    outs = []
    for o in np.ndindex(*(nOut,) * d):
        win = []
        for q in np.ndindex(*(size,) * d):
            win.append(grid[tuple(o[a] * stride + q[a] for a in range(d))])
        outs.append(win)
    return np.array(outs), nOut


def activation(z, act, prelu):
    if act == RELU:
        return np.where(z > 0, z, 0)
    if act == VLEAKY:
        return np.where(z > 0, z, z * np.float32(0.333))
    if act == LEAKY:
        return np.where(z > 0, z, z * np.float32(0.01))
    if act == PRELU:
        return np.where(z > 0, z, z * prelu)
    return z


def dense_forward(net, F, n):
    """The same layers on a dense field, in float64.  Yields (layer index, dense field, its side)."""
    d = net.dimension
    for i, l in enumerate(net.layers):
        k = l["kind"]
        if k == "conv":
            w, n = dense_windows(F, n, d, l["size"], l["stride"])
            F = w.reshape(w.shape[0], -1)  # column = offset * C + channel
        elif k == "maxpool":
            w, n = dense_windows(F, n, d, l["size"], l["stride"])
            F = w.max(1)
        elif k in ("nin", "nin_prelu"):
            W, B, pr = net.weights[i]
            p = 1.0 - l["dropout"]
            F = activation(p * (F @ W.astype(np.float64) + B.astype(np.float64)), l["act"],
                           None if pr is None else pr.astype(np.float64))
        else:
            raise AssertionError(k)
        yield i, F, n


DENSE_CASES = [
    # dimension, input channels, stack of (nFeatures, filterSize, filterStride, poolSize, poolStride, activation), top size
    (2, 3, [(32, 2, 1, 3, 2, RELU), (64, 2, 1, 3, 2, VLEAKY), (32, 1, 1, 1, 1, PRELU)], 2),
    (2, 2, [(32, 3, 1, 2, 2, LEAKY), (32, 3, 2, 1, 1, PRELU)], 2),
    (3, 1, [(32, 2, 1, 2, 2, RELU), (32, 2, 1, 2, 2, PRELU)], 1),
    (3, 2, [(32, 3, 1, 1, 1, VLEAKY), (32, 2, 2, 1, 1, RELU)], 2),
    (1, 4, [(32, 3, 1, 3, 3, RELU), (32, 2, 1, 2, 1, LEAKY)], 3),
]


@pytest.mark.parametrize("d,cin,stack,top", DENSE_CASES)
@pytest.mark.parametrize("density", [0.08, 0.5])
def test_sparse_net_equals_dense_valid_convolution_net(d, cin, stack, top, density):
    rng = np.random.default_rng(100 * d + cin + int(10 * density))
    net = oracle_net.Net(d, cin, 10)
    for f, fs, fstride, ps, pstride, act in stack:
        net.addLeNetLayerMP(f, fs, fstride, ps, pstride, act)
    n = net.finishHeadless(top)
    for i, l in enumerate(net.layers):
        if l["kind"] in ("nin", "nin_prelu"):
            W = (rng.standard_normal((l["nIn"], l["nOut"])) * np.sqrt(2.0 / l["nIn"])).astype(np.float32)
            B = (rng.standard_normal(l["nOut"]) * 0.3).astype(np.float32)  # a bias makes the background non-zero
            pr = rng.uniform(0.1, 0.4, l["nOut"]).astype(np.float32) if l["kind"] == "nin_prelu" else None
            net.set_weights(i, W, B, pr)
    batch, vol = 3, n ** d
    sample, key, row, bg, feats = [], [], [], [], []
    dense_in = []
    for b in range(batch):
        active = np.flatnonzero(rng.random(vol) < density)
        rng.shuffle(active)  # layer-0 rows are in insertion order, not key order
        F = np.zeros((vol, cin))
        bg.append(len(feats))
        feats.append(np.zeros(cin, np.float32))  # the background row of the input: zeros (Picture.h:10-11 contract)
        for k in active:
            v = rng.uniform(-1, 1, cin).astype(np.float32)
            sample.append(b)
            key.append(int(k))
            row.append(len(feats))
            feats.append(v)
            F[k] = v
        dense_in.append(F)
    feats = np.array(feats, np.float32)
    out = net.forward(batch, np.array(sample, np.int32), np.array(key, np.int64), np.array(row, np.int32),
                      np.array(bg, np.int32), feats, len(feats))
    checked = 0
    for b in range(batch):
        for i, F, side in dense_forward(net, dense_in[b], n):
            iface = out["interfaces"][i + 1]
            assert iface["spatialSize"] == side
            s, k, r, bgs = iface["grids"].flat()
            mine = s == b
            sparse = iface["features"].astype(np.float64)
            scale = np.abs(F).max() + 1e-9
            # active sites: the sparse row holds the dense value
            assert np.allclose(sparse[r[mine]], F[k[mine]], rtol=0, atol=2e-5 * scale)
            # every other site of the dense field holds one and the same vector, and it is the background row
            inactive = np.setdiff1d(np.arange(side ** d), k[mine])
            if inactive.size:
                assert bgs[b] >= 0
                assert np.allclose(F[inactive], F[inactive[0]], rtol=0, atol=1e-12 * scale + 1e-300)
                assert np.allclose(sparse[bgs[b]], F[inactive[0]], rtol=0, atol=2e-5 * scale)
            else:
                assert bgs[b] == -1
            checked += mine.sum()
    assert checked > 0


# ---------------------------------------------------------------- builder arithmetic
def test_deepc2_of_the_shrec_driver_has_a_126_field():
    """shrec2015.cpp:21 builds DeepC2(3, 5, 32, ...) and :15 renders its meshes at 40: NetworkArchitectures.cpp:13-21
    is l + 1 = 6 levels of C2, the first five followed by MP3/2; from size 1 at the top the sizes are
    1 <-C2- 2 <-MP3/2- 5 <-C2- 6 <- 13 <- 14 <- 29 <- 30 <- 61 <- 62 <- 125 <-C2- 126."""
    net = oracle_net.Net(3, 1, 50)
    l, k = 5, 32
    for i in range(l + 1):
        net.addLeNetLayerMP((i + 1) * k, 2, 1, 3 if i < l else 1, 2 if i < l else 1, VLEAKY, 0.0)
    net.addSoftmaxLayer()
    assert net.inputSpatialSize == 126
    sizes = [(x["kind"], x["inSize"], x["outSize"]) for x in net.layers if x["kind"] in ("conv", "maxpool")]
    assert sizes == [("conv", 126, 125), ("maxpool", 125, 62), ("conv", 62, 61), ("maxpool", 61, 30), ("conv", 30, 29),
                     ("maxpool", 29, 14), ("conv", 14, 13), ("maxpool", 13, 6), ("conv", 6, 5), ("maxpool", 5, 2),
                     ("conv", 2, 1)]
    # a 2^3 filter multiplies the features by 8 (SparseConvNetCUDA.cu:83-87); the classifier is not rounded
    nins = [(x["nIn"], x["nOut"]) for x in net.layers if x["kind"] == "nin"]
    assert nins == [(8, 32), (256, 64), (512, 96), (768, 128), (1024, 160), (1280, 192), (192, 50)]


def test_deepcnet_sizes_by_hand():
    """NetworkArchitectures.cpp:3-11, DeepCNet(2, 3, ...): C3 MP3/2, C2 MP3/2, C2 MP3/2, C2: 1 <- 2 <- 5 <- 6 <- 13 <- 14
    <- 29 <- 31."""
    net = oracle_net.Net(2, 1, 10)
    l = 3
    for i in range(l + 1):
        net.addLeNetLayerMP((i + 1) * 32, 3 if i == 0 else 2, 1, 3 if i < l else 1, 2 if i < l else 1, RELU, 0.0)
    net.addSoftmaxLayer()
    assert net.inputSpatialSize == 31


def test_learnt_layers_round_to_32_and_adjust_dropout():
    """SparseConvNetCUDA.cu:53-60, worked by hand: intRound(a, 32) = round(a / 32.0) * 32 (utilities.cu:103), at least
    32, except for the classifier; dropout becomes 1 - (intRound(n (1 - dropout), 32) + 0.01) / n, floored at 0."""
    net = oracle_net.Net(2, 1, 7)
    cases = [  # asked for -> built, dropout asked -> dropout kept
        (50, 64, 0.0, 0.0),  # 50 / 32 = 1.56 -> 2
        (40, 32, 0.0, 0.0),  # 1.25 -> 1
        (16, 32, 0.0, 0.0),  # 0.5 rounds to 1 (and 32 is the floor anyway)
        (5, 32, 0.0, 0.0),  # 0.16 -> 0, floored to 32
        (80, 96, 0.0, 0.0),  # 2.5 rounds away from zero -> 3
        (64, 64, 0.5, 1 - 32.01 / 64),  # 64 * 0.5 = 32 kept
        (96, 96, 0.3, 1 - 64.01 / 96),  # 96 * 0.7 = 67.2 -> int 67 -> 2.09 -> 64 kept
        (32, 32, 0.1, 0.0),  # 28.8 -> 28 -> 0.875 -> 32 kept: 1 - 32.01 / 32 < 0 -> 0
        (128, 128, 0.25, 1 - 96.01 / 128),
    ]
    for asked, built, drop_in, drop_out in cases:
        net.addLeNetLayerMP(asked, 1, 1, 1, 1, RELU, drop_in)
        l = net.layers[-1]
        assert l["nOut"] == built, (asked, l["nOut"])
        assert abs(l["dropout"] - drop_out) < 1e-6, (asked, drop_in, l["dropout"])
    net.addSoftmaxLayer()
    assert net.layers[-1]["nOut"] == 7 and net.layers[-1]["act"] == SOFTMAX
    # filterSize 1 adds no gather layer and poolSize 1 no pooling layer (SparseConvNetCUDA.cu:88-94, :106-110)
    assert all(x["kind"] == "nin" for x in net.layers)


def test_triangular_builder_passes_the_pool_size_as_min_active():
    """SparseConvNetCUDA.cu:165-168 against :183-185: the convolution's minActiveInputs is the pool size."""
    net = oracle_net.Net(2, 1, 5, triangular=True)
    net.addLeNetLayerMP(32, 3, 1, 3, 2, RELU, 0.0, minActiveInputs=1)
    net.addLeNetLayerMP(32, 2, 1, 1, 1, RELU, 0.0, minActiveInputs=7)
    convs = [x for x in net.layers if x["kind"] == "conv_tri"]
    assert [c["minActive"] for c in convs] == [3, 1]
    assert [c["fs"] for c in convs] == [6, 3]  # triangleSize(3, 2) = 6, triangleSize(2, 2) = 3 (utilities.cu:27-32)


# ---------------------------------------------------------------- finite differences through the whole net
def float64_loss(net, fwd, weights, labels):
    """The net's negative log-likelihood in float64 numpy, with the rule books of `fwd` held fixed."""
    ifaces = fwd["interfaces"]
    F = ifaces[0]["features"].astype(np.float64)
    for i, l in enumerate(net.layers):
        k, nxt = l["kind"], ifaces[i + 1]
        if k == "conv":
            F = F[nxt["rules"]].reshape(nxt["nSpatialSites"], -1)
        elif k == "maxpool":
            ps = nxt["rules"].size // nxt["nSpatialSites"]
            F = F[nxt["rules"].reshape(-1, ps)].max(1)
        elif k == "terminal":
            S = nxt["rules"].size // nxt["nSpatialSites"]
            rows = nxt["rules"].reshape(-1, S)
            F = np.stack([F[r[r >= 0]].mean(0) for r in rows])
        else:
            W, B, pr = weights[i]
            z = F @ W + B
            if l["act"] == SOFTMAX:
                z = z - z.max(1, keepdims=True)
                logp = z - np.log(np.exp(z).sum(1, keepdims=True))
                return -logp[np.arange(len(labels)), labels].sum()
            F = activation(z, l["act"], pr)
    raise AssertionError("no classifier")


def test_train_step_gradients_by_finite_differences_on_a_whole_net():
    rng = np.random.default_rng(12)
    net = oracle_net.Net(2, 2, 4)
    net.addLeNetLayerMP(32, 2, 1, 2, 2, VLEAKY)
    net.addLeNetLayerMP(32, 2, 1, 1, 1, PRELU)
    net.addTerminalPoolingLayer(2)
    net.addSoftmaxLayer()
    n = net.inputSpatialSize
    assert n == 7
    for i, l in enumerate(net.layers):
        if l["kind"] in ("nin", "nin_prelu"):
            net.set_weights(i, (rng.standard_normal((l["nIn"], l["nOut"])) * np.sqrt(2.0 / l["nIn"])).astype(np.float32),
                            (rng.standard_normal(l["nOut"]) * 0.2).astype(np.float32),
                            rng.uniform(0.15, 0.35, l["nOut"]).astype(np.float32) if l["kind"] == "nin_prelu" else None)
    batch = 3
    sample, key, row, bg, feats = [], [], [], [], []
    for b in range(batch):
        bg.append(len(feats))
        feats.append(np.zeros(2, np.float32))
        for k in np.flatnonzero(rng.random(n * n) < 0.4):
            sample.append(b)
            key.append(int(k))
            row.append(len(feats))
            feats.append(rng.uniform(-1, 1, 2).astype(np.float32))
    labels = np.array([1, 3, 0], np.int32)
    args = (batch, np.array(sample, np.int32), np.array(key, np.int64), np.array(row, np.int32), np.array(bg, np.int32),
            np.array(feats, np.float32), len(feats))
    before = {i: tuple(None if x is None else x.astype(np.float64) for x in w) for i, w in net.weights.items()}
    fwd = net.forward(*args, labels)
    assert np.isclose(fwd["nll"], float64_loss(net, fwd, before, labels), rtol=1e-5)
    lr = 0.05
    net.train_step(fwd, labels, lr, 0.0)  # no momentum: every parameter moves by -lr * gradient
    eps = 1e-5
    for i in before:
        names = ("W", "B", "PReLU")
        for which, name in enumerate(names):
            if before[i][which] is None:
                continue
            got = fwd["interfaces"][i + 1][{"W": "dW", "B": "dB", "PReLU": "dPReLU"}[name]].astype(np.float64)
            flat = before[i][which].reshape(-1)
            picks = rng.choice(flat.size, min(12, flat.size), replace=False)
            for j in picks:
                keep = flat[j]
                flat[j] = keep + eps
                up = float64_loss(net, fwd, before, labels)
                flat[j] = keep - eps
                down = float64_loss(net, fwd, before, labels)
                flat[j] = keep
                fd = (up - down) / (2 * eps)
                assert abs(got.reshape(-1)[j] - fd) <= 2e-3 * max(abs(fd), 1e-2), (i, name, j, got.reshape(-1)[j], fd)
            # ... and the step taken is -lr * gradient (slopes are kept above 0.001, not an issue at 0.15 and more)
            after = net.weights[i][which].astype(np.float64)
            assert np.allclose(after, before[i][which] - lr * got.reshape(before[i][which].shape), rtol=0, atol=2e-6)
