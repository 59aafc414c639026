"""Helpers shared by the GPU parity tests."""
import numpy as np

import oracle as orc


def flatten_samples(samples):
    """list of (bg, {key: row}) -> sample[], key[], row[], bg[] in insertion order."""
    s, k, r, bg = [], [], [], []
    for i, (b, mp) in enumerate(samples):
        bg.append(b)
        for kk, rr in mp.items():
            s.append(i)
            k.append(kk)
            r.append(rr)
    return (np.array(s, np.int32), np.array(k, np.int64), np.array(r, np.int32), np.array(bg, np.int32))


def oracle_grids(samples):
    g = orc.Grids(len(samples))
    for i, (bg, mp) in enumerate(samples):
        g.set(i, list(mp.keys()), list(mp.values()), bg)
    return g


def device_grids(scn, ctx, samples, d, n, nSites):
    s, k, r, bg = flatten_samples(samples)
    g = scn.Grids(ctx)
    g.build(len(samples), d, n, s, k, r, bg, nSites)
    return g


def assert_same_grids(dev, ora):
    s, k, r, bg = dev.download()
    os_, ok, or_, obg = ora.flat()
    assert np.array_equal(bg, obg)
    assert np.array_equal(s, os_)
    assert np.array_equal(k, ok)
    assert np.array_equal(r, or_)


# fp32 activations: within 1e-4, relative (the bar of the forward path), measured per element against a float64
# evaluation and scaled by the row the element sits in
FP32_TOL = 1e-4


def assert_probabilities(got, want64, tol=FP32_TOL):
    """Class probabilities of a batch against the float64 evaluation of the same net on the same rule books
    (oracle_net.Net.forward64): every element within `tol` of its row's scale, the row's largest probability.
    Returns the worst ratio found."""
    got = np.asarray(got, np.float64)
    want64 = np.asarray(want64, np.float64)
    assert got.shape == want64.shape
    scale = np.abs(want64).max(1, keepdims=True)
    worst = float((np.abs(got - want64) / scale).max()) if got.size else 0.0
    assert worst <= tol, "probabilities off by %.3g of the row's scale (bar %.1g)" % (worst, tol)
    return worst


def assert_nll(got, probs64, labels, tol=FP32_TOL):
    """SoftmaxClassifier's negative log-likelihood (SoftmaxClassifier.cu:39-43: minus the sum of log p[label]) against
    float64.  d(-log p) = dp / p, and dp is bounded by tol times the row's largest probability, so each sample may be
    off by tol * max(row) / p[label]; the sum by the sum of those, plus fp32 rounding of the sum itself."""
    p = np.asarray(probs64, np.float64)
    labels = np.asarray(labels)
    pl = p[np.arange(len(labels)), labels]
    want = -np.log(pl).sum()
    slack = (tol * p.max(1) / pl).sum() + 1e-6 * max(abs(want), 1.0)
    assert abs(float(got) - want) <= slack, "nll %.8g, float64 %.8g, allowed %.3g" % (got, want, slack)
