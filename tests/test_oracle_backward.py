"""Pins of the oracle's backward pass: adjoint identities for the rule-driven layers, central finite differences of a
float64 numpy loss for the soft-max gradient and the NiN layer (activation derivative, dW, dB, dA, PReLU slopes), and
algebraic identities for the weight update.  None of these repeats the oracle's own formulas."""
import numpy as np
import pytest

import oracle as orc

ACTS = {"none": 0, "relu": 1, "vleaky": 2, "leaky": 3, "tanh": 4, "prelu": 6, "sigmoid": 7}


def dot(a, b):
    return float(np.dot(a.astype(np.float64).ravel(), b.astype(np.float64).ravel()))


def test_gather_backward_is_the_adjoint_of_the_gather():
    rng = np.random.default_rng(1)
    for nIn, rowsIn, count in [(1, 5, 40), (3, 17, 200), (32, 50, 333), (70, 9, 64)]:
        rules = rng.integers(0, rowsIn, count).astype(np.int32)
        rules[rng.random(count) < 0.5] = 0  # a background row named over and over
        x = rng.standard_normal((rowsIn, nIn)).astype(np.float32)
        y = rng.standard_normal((count, nIn)).astype(np.float32)
        Gx = orc.gather_rows(x, rules, nIn)
        Gty = orc.gather_rows_backward(y, rules, rowsIn, nIn)
        assert dot(Gx, y) == pytest.approx(dot(x, Gty), rel=1e-5, abs=1e-4)
    # a row nobody names receives nothing; a single rule copies
    g = orc.gather_rows_backward(np.array([[2.0, 3.0]], np.float32), np.array([1], np.int32), 3, 2)
    assert g.tolist() == [[0, 0], [2, 3], [0, 0]]


def test_maxpool_backward_is_the_adjoint_of_the_selection():
    rng = np.random.default_rng(2)
    for C, rowsIn, nOut, ps in [(1, 6, 10, 4), (5, 20, 33, 9), (64, 30, 41, 8)]:
        rules = rng.integers(0, rowsIn, (nOut, ps)).astype(np.int32)
        rules[rng.random((nOut, ps)) < 0.4] = 0
        x = rng.standard_normal((rowsIn, C)).astype(np.float32)
        out, choice = orc.maxpool(x, rules, nOut, ps, C)
        assert np.array_equal(out.ravel(), x.ravel()[choice.ravel()])  # the forward is a selection by `choice`
        y = rng.standard_normal((nOut, C)).astype(np.float32)
        Pty = orc.maxpool_backward(y, choice, rowsIn)
        assert dot(out, y) == pytest.approx(dot(x, Pty), rel=1e-5, abs=1e-4)


def test_terminal_backward_is_the_adjoint_of_the_mean():
    rng = np.random.default_rng(3)
    C, S = 7, 6
    # three samples with 6, 2 and 1 (background only) rows; each row listed once
    rules = np.array([[0, 1, 2, 3, 4, 5], [6, 7, -1, -1, -1, -1], [8, -1, -1, -1, -1, -1]], np.int32)
    x = rng.standard_normal((9, C)).astype(np.float32)
    y = rng.standard_normal((3, C)).astype(np.float32)
    Tx = orc.terminal_pool(x, rules, 3, S, C)
    Tty = orc.terminal_pool_backward(y, rules, S, 9)
    assert dot(Tx, y) == pytest.approx(dot(x, Tty), rel=1e-5)
    assert np.allclose(Tty[6], y[1] / 2) and np.allclose(Tty[8], y[2])


def test_softmax_gradient_vs_finite_differences():
    rng = np.random.default_rng(4)
    z = rng.standard_normal((5, 11))
    labels = rng.integers(0, 11, 5).astype(np.int32)

    def nll(z):
        e = np.exp(z - z.max(1, keepdims=True))
        p = e / e.sum(1, keepdims=True)
        return -np.log(p[np.arange(len(z)), labels]).sum()

    probs = orc.softmax_rows(z.astype(np.float32))
    g = orc.softmax_grad(probs, labels)
    eps = 1e-5
    for k in range(5):
        for i in range(11):
            zp, zm = z.copy(), z.copy()
            zp[k, i] += eps
            zm[k, i] -= eps
            assert g[k, i] == pytest.approx((nll(zp) - nll(zm)) / (2 * eps), abs=2e-5)


def act64(z, act, slopes):
    if act == 0:
        return z
    if act == 1:
        return np.maximum(z, 0)
    if act == 2:
        return np.where(z > 0, z, z * np.float32(0.333))
    if act == 3:
        return np.where(z > 0, z, z * np.float32(0.01))
    if act == 4:
        return np.tanh(z)
    if act == 6:
        return np.where(z > 0, z, z * slopes)
    return 1 / (1 + np.exp(-z))


@pytest.mark.parametrize("name", sorted(ACTS))
def test_nin_backward_vs_finite_differences(name):
    act = ACTS[name]
    rng = np.random.default_rng(10 + act)
    M, K, N = 23, 9, 6
    A = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) * 0.5).astype(np.float32)
    B = (rng.standard_normal(N) * 0.3).astype(np.float32)
    pr = rng.uniform(0.1, 0.6, N).astype(np.float32) if act == 6 else None
    G = rng.standard_normal((M, N))  # loss = sum(G * layer(A))

    def loss(A_, W_, B_, pr_):
        z = A_.astype(np.float64) @ W_.astype(np.float64) + B_
        return float((G * act64(z, act, pr_)).sum())

    # stay away from the kink of the piecewise-linear activations
    z0 = A.astype(np.float64) @ W.astype(np.float64) + B
    assert np.abs(z0).min() > 1e-3
    out = orc.nin_forward(A, W, B, pr, 1.0, act)
    dZ, dB, dPr = orc.activation_backward(out, G.astype(np.float32), act, pr)
    dW = orc.sgemm_AtB(A, dZ)
    dA = orc.sgemm_ABt(dZ, W)
    eps = 1e-4

    def fd(which, idx):
        args = [A.astype(np.float64), W.astype(np.float64), B.astype(np.float64),
                pr.astype(np.float64) if pr is not None else None]
        p, m = [a.copy() if a is not None else None for a in args], [a.copy() if a is not None else None for a in args]
        p[which][idx] += eps
        m[which][idx] -= eps
        return (loss(*p) - loss(*m)) / (2 * eps)

    tol = dict(rel=2e-3, abs=2e-3)
    for _ in range(12):
        k, n, m = int(rng.integers(K)), int(rng.integers(N)), int(rng.integers(M))
        assert dW[k, n] == pytest.approx(fd(1, (k, n)), **tol)
        assert dA[m, k] == pytest.approx(fd(0, (m, k)), **tol)
        assert dB[n] == pytest.approx(fd(2, (n,)), **tol)
        if act == 6:
            assert dPr[n] == pytest.approx(fd(3, (n,)), **tol)


def test_weight_update_identities():
    rng = np.random.default_rng(5)
    n = 50
    d = rng.standard_normal(n).astype(np.float32)
    w0 = rng.standard_normal(n).astype(np.float32)
    m0 = (rng.standard_normal(n) * 0.1).astype(np.float32)
    # momentum 0: plain gradient descent, the old momentum plays no part
    w, m = w0.copy(), m0.copy()
    orc.nag_update(d, m, w, 0.1, 0.0)
    assert np.allclose(w, w0 - np.float32(0.1) * d, rtol=1e-6, atol=1e-7)
    assert np.allclose(m, -np.float32(0.1) * d, rtol=1e-6)
    # in general: m' = mu m - lr (1 - mu) d and w' = w + m' + mu (m' - m)
    w, m = w0.copy(), m0.copy()
    orc.nag_update(d, m, w, 0.03, 0.9)
    m1 = 0.9 * m0.astype(np.float64) - 0.03 * (1 - 0.9) * d
    assert np.allclose(m, m1, rtol=1e-5, atol=1e-7)
    assert np.allclose(w, w0 + m1 + 0.9 * (m1 - m0), rtol=1e-5, atol=1e-6)
    # keepPositive clamps at 0.001 (PReLU slopes)
    w, m = np.array([0.002, 0.5], np.float32), np.zeros(2, np.float32)
    orc.nag_update(np.array([1.0, 1.0], np.float32), m, w, 0.1, 0.0, keepPositive=True)
    assert w[0] == np.float32(0.001) and w[1] == pytest.approx(0.4)
