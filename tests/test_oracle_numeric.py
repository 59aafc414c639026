"""Pins for the oracle's numeric layers (CPU only): closed forms, brute force,
special cases that reduce to a library routine."""
import numpy as np
import pytest

import oracle as orc


def test_gather_is_exact_row_copy():
    rng = np.random.default_rng(0)
    inp = rng.standard_normal((37, 5)).astype(np.float32)
    rules = rng.integers(0, 37, size=200).astype(np.int32)
    out = orc.gather_rows(inp, rules, 5)
    assert np.array_equal(out, inp[rules])
    # viewed as the im2col matrix [nOut x fs*C]: column k*C + c holds window offset k
    fs = 4
    m = out.reshape(-1, fs * 5)
    for r in range(m.shape[0]):
        for k in range(fs):
            assert np.array_equal(m[r, k * 5:(k + 1) * 5], inp[rules[r * fs + k]])


@pytest.mark.parametrize("act", [orc.NOSIGMOID, orc.RELU, orc.LEAKYRELU, orc.VLEAKYRELU, orc.PRELU])
@pytest.mark.parametrize("p", [1.0, 0.75])
def test_nin_against_float64_gemm(act, p):
    rng = np.random.default_rng(act * 10 + int(p * 4))
    M, K, N = 53, 37, 32
    A = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    B = rng.standard_normal(N).astype(np.float32)
    pr = rng.uniform(0.1, 0.4, N).astype(np.float32)
    z = p * (A.astype(np.float64) @ W.astype(np.float64) + B.astype(np.float64))
    slope = {orc.NOSIGMOID: None, orc.RELU: 0.0, orc.LEAKYRELU: np.float32(0.01),
             orc.VLEAKYRELU: np.float32(0.333), orc.PRELU: pr.astype(np.float64)}[act]
    want = z if slope is None else np.where(z > 0, z, z * slope)
    got = orc.nin_forward(A, W, B, pr, p, act)
    got64 = orc.nin_forward(A, W, B, pr, p, act, f64=True)
    assert np.allclose(got64, want, rtol=1e-12, atol=1e-12)
    scale = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
    assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-6)


def test_nin_special_cases():
    rng = np.random.default_rng(5)
    M, K = 9, 32
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal(K).astype(np.float32)
    # W = I: output is A + B exactly
    out = orc.nin_forward(A, np.eye(K, dtype=np.float32), B, None, 1.0, orc.NOSIGMOID)
    assert np.array_equal(out, A + B)
    # W = 0: every row is act(p * B)
    out = orc.nin_forward(A, np.zeros((K, K), np.float32), B, None, 0.5, orc.RELU)
    assert np.array_equal(out, np.tile(np.maximum(np.float32(0.5) * B, 0), (M, 1)))
    # a single non-zero weight moves one input column to one output column
    W = np.zeros((K, K), np.float32)
    W[3, 7] = 2.0
    out = orc.nin_forward(A, W, np.zeros(K, np.float32), None, 1.0, orc.NOSIGMOID)
    want = np.zeros((M, K), np.float32)
    want[:, 7] = 2.0 * A[:, 3]
    assert np.array_equal(out, want)
    # W is [K x N] row-major: W[k, n] multiplies input column k (not transposed)
    W = rng.standard_normal((K, 64)).astype(np.float32)
    out = orc.nin_forward(A[:, :K], W, np.zeros(64, np.float32), None, 1.0, orc.NOSIGMOID)
    assert np.allclose(out, A @ W, rtol=1e-4, atol=1e-4)


def test_softmax_closed_form():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((11, 10)) * 5).astype(np.float32)
    y = orc.softmax_rows(x)
    e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    assert np.allclose(y, e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-7)
    assert np.allclose(y.sum(1), 1, atol=1e-5)
    assert np.array_equal(y.argmax(1), x.argmax(1))
    # the running maximum starts at -10000: rows entirely below it are shifted by -10000
    lo = np.full((1, 3), -10050.0, np.float32)
    lo[0, 1] = -10040.0
    y = orc.softmax_rows(lo)
    e = np.exp(lo.astype(np.float64) + 10000.0)
    assert np.allclose(y, e / e.sum(), rtol=1e-4)
    # softmax through the NiN head
    A = rng.standard_normal((4, 8)).astype(np.float32)
    W = rng.standard_normal((8, 5)).astype(np.float32)
    B = rng.standard_normal(5).astype(np.float32)
    z = orc.nin_forward(A, W, B, None, 1.0, orc.NOSIGMOID)
    assert np.array_equal(orc.nin_forward(A, W, B, None, 1.0, orc.SOFTMAX), orc.softmax_rows(z))


def test_maxpool_brute_force_ties_and_negative_rules():
    rng = np.random.default_rng(9)
    nIn, Cn, ps, nOut = 40, 6, 5, 30
    inp = rng.integers(-3, 4, size=(nIn, Cn)).astype(np.float32)  # many ties
    rules = rng.integers(-1, nIn, size=(nOut, ps)).astype(np.int32)
    rules[:, 0] = np.abs(rules[:, 0])  # at least one valid entry per row
    rules[3] = [-1, -1, 7, 7, -1]
    out, choice = orc.maxpool(inp, rules, nOut, ps, Cn)
    for r in range(nOut):
        for c in range(Cn):
            best, arg = None, None
            for p in range(ps):
                if rules[r, p] < 0:
                    continue
                v = inp[rules[r, p], c]
                if best is None or v > best:  # strict: the first maximum wins
                    best, arg = v, rules[r, p] * Cn + c
            assert out[r, c] == best and choice[r, c] == arg
    assert np.array_equal(inp.reshape(-1)[choice], out)


def test_terminal_pool_is_mean_over_listed_rows():
    rng = np.random.default_rng(4)
    inp = rng.standard_normal((20, 32)).astype(np.float32)
    S = 6
    rules = np.full((3, S), -1, np.int32)
    rules[0, :4] = [3, 1, 19, 7]
    rules[1, :6] = [0, 2, 4, 6, 8, 10]
    rules[2, :1] = [5]
    out = orc.terminal_pool(inp, rules, 3, S, 32)
    for b in range(3):
        rows = [r for r in rules[b] if r >= 0]
        want = inp[rows].astype(np.float64).mean(0)
        assert np.allclose(out[b], want, rtol=1e-5, atol=1e-6)
        seq = np.zeros(32, np.float32)
        for r in rows:
            seq = seq + inp[r]
        assert np.array_equal(out[b], seq / np.float32(len(rows)))


def test_top_indices_and_classifier():
    rng = np.random.default_rng(6)
    for n in (1, 2, 5, 17):
        for k in range(1, min(n, 4) + 1):
            v = rng.integers(0, 4, n).astype(np.float32)  # ties
            got = orc.top_indices(v, k)
            want = sorted(range(n), key=lambda i: (-v[i], i))[:k]  # ties keep the lower index
            assert got.tolist() == want
    probs = np.array([[0.1, 0.7, 0.2], [0.5, 0.25, 0.25], [0.0, 0.0, 1.0]], np.float32)
    labels = np.array([1, 2, 0], np.int32)
    pred, mistakes, nll = orc.softmax_classifier(probs, labels, 1)
    assert pred[:, 0].tolist() == [1, 0, 2] and mistakes == 2
    assert np.isclose(nll, -(np.log(0.7) + np.log(0.25) + np.log(1e-15)), rtol=1e-5)
    pred, mistakes, _ = orc.softmax_classifier(probs, labels, 2)
    assert pred.tolist() == [[1, 2], [0, 1], [2, 0]] and mistakes == 1
