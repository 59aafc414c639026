"""The backward pass and the weight update through the C ABI against the oracle.
Sums that the reference itself leaves to float atomics in no fixed order are held to 1e-4 of the sum of magnitudes;
assignments and element-wise results are bit-exact."""
import numpy as np
import pytest

import oracle as orc

pytestmark = pytest.mark.gpu


def close(got, want, scale, tol=1e-4):
    got, want = got.astype(np.float64), want.astype(np.float64)
    bad = np.abs(got - want) > tol * scale + 1e-30
    assert not bad.any(), (np.abs(got - want).max(), np.argwhere(bad)[:5])


def test_softmax_gradient_bit_exact(scn, ctx):
    rng = np.random.default_rng(0)
    for B, N in [(1, 1), (7, 10), (100, 100), (33, 1000)]:
        probs = orc.softmax_rows(rng.standard_normal((B, N)).astype(np.float32))
        labels = rng.integers(0, N, B).astype(np.int32)
        d = ctx.empty((B, N), np.float32)
        ctx.softmax_grad(ctx.array(probs), ctx.array(labels), d, B, N)
        assert np.array_equal(d.download(), orc.softmax_grad(probs, labels))


@pytest.mark.parametrize("act", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("M,N", [(1, 32), (77, 100), (5000, 64), (2049, 800), (300, 3)])
def test_activation_backward(scn, ctx, act, M, N):
    rng = np.random.default_rng(act * 1000 + M + N)
    print("activation backward act=%d M=%d N=%d" % (act, M, N), flush=True)
    out = rng.standard_normal((M, N)).astype(np.float32)
    if act in (1,):
        out = np.maximum(out, 0)
    delta = rng.standard_normal((M, N)).astype(np.float32)
    pr = rng.uniform(0.05, 0.5, N).astype(np.float32) if act == 6 else None
    d_delta = ctx.array(delta)
    d_db = ctx.array(np.full(N, 7, np.float32))  # must be overwritten, not added to
    d_dpr = ctx.array(np.full(N, 7, np.float32)) if act == 6 else None
    ctx.activation_backward(ctx.array(out), d_delta, M, N, act, ctx.array(pr) if pr is not None else None, d_db, d_dpr)
    wd, wdb, wdpr = orc.activation_backward(out, delta, act, pr)
    assert np.array_equal(d_delta.download(), wd)
    close(d_db.download(), wdb, np.abs(wd).sum(0))
    if act == 6:
        close(d_dpr.download(), wdpr, (np.abs(delta) * np.abs(out) / pr).sum(0))


@pytest.mark.parametrize("M,K,N", [(1, 1, 1), (50, 12, 32), (1000, 128, 64), (4097, 288, 64), (333, 100, 100),
                                   (20000, 256, 96), (2500, 800, 800), (100, 192, 100), (70000, 1728, 64),
                                   (5000, 64, 48), (3000, 132, 52), (1024, 260, 132), (9999, 1280, 480)])
def test_weight_gradient_AtB(scn, ctx, M, K, N):
    rng = np.random.default_rng(M + K + N)
    print("AtB M=%d K=%d N=%d" % (M, K, N), flush=True)
    A = rng.standard_normal((M, K)).astype(np.float32)
    D = rng.standard_normal((M, N)).astype(np.float32)
    d_dW = ctx.array(np.full((K, N), 3, np.float32))
    ctx.sgemm_AtB(ctx.array(A), ctx.array(D), d_dW, M, K, N)
    orc.set_threads(8)
    want = orc.sgemm_AtB(A, D)
    scale = np.sqrt((A.astype(np.float64) ** 2).sum(0))[:, None] * np.sqrt((D.astype(np.float64) ** 2).sum(0))[None, :]
    close(d_dW.download(), want, scale + 1e-6)
    # a one-hot D picks out rows of A exactly
    if M >= 2 and N >= 2:
        D[:] = 0
        D[M // 2, 1] = 1
        ctx.sgemm_AtB(ctx.array(A), ctx.array(D), d_dW, M, K, N)
        got = d_dW.download()
        assert np.array_equal(got[:, 1], A[M // 2]) and not got[:, 0].any()


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (50, 32, 12), (1000, 64, 128), (4097, 64, 288), (333, 100, 192),
                                   (20000, 96, 256), (2500, 800, 800), (100, 100, 192)])
def test_input_gradient_ABt(scn, ctx, M, N, K):
    rng = np.random.default_rng(M + K + N + 1)
    print("ABt M=%d N=%d K=%d" % (M, N, K), flush=True)
    D = rng.standard_normal((M, N)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    d_dA = ctx.empty((M, K), np.float32)
    ws = ctx.empty(scn.lib().scn_sgemm_ABt_workspace(N, K), np.float32)
    ctx.sgemm_ABt(ctx.array(D), ctx.array(W), d_dA, M, N, K, ws)
    orc.set_threads(8)
    want = orc.sgemm_ABt(D, W)
    scale = np.abs(D).astype(np.float64) @ np.abs(W).astype(np.float64).T
    close(d_dA.download(), want, scale + 1e-6)


def test_weight_update(scn, ctx):
    rng = np.random.default_rng(3)
    for n in (1, 100, 12345, 800 * 800):
        for keep in (False, True):
            d = rng.standard_normal(n).astype(np.float32)
            w = rng.standard_normal(n).astype(np.float32)
            m = (rng.standard_normal(n) * 0.1).astype(np.float32)
            d_w, d_m = ctx.array(w), ctx.array(m)
            ctx.nag_update(ctx.array(d), d_m, d_w, n, 0.003, 0.99, keep)
            orc.nag_update(d, m, w, 0.003, 0.99, keep)
            # (a fused multiply-add more or less than the host compiler chose: a few ulp of the terms)
            assert np.allclose(d_w.download(), w, rtol=1e-6, atol=1e-7)
            assert np.allclose(d_m.download(), m, rtol=1e-6, atol=1e-8)


def test_weight_update_of_several_tensors_in_one_launch(scn, ctx):
    """scn_nag_update_many = scn_nag_update on each tensor (bit for bit: the same arithmetic), gradients left zero
    when asked; sizes chosen so that tensors end inside, at the end of and one past a workgroup of 256."""
    rng = np.random.default_rng(4)
    for sizes, clear in [((100,), True), ((96, 256 * 96, 96), True), ((257, 1, 256, 511), False),
                         ((0, 800 * 800, 800), True), ((5, 0, 7), False), ((), True)]:
        print("nag_update_many sizes", sizes, flush=True)
        items, single = [], []
        for k, n in enumerate(sizes):
            d = rng.standard_normal(n).astype(np.float32)
            w = rng.standard_normal(n).astype(np.float32)
            m = (rng.standard_normal(n) * 0.1).astype(np.float32)
            keep = k == 0
            d_d, d_m, d_w = ctx.array(d), ctx.array(m), ctx.array(w)
            items.append((d_d, d_m, d_w, n, keep))
            s_m, s_w = ctx.array(m), ctx.array(w)
            if n:
                ctx.nag_update(ctx.array(d), s_m, s_w, n, 0.003, 0.99, keep)
            single.append((d, s_m, s_w))
        ctx.nag_update_many(items, 0.003, 0.99, clear)
        for (d_d, d_m, d_w, n, keep), (d, s_m, s_w) in zip(items, single):
            if n == 0:
                continue
            assert np.array_equal(d_w.download(), s_w.download())
            assert np.array_equal(d_m.download(), s_m.download())
            assert np.array_equal(d_d.download(), np.zeros(n, np.float32) if clear else d)
    with pytest.raises(scn.ScnError):
        z = ctx.array(np.zeros(4, np.float32))
        ctx.nag_update_many([(z, z, z, 4, False)] * (scn.NAG_MAX + 1), 0.1, 0.9)


def test_accumulating_products_add_to_what_is_there(scn, ctx):
    """The beta = 1 variants: on zeroed buffers they are the plain entry points, on others they add."""
    rng = np.random.default_rng(5)
    for M, K, N in [(50, 12, 32), (4097, 288, 64), (70000, 256, 96), (0, 8, 8)]:
        print("accumulating products M=%d K=%d N=%d" % (M, K, N), flush=True)
        A = rng.standard_normal((M, K)).astype(np.float32)
        D = rng.standard_normal((M, N)).astype(np.float32)
        base = rng.standard_normal((K, N)).astype(np.float32)
        plain, acc = ctx.empty((K, N), np.float32), ctx.array(base)
        ctx.sgemm_AtB(ctx.array(A), ctx.array(D), plain, M, K, N)
        ctx.sgemm_AtB(ctx.array(A), ctx.array(D), acc, M, K, N, accumulate=True)
        scale = np.sqrt((A.astype(np.float64) ** 2).sum(0))[:, None] * np.sqrt((D.astype(np.float64) ** 2).sum(0))[None]
        close(acc.download(), base.astype(np.float64) + plain.download(), scale + np.abs(base) + 1e-6)
        for act in (1, 6):
            out = rng.standard_normal((M, N)).astype(np.float32)
            pr = ctx.array(rng.uniform(0.05, 0.5, N).astype(np.float32)) if act == 6 else None
            b0 = rng.standard_normal(N).astype(np.float32)
            p_d, a_d = ctx.array(D), ctx.array(D)
            p_db, a_db = ctx.empty(N, np.float32), ctx.array(b0)
            p_dp, a_dp = (ctx.empty(N, np.float32), ctx.array(b0)) if act == 6 else (None, None)
            ctx.activation_backward(ctx.array(out), p_d, M, N, act, pr, p_db, p_dp)
            ctx.activation_backward(ctx.array(out), a_d, M, N, act, pr, a_db, a_dp, accumulate=True)
            assert np.array_equal(p_d.download(), a_d.download())
            mag = np.abs(p_d.download()).sum(0) + np.abs(b0)
            close(a_db.download(), b0.astype(np.float64) + p_db.download(), mag + 1e-6)
            if act == 6:
                close(a_dp.download(), b0.astype(np.float64) + p_dp.download(),
                      (np.abs(D) * np.abs(out)).sum(0) / 0.05 + np.abs(b0) + 1e-6)


@pytest.mark.parametrize("nIn,rowsIn,count", [(1, 5, 40), (3, 1000, 33333), (32, 5000, 100001), (64, 2000, 54321),
                                              (96, 300, 9999), (160, 77, 4096), (5, 10, 31)])
def test_convolution_backward_scatter(scn, ctx, nIn, rowsIn, count):
    rng = np.random.default_rng(nIn + rowsIn + count)
    print("scatter nIn=%d rows=%d count=%d" % (nIn, rowsIn, count), flush=True)
    rules = rng.integers(0, rowsIn, count).astype(np.int32)
    rules[rng.random(count) < 0.6] = rowsIn // 2  # the background row of a sparse rule book
    rules[rng.random(count) < 0.01] = -1
    dconv = rng.standard_normal((count, nIn)).astype(np.float32)
    d_din = ctx.array(np.zeros((rowsIn, nIn), np.float32))
    ctx.gather_rows_backward(d_din, ctx.array(dconv), ctx.array(rules), count, nIn)
    want = orc.gather_rows_backward(dconv, rules, rowsIn, nIn)
    mag = orc.gather_rows_backward(np.abs(dconv), rules, rowsIn, nIn)
    close(d_din.download(), want, mag)
    # integers add exactly in any order
    dconv = rng.integers(-3, 4, (count, nIn)).astype(np.float32)
    d_din = ctx.array(np.zeros((rowsIn, nIn), np.float32))
    ctx.gather_rows_backward(d_din, ctx.array(dconv), ctx.array(rules), count, nIn)
    assert np.array_equal(d_din.download(), orc.gather_rows_backward(dconv, rules, rowsIn, nIn))


@pytest.mark.parametrize("C,rowsIn,nOut,ps", [(1, 6, 10, 4), (32, 3000, 7777, 9), (64, 500, 2001, 8), (96, 100, 333, 27),
                                              (5, 20, 65, 4)])
def test_maxpool_backward(scn, ctx, C, rowsIn, nOut, ps):
    rng = np.random.default_rng(C + rowsIn + nOut)
    print("maxpool backward C=%d" % C, flush=True)
    rules = rng.integers(0, rowsIn, (nOut, ps)).astype(np.int32)
    rules[rng.random((nOut, ps)) < 0.5] = 0
    x = rng.standard_normal((rowsIn, C)).astype(np.float32)
    _, choice = orc.maxpool(x, rules, nOut, ps, C)
    dout = rng.integers(-3, 4, (nOut, C)).astype(np.float32)  # integers: exact in any order
    d_din = ctx.array(np.zeros((rowsIn, C), np.float32))
    ctx.maxpool_backward(d_din, ctx.array(dout), nOut, C, ctx.array(choice))
    assert np.array_equal(d_din.download(), orc.maxpool_backward(dout, choice, rowsIn))
    dout = rng.standard_normal((nOut, C)).astype(np.float32)
    d_din = ctx.array(np.zeros((rowsIn, C), np.float32))
    ctx.maxpool_backward(d_din, ctx.array(dout), nOut, C, ctx.array(choice))
    close(d_din.download(), orc.maxpool_backward(dout, choice, rowsIn), orc.maxpool_backward(np.abs(dout), choice, rowsIn))


def test_terminal_pool_backward_bit_exact(scn, ctx):
    rng = np.random.default_rng(9)
    for C in (3, 100, 192, 800):
        B, S, rows = 37, 9, 400
        rules = np.full((B, S), -1, np.int32)
        perm = rng.permutation(rows)
        at = 0
        for b in range(B):
            n = 1 + b % S
            rules[b, :n] = perm[at:at + n]
            at += n
        dout = rng.standard_normal((B, C)).astype(np.float32)
        d_din = ctx.array(np.zeros((rows, C), np.float32))
        ctx.terminal_pool_backward(d_din, ctx.array(dout), ctx.array(rules), B, C, S)
        assert np.array_equal(d_din.download(), orc.terminal_pool_backward(dout, rules, S, rows))


def test_dropout_sub_matrix_and_its_update(scn, ctx):
    """scn_shrink_matrix picks W[inPresent][outPresent]; scn_nag_update_shrunk moves exactly those entries."""
    rng = np.random.default_rng(21)
    for K, N, Kp, Np in [(12, 32, 12, 16), (256, 64, 128, 32), (100, 100, 37, 100), (1, 800, 1, 123)]:
        W = rng.standard_normal((K, N)).astype(np.float32)
        M = (rng.standard_normal((K, N)) * 0.1).astype(np.float32)
        inP = np.sort(rng.choice(K, Kp, replace=False)).astype(np.int32)
        outP = np.sort(rng.choice(N, Np, replace=False)).astype(np.int32)
        d_w = ctx.empty((Kp, Np), np.float32)
        d_W, d_M = ctx.array(W), ctx.array(M)
        ctx.shrink_matrix(d_W, d_w, ctx.array(inP), ctx.array(outP), N, Kp, Np)
        assert np.array_equal(d_w.download(), W[np.ix_(inP, outP)])
        delta = rng.standard_normal((Kp, Np)).astype(np.float32)
        ctx.nag_update_shrunk(ctx.array(delta), d_M, d_W, ctx.array(inP), ctx.array(outP), N, Kp, Np, 0.01, 0.9)
        subW, subM = np.ascontiguousarray(W[np.ix_(inP, outP)]), np.ascontiguousarray(M[np.ix_(inP, outP)])
        orc.nag_update(delta, subM, subW, 0.01, 0.9)
        wantW, wantM = W.copy(), M.copy()
        wantW[np.ix_(inP, outP)], wantM[np.ix_(inP, outP)] = subW, subM
        gotW, gotM = d_W.download(), d_M.download()
        untouched = np.ones((K, N), bool)
        untouched[np.ix_(inP, outP)] = False
        assert np.array_equal(gotW[untouched], W[untouched]) and np.array_equal(gotM[untouched], M[untouched])
        assert np.allclose(gotW, wantW, rtol=1e-6, atol=1e-7) and np.allclose(gotM, wantM, rtol=1e-6, atol=1e-8)
    # a vector is a matrix of one row: null row list
    B = rng.standard_normal(64).astype(np.float32)
    outP = np.array([3, 9, 63], np.int32)
    d_b = ctx.empty(3, np.float32)
    scn._check(scn.lib().scn_shrink_matrix(ctx.h, ctx.array(B).ptr, d_b.ptr, None, ctx.array(outP).ptr, 64, 1, 3))
    assert np.array_equal(d_b.download(), B[outP])


def test_empty_inputs_and_bad_arguments(scn, ctx):
    """M = 0 is legal everywhere (gradients of nothing are zero); null buffers and bad sizes are refused."""
    K, N = 8, 16
    one = ctx.array(np.ones(4, np.float32))
    d_db = ctx.array(np.full(N, 5, np.float32))
    ctx.activation_backward(one, one, 0, N, scn.RELU, None, d_db, None)
    assert not d_db.download().any()
    d_dW = ctx.array(np.full((K, N), 5, np.float32))
    ctx.sgemm_AtB(one, one, d_dW, 0, K, N)
    assert not d_dW.download().any()
    ws = ctx.empty(scn.lib().scn_sgemm_ABt_workspace(N, K), np.float32)
    ctx.sgemm_ABt(one, one, one, 0, N, K, ws)
    ctx.softmax_grad(one, ctx.array(np.zeros(1, np.int32)), one, 0, 4)
    ctx.gather_rows_backward(one, one, ctx.array(np.zeros(1, np.int32)), 0, 4)
    ctx.maxpool_backward(one, one, 0, 4, ctx.array(np.zeros(1, np.int32)))
    ctx.terminal_pool_backward(one, one, ctx.array(np.zeros(1, np.int32)), 0, 4, 1)
    ctx.nag_update(one, one, one, 0, 0.1, 0.9)
    assert ctx.sum_abs(one, 0) == 0.0 and ctx.sum_abs(one, 4) == 4.0
    ctx.scale(one, 4, 0.5)
    assert one.download().tolist() == [0.5] * 4
    L = scn.lib()
    assert L.scn_activation_backward(ctx.h, one.ptr, one.ptr, 1, 4, 99, None, one.ptr, None) == scn.ERR_ARG
    assert L.scn_activation_backward(ctx.h, one.ptr, one.ptr, 1, 4, scn.PRELU, None, one.ptr, None) == scn.ERR_ARG
    assert L.scn_sgemm_AtB(ctx.h, None, one.ptr, one.ptr, 4, 1, 1) == scn.ERR_ARG
    assert L.scn_sgemm_ABt(ctx.h, one.ptr, one.ptr, one.ptr, 4, 1, 1, None) == scn.ERR_ARG
    assert L.scn_nag_update(ctx.h, one.ptr, None, one.ptr, 4, 0.1, 0.9, 0) == scn.ERR_ARG
    assert L.scn_gather_rows_backward(ctx.h, one.ptr, one.ptr, None, 4, 1) == scn.ERR_ARG
    assert L.scn_terminal_pool_backward(ctx.h, one.ptr, one.ptr, one.ptr, 1, 4, 0) == scn.ERR_ARG
    assert b"scn_terminal_pool_backward" in L.scn_last_error()
