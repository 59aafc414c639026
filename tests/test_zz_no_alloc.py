"""scn_sgemm_ABt_static: dA = D W^T with the transposed weights in the library's
static device array instead of a caller's workspace (for callers that cannot
allocate).  Checked against scn_sgemm_ABt (bit for bit: same kernels, same
order) and against the oracle (1e-4 of the row's scale), on two calls in a row
that share the array, the second smaller than the first."""
import numpy as np
import pytest

import oracle as orc

pytestmark = pytest.mark.gpu


def run_pair(scn, ctx, M, N, K, seed):
    rng = np.random.default_rng(seed)
    print("ABt static M=%d N=%d K=%d" % (M, N, K), flush=True)
    D = rng.standard_normal((M, N)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    d_D, d_W = ctx.array(D), ctx.array(W)
    ref = ctx.empty((M, K), np.float32)
    ws = ctx.empty(scn.lib().scn_sgemm_ABt_workspace(N, K), np.float32)
    ctx.sgemm_ABt(d_D, d_W, ref, M, N, K, ws)
    got = ctx.empty((M, K), np.float32)
    ctx.sgemm_ABt_static(d_D, d_W, got, M, N, K)
    g, r = got.download(), ref.download()
    assert np.array_equal(g, r)
    orc.set_threads(8)
    want = orc.sgemm_ABt(D, W)
    scale = np.abs(D).astype(np.float64) @ np.abs(W).astype(np.float64).T + 1e-6
    assert np.max(np.abs(g.astype(np.float64) - want) / scale) <= 1e-4


def test_two_calls_share_the_static_array(scn, ctx):
    # the first call leaves 800 x 800 transposed weights in the array, the
    # second uses a corner of it; then a shape whose zero bias sits in the array
    # too (K beyond the context's own row of zeros)
    run_pair(scn, ctx, 2500, 800, 800, 1)
    run_pair(scn, ctx, 333, 100, 192, 2)
    run_pair(scn, ctx, 64, 32, 5000, 3)
    run_pair(scn, ctx, 7, 1, 1, 4)


def test_sizes_beyond_the_array_are_refused(scn, ctx):
    L = scn.lib()
    limit = L.scn_sgemm_ABt_static_limit()
    assert limit == 1 << 20
    one = ctx.empty(4, np.float32)
    # (argument check only: nothing is launched)
    assert L.scn_sgemm_ABt_static(ctx.h, one.ptr, one.ptr, one.ptr, 4, 1024, 1024) == scn.ERR_CAPACITY
    assert "static" in L.scn_last_error().decode()
    assert L.scn_sgemm_ABt_static(ctx.h, one.ptr, one.ptr, one.ptr, 4, 0, 4) == scn.ERR_ARG
    # an empty product is not an error and launches nothing
    assert L.scn_sgemm_ABt_static(ctx.h, one.ptr, one.ptr, one.ptr, 0, 4, 4) == scn.OK
