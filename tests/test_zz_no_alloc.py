"""scn_sgemm_ABt_static: dA = D W^T with the transposed weights in the library's
static device array instead of a caller's workspace (for callers that cannot
allocate).  Checked against scn_sgemm_ABt (bit for bit: same kernels, same
order) and against the oracle (1e-4 of the row's scale), on two calls in a row
that share the array, the second smaller than the first."""
import ctypes as C

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


def free_device_memory():
    """Free bytes of the current device, from the HIP runtime the library itself is linked to."""
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_the_static_call_allocates_nothing(scn, ctx):
    """What the entry point is for: device memory is as free after its calls as before them -- also after the first
    call of a context made just now -- while the same product through a caller's workspace takes that workspace."""
    rng = np.random.default_rng(5)
    M, N, K = 900, 512, 768
    d_D = ctx.array(rng.standard_normal((M, N)).astype(np.float32))
    d_W = ctx.array(rng.standard_normal((K, N)).astype(np.float32))
    got = ctx.empty((M, K), np.float32)
    fresh = scn.Context()
    try:
        fresh.sync()
        ctx.sync()
        before = free_device_memory()
        # (inputs and output belong to the other context: device memory is the device's)
        fresh.sgemm_ABt_static(d_D, d_W, got, M, N, K)
        fresh.sync()
        assert free_device_memory() == before
        for _ in range(3):
            ctx.sgemm_ABt_static(d_D, d_W, got, M, N, K)
        ctx.sync()
        assert free_device_memory() == before
        # the method does see an allocation of the size the call would need
        ws = ctx.empty(scn.lib().scn_sgemm_ABt_workspace(N, K) + (8 << 20), np.float32)
        assert free_device_memory() < before
        ws.free()
    finally:
        fresh.close()


def test_a_second_context_waits_its_turn(scn, ctx):
    """The array is one per device: a call from another context is refused while the last call that used the array
    has not finished, and accepted once it has."""
    L = scn.lib()
    rng = np.random.default_rng(6)
    M, N, K = 200000, 256, 256  # long enough to be still running when the other context asks
    d_D = ctx.array(rng.standard_normal((M, N)).astype(np.float32))
    d_W = ctx.array(rng.standard_normal((K, N)).astype(np.float32))
    got = ctx.empty((M, K), np.float32)
    other = scn.Context()
    small = other.empty((4, K), np.float32)
    ctx.sync()
    for _ in range(20):
        ctx.sgemm_ABt_static(d_D, d_W, got, M, N, K)
    rc = L.scn_sgemm_ABt_static(other.h, d_D.ptr, d_W.ptr, small.ptr, 4, N, K)
    ctx.sync()
    if rc != scn.OK:  # (the twenty products were still on their way: the usual case)
        assert rc == scn.ERR_STATE and "another context" in L.scn_last_error().decode()
    other.sgemm_ABt_static(d_D, d_W, small, 4, N, K)
    other.sync()
    ref = ctx.empty((4, K), np.float32)
    ws = ctx.empty(L.scn_sgemm_ABt_workspace(N, K), np.float32)
    ctx.sgemm_ABt(d_D, d_W, ref, 4, N, K, ws)
    assert np.array_equal(small.download(), ref.download())
    other.close()
