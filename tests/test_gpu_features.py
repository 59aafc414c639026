"""Feature kernels against the CPU oracle (through the C ABI)."""
import numpy as np
import pytest

import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("nIn", [1, 3, 4, 32, 33, 64, 160, 288, 1030])
def test_gather_bit_exact(scn, ctx, nIn):
    rng = np.random.default_rng(nIn)
    rows = 501
    inp = rng.standard_normal((rows, nIn)).astype(np.float32)
    for count in (1, 255, 256, 257, 5000):
        print("gather nIn=%d count=%d" % (nIn, count), flush=True)
        rules = rng.integers(0, rows, size=count).astype(np.int32)
        d_out = ctx.empty((count, nIn), np.float32)
        ctx.gather_rows(ctx.array(inp), d_out, ctx.array(rules), count, nIn)
        assert np.array_equal(d_out.download(), orc.gather_rows(inp, rules, nIn))


@pytest.mark.parametrize("C,ps", [(32, 4), (32, 9), (64, 8), (96, 27), (3, 4), (160, 9), (5, 3)])
def test_maxpool_values_and_argmax_bit_exact(scn, ctx, C, ps):
    rng = np.random.default_rng(C * 100 + ps)
    rows, nOut = 300, 777
    # quantised values force ties; the first maximum in window order must win
    inp = rng.integers(-2, 3, size=(rows, C)).astype(np.float32)
    rules = rng.integers(-1, rows, size=(nOut, ps)).astype(np.int32)
    rules[:, 0] = np.abs(rules[:, 0])
    print("maxpool C=%d ps=%d" % (C, ps), flush=True)
    d_out = ctx.empty((nOut, C), np.float32)
    d_choice = ctx.empty((nOut, C), np.int32)
    ctx.maxpool(ctx.array(inp), d_out, ctx.array(rules), nOut, ps, C, d_choice)
    o_out, o_choice = orc.maxpool(inp, rules, nOut, ps, C)
    assert np.array_equal(d_out.download(), o_out)
    assert np.array_equal(d_choice.download(), o_choice)
    # random floats as well
    inp = rng.standard_normal((rows, C)).astype(np.float32)
    ctx.maxpool(ctx.array(inp), d_out, ctx.array(rules), nOut, ps, C, d_choice)
    o_out, o_choice = orc.maxpool(inp, rules, nOut, ps, C)
    assert np.array_equal(d_out.download(), o_out)
    assert np.array_equal(d_choice.download(), o_choice)


def test_terminal_pool_bit_exact(scn, ctx):
    rng = np.random.default_rng(1)
    rows, C, B, S = 400, 192, 37, 9
    inp = rng.standard_normal((rows, C)).astype(np.float32)
    rules = np.full((B, S), -1, np.int32)
    for b in range(B):
        n = 1 + b % S
        rules[b, :n] = rng.integers(0, rows, n)
    d_out = ctx.empty((B, C), np.float32)
    ctx.terminal_pool(ctx.array(inp), d_out, ctx.array(rules), B, S, C)
    assert np.array_equal(d_out.download(), orc.terminal_pool(inp, rules, B, S, C))


@pytest.mark.parametrize("C", [32, 5])
def test_pooling_over_an_input_without_rows(scn, ctx, C):
    """Every rule negative and no input row at all (a null input): max-pooling gives zeros and choice 0, terminal
    pooling 0 / 0, as the oracle does; nothing of the input is read."""
    nOut, ps = 70, 9
    rules = np.full((nOut, ps), -1, np.int32)
    d_out = ctx.array(np.full((nOut, C), 7, np.float32))
    d_choice = ctx.array(np.full((nOut, C), 7, np.int32))

    class null:  # no input buffer at all
        ptr = None

    ctx.maxpool(null, d_out, ctx.array(rules), nOut, ps, C, d_choice)
    o_out, o_choice = orc.maxpool(np.zeros((1, C), np.float32), rules, nOut, ps, C)
    assert np.array_equal(d_out.download(), o_out) and np.array_equal(d_choice.download(), o_choice)
    ctx.terminal_pool(null, d_out, ctx.array(rules), nOut, ps, C)
    want = orc.terminal_pool(np.zeros((1, C), np.float32), rules, nOut, ps, C)
    assert np.array_equal(np.isnan(d_out.download()), np.isnan(want)) and np.all(np.isnan(want))


def test_softmax(scn, ctx):
    rng = np.random.default_rng(2)
    for M, N in ((100, 100), (7, 40), (3, 1), (130, 1000)):
        x = (rng.standard_normal((M, N)) * 4).astype(np.float32)
        d_out = ctx.empty((M, N), np.float32)
        ctx.softmax_rows(ctx.array(x), d_out, M, N)
        got = d_out.download()
        want = orc.softmax_rows(x)
        # tolerance: fp32 forward path, 1e-4 relative
        assert np.allclose(got, want, rtol=1e-4, atol=1e-7)
        assert np.array_equal(got.argmax(1), want.argmax(1))
    lo = np.full((1, 3), -10050.0, np.float32)
    lo[0, 1] = -10040.0
    d_out = ctx.empty((1, 3), np.float32)
    ctx.softmax_rows(ctx.array(lo), d_out, 1, 3)
    assert np.allclose(d_out.download(), orc.softmax_rows(lo), rtol=1e-4)


SHAPES = [(1000, 12, 32), (777, 128, 64), (513, 256, 96), (300, 384, 128), (129, 512, 160), (400, 160, 192),
          (100, 192, 100), (64, 288, 64), (5, 7, 3), (2000, 27, 32), (257, 1728, 64),
          # enough 16-row panels that wavefronts of the W-resident kernel walk several, last one ragged
          (70001, 128, 64), (40003, 256, 96),
          # W-resident kernel: an odd number of prefetch groups, a 48-column slice, many narrow slices
          (600, 160, 192), (1000, 64, 48), (2469, 512, 160),
          # few rows (split-k kernel): ragged row and column blocks; few input channels (thin kernel)
          (3, 40, 100), (511, 1024, 36), (83, 9, 5), (5000, 12, 32), (4097, 28, 100),
          # contractions too long for W to stay in LDS (W-streaming kernel): narrow slices with a ragged
          # last group of panels, two-step slabs with a 48-column slice, many slices
          (1500, 1728, 64), (1100, 2016, 48), (1025, 3200, 320)]
# ... and with enough rows for its wide slices (64 and 96 columns)
STREAMED_WIDE = [(66001, 1728, 64), (33005, 1728, 96)]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("act", ["NOSIGMOID", "RELU", "LEAKYRELU", "VLEAKYRELU", "PRELU", "SOFTMAX"])
def test_nin_fp32(scn, ctx, M, K, N, act):
    """fp32 activations within 1e-4 relative of the oracle (scaled by the
    magnitude of the contraction, since individual outputs can cancel)."""
    a = getattr(scn, act)
    rng = np.random.default_rng(M + K + N + a)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    B = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    pr = rng.uniform(0.1, 0.4, N).astype(np.float32)
    p = 0.75 if act == "RELU" else 1.0
    print("nin M=%d K=%d N=%d act=%s" % (M, K, N, act), flush=True)
    d_out = ctx.empty((M, N), np.float32)
    ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(B), ctx.array(pr), d_out, M, K, N, p, a, scn.FP32)
    got = d_out.download()
    want64 = orc.nin_forward(A, W, B, pr, p, a, f64=True)
    want32 = orc.nin_forward(A, W, B, pr, p, a)
    if act == "SOFTMAX":
        assert np.allclose(got, want64, rtol=1e-4, atol=1e-6)
        return
    scale = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
    assert np.all(np.abs(got - want64) <= 1e-4 * scale)
    # and no further from fp64 than the oracle's own fp32 accumulation, within a factor
    err_gpu = np.abs(got - want64).max()
    err_cpu = np.abs(want32 - want64).max()
    assert err_gpu <= 4 * err_cpu + 1e-6
    rel = np.linalg.norm(got - want64) / max(np.linalg.norm(want64), 1e-30)
    assert rel <= 1e-4


@pytest.mark.parametrize("M,K,N", STREAMED_WIDE)
@pytest.mark.parametrize("act", ["RELU", "PRELU"])
def test_nin_fp32_streamed_w_wide_slices(scn, ctx, M, K, N, act):
    test_nin_fp32(scn, ctx, M, K, N, act)


@pytest.mark.parametrize("M,K,N", [(777, 128, 64), (5, 7, 3), (40003, 256, 96), (1500, 1728, 64), (4097, 28, 100)])
@pytest.mark.parametrize("act", ["TANH", "SIGMOID"])
def test_nin_fp32_squashing_activations(scn, ctx, M, K, N, act):
    """tanh and the logistic function (SigmoidLayer.cu:43-48, 80-85): a pass over the output of any NiN kernel."""
    a = getattr(scn, act)
    rng = np.random.default_rng(M + K + N + a)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    B = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    d_out = ctx.empty((M, N), np.float32)
    ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(B), None, d_out, M, K, N, 0.9, a, scn.FP32)
    got = d_out.download()
    want64 = orc.nin_forward(A, W, B, None, 0.9, a, f64=True)
    # both functions have slope <= 1: the error of the contraction carries over at most unchanged
    scale = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
    assert np.all(np.abs(got - want64) <= 1e-4 * scale + 1e-6)
    pre = np.float64(np.float32(0.9)) * (A.astype(np.float64) @ W.astype(np.float64) + B)
    closed = np.tanh(pre) if act == "TANH" else 1.0 / (1.0 + np.exp(-pre))
    assert np.allclose(want64, closed, rtol=1e-9, atol=1e-12)  # the oracle against the closed form
    assert np.allclose(orc.nin_forward(A, W, B, None, 0.9, a), closed, rtol=1e-4, atol=1e-5)


def test_nin_special_cases(scn, ctx):
    rng = np.random.default_rng(3)
    M, K = 70, 64
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal(K).astype(np.float32)
    d_out = ctx.empty((M, K), np.float32)
    ctx.nin_forward(ctx.array(A), ctx.array(np.eye(K, dtype=np.float32)), ctx.array(B), None, d_out, M, K, K, 1.0,
                    scn.NOSIGMOID)
    assert np.array_equal(d_out.download(), A + B)
    W = np.zeros((K, K), np.float32)
    W[3, 7] = 2.0
    ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(np.zeros(K, np.float32)), None, d_out, M, K, K, 1.0,
                    scn.NOSIGMOID)
    want = np.zeros((M, K), np.float32)
    want[:, 7] = 2.0 * A[:, 3]
    assert np.array_equal(d_out.download(), want)
    with pytest.raises(scn.ScnError):
        ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(B), None, d_out, M, K, K, 1.0, 8)  # no such activation
    with pytest.raises(scn.ScnError):
        ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(B), None, d_out, M, K, K, 1.0, scn.PRELU)


def to_bf16(x):
    """Round fp32 to bf16 (nearest even) and back, in numpy."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32)


@pytest.mark.parametrize("M,K,N", [(777, 128, 64), (513, 256, 96), (129, 512, 160), (400, 160, 192), (100, 192, 100),
                                   (3000, 1728, 64), (64, 288, 32), (2000, 64, 32)])
@pytest.mark.parametrize("act", ["RELU", "PRELU", "NOSIGMOID"])
def test_nin_bf16(scn, ctx, M, K, N, act):
    check_nin_bf16(scn, ctx, M, K, N, act)


# the bf16 W-streaming kernel with wide slices (64 and 96 columns), every depth of its prefetch ring
# (K / 32 a multiple of 4, of 6, of neither), ragged last groups
# ... and the wide contractions of the GEMM-bound 2-D net (K up to 2560, N up to 800)
@pytest.mark.parametrize("M,K,N", [(66001, 1728, 64), (33005, 192, 96), (40003, 256, 96), (70001, 320, 128),
                                   (1, 64, 32), (15, 128, 32), (255, 512, 160), (1025, 3200, 320), (2600, 2560, 800)])
def test_nin_bf16_streamed_w(scn, ctx, M, K, N):
    check_nin_bf16(scn, ctx, M, K, N, "PRELU", x3=False)


def check_nin_bf16(scn, ctx, M, K, N, act, x3=True):
    """bf16 operands, fp32 accumulation: within 2e-2 relative of the fp32
    oracle, and within 1e-4 of the same contraction with operands rounded to
    bf16 on the host (i.e. the rounding is the only difference)."""
    a = getattr(scn, act)
    rng = np.random.default_rng(M + K + N + a)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    B = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    pr = rng.uniform(0.1, 0.4, N).astype(np.float32)
    print("nin bf16 M=%d K=%d N=%d act=%s" % (M, K, N, act), flush=True)
    d_out = ctx.empty((M, N), np.float32)
    ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(B), ctx.array(pr), d_out, M, K, N, 1.0, a, scn.BF16)
    got = d_out.download()
    want = orc.nin_forward(A, W, B, pr, 1.0, a, f64=True)
    scale = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
    assert np.all(np.abs(got - want) <= 2e-2 * scale)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 2e-2
    rounded = orc.nin_forward(to_bf16(A), to_bf16(W), B, pr, 1.0, a, f64=True)
    assert np.all(np.abs(got - rounded) <= 1e-4 * scale)
    if K >= 64:  # the rounding is really there: the result differs from fp32
        assert np.abs(got - want).max() > 1e-5
    if not x3:
        return
    # hi + lo operand pairs, three MFMAs per tile: back within the fp32 tolerance
    ctx.nin_forward(ctx.array(A), ctx.array(W), ctx.array(B), ctx.array(pr), d_out, M, K, N, 1.0, a, scn.BF16X3)
    got3 = d_out.download()
    assert np.all(np.abs(got3 - want) <= 1e-4 * scale)
    assert np.linalg.norm(got3 - want) / np.linalg.norm(want) <= 1e-4


# (a few rows: the deepest convolutions of a batch of one to four samples)
@pytest.mark.parametrize("rows,fs,nIn,N", [(700, 4, 32, 64), (3000, 9, 64, 96), (513, 27, 64, 64), (66001, 27, 64, 64),
                                           (33005, 8, 24, 96), (1100, 4, 112, 160), (1, 4, 32, 64), (7, 4, 128, 160),
                                           (100, 9, 64, 96), (255, 4, 96, 128)])
def test_fused_gather_nin_bf16_matches_the_two_kernels_bit_for_bit(scn, ctx, rows, fs, nIn, N):
    """scn_conv_nin_forward_p with bf16 operands: the same bits as gather + bf16 NiN, and the bf16 bar against the
    oracle."""
    rng = np.random.default_rng(rows + fs + nIn + N)
    nInRows = 500
    inp = rng.uniform(-1, 1, (nInRows, nIn)).astype(np.float32)
    rules = rng.integers(0, nInRows, (rows, fs)).astype(np.int32)
    rules[rng.random((rows, fs)) < 0.2] = -1
    K = fs * nIn
    W = (rng.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    B = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    assert scn.lib().scn_conv_nin_supported_p(fs, nIn, N, scn.BF16)
    d_in, d_rules, d_W, d_B = ctx.array(inp), ctx.array(rules), ctx.array(W), ctx.array(B)
    fused = ctx.empty((rows, N), np.float32)
    ctx.conv_nin_forward(d_in, d_rules, fs, nIn, d_W, d_B, None, fused, rows, N, 1.0, scn.RELU, scn.BF16)
    g = ctx.empty((rows, K), np.float32)
    two = ctx.empty((rows, N), np.float32)
    ctx.gather_rows(d_in, g, d_rules, rows * fs, nIn)
    ctx.nin_forward(g, d_W, d_B, None, two, rows, K, N, 1.0, scn.RELU, scn.BF16)
    assert np.array_equal(fused.download(), two.download())
    gathered = np.where(rules[:, :, None] >= 0, inp[np.maximum(rules, 0)], 0).reshape(rows, K).astype(np.float32)
    scale = np.abs(gathered).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
    want = orc.nin_forward(gathered, W, B, None, 1.0, scn.RELU, f64=True)
    assert np.all(np.abs(fused.download() - want) <= 2e-2 * scale)
    rounded = orc.nin_forward(to_bf16(gathered), to_bf16(W), B, None, 1.0, scn.RELU, f64=True)
    assert np.all(np.abs(fused.download() - rounded) <= 1e-4 * scale)
    # channels not in multiples of 8, a contraction not of 64, the split mode: not fused with bf16 operands
    assert not scn.lib().scn_conv_nin_supported_p(4, 20, 64, scn.BF16)
    assert not scn.lib().scn_conv_nin_supported_p(3, 32, 64, scn.BF16)
    assert not scn.lib().scn_conv_nin_supported_p(4, 32, 64, scn.BF16X3)
    assert scn.lib().scn_conv_nin_supported_p(4, 20, 64, scn.FP32)


def test_gather_negative_rule_is_zero_row(scn, ctx):
    rng = np.random.default_rng(4)
    inp = rng.standard_normal((50, 32)).astype(np.float32)
    rules = rng.integers(0, 50, 1000).astype(np.int32)
    rules[::7] = -1
    d_out = ctx.empty((1000, 32), np.float32)
    ctx.gather_rows(ctx.array(inp), d_out, ctx.array(rules), 1000, 32)
    want = np.where(rules[:, None] < 0, np.float32(0), inp[np.maximum(rules, 0)])
    assert np.array_equal(d_out.download(), want)


def test_argument_errors(scn, ctx):
    d = ctx.empty(16, np.float32)
    r = ctx.empty(16, np.int32)
    with pytest.raises(scn.ScnError):
        ctx.gather_rows(d, d, r, 4, 0)
    with pytest.raises(scn.ScnError):
        ctx.maxpool(d, d, r, 4, 0, 4, r)
    with pytest.raises(scn.ScnError):
        ctx.terminal_pool(d, d, r, 1, 0, 4)
    with pytest.raises(scn.ScnError):
        ctx.softmax_rows(d, d, 1, 0)
    # zero-sized work is accepted and does nothing
    ctx.gather_rows(d, d, r, 0, 4)
    ctx.maxpool(d, d, r, 0, 2, 4, r)
    ctx.sync()


@pytest.mark.parametrize("rows,fs,nIn,N", [(700, 4, 32, 64), (3000, 9, 64, 96), (513, 27, 64, 64), (129, 8, 96, 128),
                                           (5000, 4, 128, 160), (64, 1, 4, 32), (300, 25, 8, 100),
                                           # W-streaming kernel: every width of slice, every size of rule load
                                           (1500, 27, 64, 64), (66001, 27, 64, 64), (33005, 9, 192, 96),
                                           (1100, 4, 504, 48),
                                           # ... slabs of 32 k within one filter position (32 and 96 channels)
                                           (2000, 27, 32, 64), (40001, 9, 96, 64),
                                           # few channels: the thin kernel (and the few-rows kernel) through the rules
                                           (83597, 4, 3, 32), (20000, 8, 1, 32), (300, 4, 3, 32), (400, 16, 2, 32),
                                           (9000, 16, 2, 64), (2500, 4, 2, 160), (5000, 2, 6, 36)])
@pytest.mark.parametrize("act", ["RELU", "PRELU"])
def test_fused_gather_nin_matches_the_two_kernels_bit_for_bit(scn, ctx, rows, fs, nIn, N, act):
    a = getattr(scn, act)
    rng = np.random.default_rng(rows + fs + nIn + N)
    nInRows = 400
    inp = rng.uniform(-1, 1, (nInRows, nIn)).astype(np.float32)
    rules = rng.integers(0, nInRows, (rows, fs)).astype(np.int32)
    rules[rng.random((rows, fs)) < 0.2] = -1  # no input site there
    K = fs * nIn
    W = (rng.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    B = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    pr = rng.uniform(0.1, 0.4, N).astype(np.float32)
    assert scn.lib().scn_conv_nin_supported(fs, nIn, N)
    print("fused rows=%d fs=%d nIn=%d N=%d" % (rows, fs, nIn, N), flush=True)
    d_in, d_rules, d_W, d_B, d_pr = ctx.array(inp), ctx.array(rules), ctx.array(W), ctx.array(B), ctx.array(pr)
    fused = ctx.empty((rows, N), np.float32)
    ctx.conv_nin_forward(d_in, d_rules, fs, nIn, d_W, d_B, d_pr, fused, rows, N, 1.0, a)
    g = ctx.empty((rows, K), np.float32)
    two = ctx.empty((rows, N), np.float32)
    ctx.gather_rows(d_in, g, d_rules, rows * fs, nIn)
    ctx.nin_forward(g, d_W, d_B, d_pr, two, rows, K, N, 1.0, a, scn.FP32)
    assert np.array_equal(fused.download(), two.download())
    # (a rule of -1 reads as a row of zeros; the oracle's gather has the reference's rules, which name a zero row)
    gathered = np.where(rules[:, :, None] >= 0, inp[np.maximum(rules, 0)], 0).reshape(rows, K).astype(np.float32)
    want = orc.nin_forward(gathered, W, B, pr, 1.0, a, f64=True)
    scale = np.abs(gathered).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)
    assert np.all(np.abs(fused.download() - want) <= 1e-4 * scale)
    assert not scn.lib().scn_conv_nin_supported(64, 32, 64)  # window too large for the staged rules
    assert scn.lib().scn_conv_nin_supported(4, 3, 32)  # few channels, contraction of 12: the thin kernel
    assert not scn.lib().scn_conv_nin_supported(9, 3, 32)  # channels not a multiple of 4 and a contraction beyond it
    assert not scn.lib().scn_conv_nin_supported(5, 3, 32)  # ... or not a multiple of 4


@pytest.mark.parametrize("M,rows,fs,nIn,N,act", [
    (40000, 9000, 27, 64, 64, "RELU"), (20011, 5000, 8, 64, 96, "PRELU"), (7000, 3000, 4, 32, 64, "VLEAKYRELU"),
    (1030, 400, 9, 128, 160, "RELU"), (3, 10, 4, 64, 32, "NOSIGMOID"), (2600, 700, 4, 96, 128, "LEAKYRELU"),
    # a shape the bf16 kernel does not take (few channels): what scn_conv_nin_forward_p(SCN_BF16) does
    (5000, 1000, 4, 3, 32, "RELU")])
def test_bf16_rows_rounded_once_give_the_same_bits(scn, ctx, M, rows, fs, nIn, N, act):
    """scn_conv_nin_forward_a16 (the input matrix rounded to bf16 once, the contraction reading those rows) against
    scn_conv_nin_forward_p with SCN_BF16 (rows rounded in registers as they are read): the same bits, and within the
    bf16 bar (2e-2 of the row's scale) of the oracle."""
    rng = np.random.default_rng(M + rows + N)
    act_id = getattr(scn, act)
    K = fs * nIn
    src = rng.standard_normal((rows, nIn)).astype(np.float32)
    rules = rng.integers(-1, rows, size=(M, fs)).astype(np.int32)
    W = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    B = rng.standard_normal(N).astype(np.float32)
    prelu = rng.uniform(0.1, 0.4, N).astype(np.float32) if act == "PRELU" else None
    d_src, d_rules, d_W, d_B = ctx.array(src), ctx.array(rules), ctx.array(W), ctx.array(B)
    d_prelu = ctx.array(prelu) if prelu is not None else None
    print("a16 M=%d rows=%d fs=%d nIn=%d N=%d %s" % (M, rows, fs, nIn, N, act), flush=True)
    one = ctx.array(np.full((M, N), 9, np.float32))
    two = ctx.array(np.full((M, N), 9, np.float32))
    rows16 = ctx.empty((rows * nIn + 8) // 2, np.float32)  # two bytes an element
    ctx.conv_nin_forward(d_src, d_rules, fs, nIn, d_W, d_B, d_prelu, one, M, N, 0.9, act_id, scn.BF16)
    ctx.conv_nin_forward_a16(d_src, rows, rows16, d_rules, fs, nIn, d_W, d_B, d_prelu, two, M, N, 0.9, act_id)
    got = two.download()
    assert np.array_equal(got, one.download())
    G = np.where(rules[:, :, None] >= 0, src[np.maximum(rules, 0)], 0).reshape(M, K).astype(np.float32)
    want = orc.nin_forward(G, W, B, prelu, 0.9, act_id, f64=True)
    scale = 0.9 * (np.abs(G).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(B)) + 1e-6
    assert np.max(np.abs(got - want) / scale) <= 2e-2


def test_maxpool_refuses_inputs_beyond_32_bit_choices(scn, ctx):
    """poolingChoices are 32-bit element indices into the input (MaxPoolingLayer.cu:9-35): the entry point that is told
    the input's row count refuses 2^31 elements and more.  An argument check: nothing is launched, no such buffer
    is needed."""
    L = scn.lib()
    one = ctx.empty(4, np.float32)
    rows = (1 << 31) // 64
    assert L.scn_maxpool_checked(ctx.h, one.ptr, rows, one.ptr, one.ptr, 1, 1, 64, one.ptr) == scn.ERR_CAPACITY
    assert "32-bit" in L.scn_last_error().decode()
    assert L.scn_maxpool_checked(ctx.h, one.ptr, -1, one.ptr, one.ptr, 1, 1, 64, one.ptr) == scn.ERR_ARG
    # the largest input that fits, with no output rows asked for: accepted
    assert L.scn_maxpool_checked(ctx.h, one.ptr, rows - 1, one.ptr, one.ptr, 0, 1, 64, one.ptr) == scn.OK
    # ... and an ordinary call gives what scn_maxpool gives
    rng = np.random.default_rng(1)
    feats = rng.standard_normal((50, 8)).astype(np.float32)
    rules = rng.integers(0, 50, (20, 4)).astype(np.int32)
    d_f, d_r = ctx.array(feats), ctx.array(rules)
    a, ca, b, cb = ctx.empty((20, 8), np.float32), ctx.empty((20, 8), np.int32), ctx.empty((20, 8), np.float32), ctx.empty((20, 8), np.int32)
    ctx.maxpool(d_f, a, d_r, 20, 4, 8, ca)
    assert L.scn_maxpool_checked(ctx.h, d_f.ptr, 50, b.ptr, d_r.ptr, 20, 4, 8, cb.ptr) == scn.OK
    assert np.array_equal(a.download(), b.download()) and np.array_equal(ca.download(), cb.download())
