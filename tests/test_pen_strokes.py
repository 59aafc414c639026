"""Pen-stroke front-end (OnlineHandwritingPicture) of the host library against the
oracle restatement, hand-computed characters and closed forms.  CPU only, except the
last test, which runs characters through a 2-D net on the GPU."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import pen_picture as pen  # noqa: E402
from gpu_util import assert_probabilities


def hostapi():
    from conftest import load_scn
    load_scn()
    from sparseconvnet_archived_amd import hostapi as h
    if not os.path.exists(h.LIB_PATH):
        pytest.skip("libscn_host.so is not built")
    return h


def one_character(strokes, enc, side, render=8, normalize=False, seed=-1, batch_type=None):
    h = hostapi()
    ds = h.Dataset("pen", pen.ENCODING_FEATURES[enc], 10, h.TESTBATCH if batch_type is None else batch_type)
    ds.add_strokes(strokes, render, enc, 3, normalize)
    out = ds.codify(0, side, seed)
    ds.close()
    return out


def test_constant_speed_on_a_straight_stroke():
    h = hostapi()
    # length 10 at density 0.1: 100 intervals, 101 points, equally spaced, ends kept
    for got in (h.constant_speed([(0, 0), (10, 0)], 0.1), pen.constant_speed([(0, 0), (10, 0)], 0.1)):
        assert got.shape == (101, 2)
        assert np.allclose(got[:, 0], np.arange(101) / 10.0, atol=2e-5) and np.all(got[:, 1] == 0)
    # the multiplier multiplies the number of intervals
    assert len(h.constant_speed([(0, 0), (3, 4)], 0.5, 3)) == 10 * 3 + 1
    # a stroke shorter than half the density collapses to its first point; so does a single point
    assert h.constant_speed([(1, 2), (1.01, 2)], 0.1).tolist() == [[1, 2]]
    assert h.constant_speed([(5, 6)], 0.1).tolist() == [[5, 6]]


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_constant_speed_on_polylines(seed):
    h = hostapi()
    rng = np.random.default_rng(seed)
    stroke = np.cumsum(rng.uniform(-3, 3, (12, 2)), 0)
    got = h.constant_speed(stroke, 0.1)
    want = pen.constant_speed(stroke, 0.1)
    assert got.shape == want.shape and np.array_equal(got, want)  # the same arithmetic, bit for bit
    seg = np.linalg.norm(np.diff(stroke, axis=0), axis=1)
    assert len(got) == int(0.5 + np.float32(seg.sum()) / np.float32(0.1)) + 1
    assert np.allclose(got[0], stroke[0]) and np.allclose(got[-1], stroke[-1], atol=1e-3)
    # every point lies on the polyline: distance to the nearest segment is ~0
    for p in got[:: max(1, len(got) // 40)]:
        a, b = stroke[:-1], stroke[1:]
        t = np.clip(((p - a) * (b - a)).sum(1) / ((b - a) ** 2).sum(1), 0, 1)
        assert np.min(np.linalg.norm(a + t[:, None] * (b - a) - p, axis=1)) < 1e-3
    # consecutive points are one density apart along the path (never more in a straight line)
    assert np.all(np.linalg.norm(np.diff(got, axis=0), axis=1) <= 0.1 * 1.01)


def test_hand_computed_simple_encoding():
    # a horizontal stroke from x = -1.95 to 2.05 at y = 0.25 in a lattice of side 8 (origin at cell 4):
    # 41 samples 0.1 apart; cell a0 = trunc(x + 4): ten samples each in cells 2..5, one in cell 6; a1 = 4
    strokes = [[(-1.95, 0.25), (2.05, 0.25)]]
    want_keys = [a0 * 8 + 4 for a0 in (2, 3, 4, 5, 6)]
    for keys, rows, bg, feats in (one_character(strokes, pen.SIMPLE, 8), pen.codify(strokes, 8, pen.SIMPLE, 8)):
        assert list(keys) == want_keys and list(rows) == [1, 2, 3, 4, 5] and bg == 0
        assert feats[:, 0].tolist() == [0, 10, 10, 10, 10, 1]


def test_negative_coordinates_truncate_toward_zero():
    # x + side/2 in (-1, 0) converts to cell 0, not -1: such samples land inside (the reference's int conversion)
    strokes = [[(-4.75, 0.5), (-4.25, 0.5)]]  # x + 4 in [-0.75, -0.25]
    keys, rows, bg, feats = one_character(strokes, pen.SIMPLE, 8)
    assert list(keys) == [0 * 8 + 4] and feats[1, 0] == 6
    # and one cell further out is outside
    keys, _, _, feats = one_character([[(-5.75, 0.5), (-5.25, 0.5)]], pen.SIMPLE, 8)
    assert len(keys) == 0 and feats.shape == (1, 1)


def test_hand_computed_octogram():
    # direction at pi/8 between compass points 0 and 1: each gets weight 1 - (pi/8)/(pi/4) = 1/2 per sample;
    # 1 unit long inside cell (4, 4): 11 samples, the last one has no direction -> 10 x 0.5
    c, s = np.cos(np.pi / 8), np.sin(np.pi / 8)
    strokes = [[(0.02, 0.02), (0.02 + c, 0.02 + s)]]
    for keys, rows, bg, feats in (one_character(strokes, pen.OCTOGRAM, 8), pen.codify(strokes, 8, pen.OCTOGRAM, 8)):
        assert list(keys) == [4 * 8 + 4]
        assert np.allclose(feats[1], [5, 5, 0, 0, 0, 0, 0, 0], atol=2e-3)
    # the opposite direction: compass points 4 and 5
    back = [strokes[0][::-1]]
    feats = one_character(back, pen.OCTOGRAM, 8)[3]
    assert np.allclose(feats[1], [0, 0, 0, 0, 5, 5, 0, 0], atol=2e-3)
    # without orientation both give the same 4 features
    f1 = one_character(strokes, pen.UNDIRECTED_OCTOGRAM, 8)[3]
    f2 = one_character(back, pen.UNDIRECTED_OCTOGRAM, 8)[3]
    assert np.allclose(f1[1], [5, 5, 0, 0], atol=2e-3) and np.allclose(f1, f2, atol=1e-4)


def test_hand_computed_space_time():
    # one vertical stroke of 21 samples (length 2) at x = 0.5 in a lattice of side 8: a0 = 4, a1 = trunc(y + 4),
    # y = -0.95 + 0.1 z.  Time axis with render = 45: a2 = trunc(45 * (z - 21 // 2) * 0.02 + 8 // 2)
    # = trunc(0.9 (z - 10) + 4): z = 5..14 give -0.5, 0.4, 1.3, 2.2, 3.1, 4.0, 4.9, 5.8, 6.7, 7.6 -> cells
    # 0, 0, 1, 2, 3, 4, 4, 5, 6, 7 (-0.5 truncates toward zero); z = 4 gives -1.4 and z = 15 gives 8.5: outside.
    strokes = [[(0.5, -0.95), (0.5, 1.05)]]
    want_cells = [(4, 3, 0), (4, 3, 1), (4, 3, 2), (4, 3, 3), (4, 4, 4), (4, 4, 5), (4, 4, 6), (4, 4, 7)]
    want_keys = [(x * 8 + y) * 8 + t for x, y, t in want_cells]
    want_counts = [2, 1, 1, 1, 2, 1, 1, 1]
    for keys, rows, bg, feats in (one_character(strokes, pen.SPACETIME3D, 8, render=45),
                                  pen.codify(strokes, 45, pen.SPACETIME3D, 8)):
        assert list(keys) == want_keys and bg == 0
        assert feats[:, 0].tolist() == [0] + want_counts
    # the vector variant adds the unit direction (0, 1) of every sample but each stroke's last
    for keys, rows, bg, f3 in (one_character(strokes, pen.VECTOR_SPACETIME3D, 8, render=45),
                               pen.codify(strokes, 45, pen.VECTOR_SPACETIME3D, 8)):
        assert list(keys) == want_keys and f3.shape == (9, 3)
        assert f3[1:, 0].tolist() == want_counts and np.allclose(f3[1:, 1], 0, atol=1e-6)
        assert np.allclose(f3[1:, 2], want_counts, atol=1e-5)


def random_character(rng, nStrokes=3):
    return [np.cumsum(rng.uniform(-1.5, 1.5, (int(rng.integers(2, 9)), 2)), 0) + rng.uniform(-2, 2, 2)
            for _ in range(nStrokes)]


@pytest.mark.parametrize("enc", [pen.SIMPLE, pen.OCTOGRAM, pen.UNDIRECTED_OCTOGRAM, pen.SPACETIME3D,
                                 pen.VECTOR_SPACETIME3D])
@pytest.mark.parametrize("seed,side,render", [(1, 16, 12), (2, 32, 30), (3, 48, 40)])
def test_codify_matches_the_oracle(enc, seed, side, render):
    """normalize + codify: the same cells in the same order as the oracle; features to 1e-5 (the two sides call
    different single-precision cos / sin / acos implementations)."""
    rng = np.random.default_rng(seed)
    strokes = random_character(rng)
    keys, rows, bg, feats = one_character(strokes, enc, side, render=render, normalize=True)
    want = pen.codify(pen.normalize(strokes, render), render, enc, side)
    assert list(keys) == list(want[0]) and list(rows) == list(want[1]) and bg == 0
    assert feats.shape == want[3].shape and np.allclose(feats, want[3], rtol=1e-5, atol=1e-5)
    assert len(keys) > 3


def test_normalize_fits_the_render_square():
    rng = np.random.default_rng(5)
    strokes = random_character(rng, 4)
    out = pen.normalize(strokes, 20)
    allp = np.concatenate(out)
    ext = allp.max(0) - allp.min(0)
    assert abs(ext.max() - 20) < 1e-4 and np.allclose(allp.max(0) + allp.min(0), 0, atol=1e-9)
    # the host library: a normalized character of render size r codified into a lattice of side r + 2 stays inside
    keys, _, _, feats = one_character(strokes, pen.SIMPLE, 22, render=20, normalize=True)
    total = sum(len(pen.constant_speed(s, 0.1)) for s in out)
    assert feats[:, 0].sum() == total


def test_distort_and_unavailable_encodings():
    h = hostapi()
    rng = np.random.default_rng(6)
    strokes = random_character(rng)
    # a test batch is not distorted; a training batch is: moved by at most 0.1875 render, stretched by at most 1.3
    plain = one_character(strokes, pen.SIMPLE, 40, render=20, normalize=True)
    same = one_character(strokes, pen.SIMPLE, 40, render=20, normalize=True, seed=4)
    assert list(plain[0]) == list(same[0]) and np.array_equal(plain[3], same[3])
    moved = one_character(strokes, pen.SIMPLE, 40, render=20, normalize=True, seed=4, batch_type=h.TRAINBATCH)
    again = one_character(strokes, pen.SIMPLE, 40, render=20, normalize=True, seed=4, batch_type=h.TRAINBATCH)
    assert list(moved[0]) == list(again[0]) and list(moved[0]) != list(plain[0])
    a = np.stack([moved[0] // 40, moved[0] % 40], 1) - 20
    assert np.abs(a).max() <= 10 * 1.3 * 1.05 + 0.1875 * 20 + 1
    ds = h.Dataset("pen", 3, 10)
    with pytest.raises(ValueError):
        ds.add_strokes(strokes, 20, 3)  # LogSignature1
    with pytest.raises(ValueError):
        ds.add_strokes(strokes, 20, pen.OCTOGRAM)  # 8 features into a dataset of 3
    ds.close()


def test_pendigits_file(tmp_path):
    h = hostapi()
    path = tmp_path / "digits.tra"
    path.write_text(""".LEXICON "0" "1"
.SEGMENT DIGIT 0-0 ? "7"
.COMMENT 7 id
.PEN_DOWN
 10 200
 60 200
 60 100
.PEN_UP
.DT 100
.PEN_DOWN
 30 150
 50 150
.PEN_UP
.SEGMENT DIGIT 0-0 ? "1"
.COMMENT 1 id
.PEN_DOWN
 40 300
 40 100
.PEN_UP
""")
    ds = h.Dataset("digits", 1, 10)
    assert ds.add_pendigits_file(path, 16, pen.SIMPLE) == 2 and len(ds) == 2
    # the first character: file points (x, y) become (-y, x); then normalized to 16 across its larger extent
    strokes = [[(-200, 10), (-200, 60), (-100, 60)], [(-150, 30), (-150, 50)]]
    want = pen.codify(pen.normalize(strokes, 16), 16, pen.SIMPLE, 20)
    keys, rows, bg, feats = ds.codify(0, 20)
    assert list(keys) == list(want[0]) and np.array_equal(feats, want[3])
    want1 = pen.codify(pen.normalize([[(-300, 40), (-100, 40)]], 16), 16, pen.SIMPLE, 20)
    keys1, _, _, feats1 = ds.codify(1, 20)
    assert list(keys1) == list(want1[0]) and np.array_equal(feats1, want1[3])
    ds.close()
    ds = h.Dataset("digits", 1, 10)
    with pytest.raises(IOError):
        ds.add_pendigits_file(tmp_path / "missing.tra", 16, pen.SIMPLE)
    ds.close()


@pytest.mark.gpu
def test_characters_through_a_2d_net(scn):
    """Octogram characters through a small 2-D net: processDataset-style batches of the stroke pictures give the
    oracle's probabilities for the cells and features the oracle's codify produces."""
    import oracle_net
    from sparseconvnet_archived_amd import hostapi as h, synthetic
    rng = np.random.default_rng(12)
    net = h.Net(2, 8, 10, threads=2)
    ora = oracle_net.Net(2, 8, 10)
    for n_ in (net, ora):
        n_.addLeNetLayerMP(32, 3, 1, 2, 2, synthetic.VLEAKYRELU)
        n_.addLeNetLayerMP(64, 2, 1, 2, 2, synthetic.VLEAKYRELU)
        n_.addTerminalPoolingLayer(2)
        n_.addSoftmaxLayer()
    for i, (W, B, pr) in synthetic.he_normal_weights(net.layers(), 4).items():
        net.set_weights(i, W, B, pr)
        ora.set_weights(i, W, B, pr)
    side = net.inputSpatialSize
    render = side - 4
    ds = h.Dataset("characters", 8, 10, h.TESTBATCH)
    chars = [random_character(rng) for _ in range(7)]
    for k, c in enumerate(chars):
        ds.add_strokes(c, render, pen.OCTOGRAM, k % 10)
    S, K, R, bg, feats, n = [], [], [], [], [], 0
    for k, c in enumerate(chars):
        keys, rows, b, f = pen.codify(pen.normalize(c, render), render, pen.OCTOGRAM, side)
        S += [k] * len(keys)
        K += list(keys)
        R += list(rows + n)
        bg.append(b + n)
        feats.append(f)
        n += len(f)
    want = ora.forward(len(chars), np.array(S, np.int32), np.array(K, np.int64), np.array(R, np.int32),
                       np.array(bg, np.int32), np.concatenate(feats), n,
                       np.array([k % 10 for k in range(len(chars))], np.int32))
    net.begin(ds, len(chars))
    assert net.next_batch()
    out = net.batch_outputs()
    assert_probabilities(out["probabilities"], ora.forward64(want))
    net.end()
    net.close()
