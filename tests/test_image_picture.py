"""Array-backed image front-end (OpenCVPicture without OpenCV) of the host library against
the oracle restatement and hand-computed images; MNIST / CIFAR-10 readers on files written
here.  CPU only, except the last test, which runs images through a 2-D net on the GPU."""
import os
import struct
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import image_picture as img  # noqa: E402
from gpu_util import assert_probabilities


def hostapi():
    from conftest import load_scn
    load_scn()
    from sparseconvnet_archived_amd import hostapi as h
    if not os.path.exists(h.LIB_PATH):
        pytest.skip("libscn_host.so is not built")
    return h


def one_image(pixels, bg, side, seed=-1, batch_type=None, jiggle=0):
    h = hostapi()
    pixels = np.asarray(pixels, np.float32)
    ch = 1 if pixels.ndim == 2 else pixels.shape[2]
    ds = h.Dataset("img", ch, 10, h.TESTBATCH if batch_type is None else batch_type)
    ds.add_image(pixels, bg, 3, jiggle)
    out = ds.codify(0, side, seed)
    ds.close()
    return out


def test_hand_computed_image():
    # 3 rows x 4 columns, background 0, field of side 8: the constructor's offsets are xOffset = -(3 // 2) = -1
    # (from the row count) and yOffset = -(4 // 2) = -2; pixel (column x, row y) lands in cell
    # (x - 1 + 4) * 8 + (y - 2 + 4).  Columns are the outer loop.
    px = np.zeros((3, 4), np.float32)
    px[1, 2] = 200  # x = 2, y = 1 -> 5 * 8 + 3
    px[0, 0] = 3    # x = 0, y = 0 -> 3 * 8 + 2   (|3 - 0| > 2)
    px[2, 0] = 2    # not more than 2 away from the background: not a site
    px[2, 3] = 255  # x = 3, y = 2 -> 6 * 8 + 4
    want_keys = [3 * 8 + 2, 5 * 8 + 3, 6 * 8 + 4]
    for keys, rows, bg, feats in (one_image(px, 0, 8), img.codify(px, 0, 8)):
        assert list(keys) == want_keys and list(rows) == [1, 2, 3] and bg == 0
        assert np.allclose(feats[:, 0], [0, 3 / 255, 200 / 255, 1.0], atol=1e-7)


def test_colour_scaling_and_any_channel():
    # background 128: divisor max(127, 128) = 128; background 200: divisor 200; a pixel is a site when ANY channel differs
    px = np.full((2, 2, 3), 128, np.float32)
    px[0, 1] = (128, 131, 128)
    px[1, 0] = (0, 128, 255)
    keys, rows, bg, feats = one_image(px, 128, 4)
    assert np.allclose(feats[1:], [[-1.0, 0.0, 127 / 128], [0.0, 3 / 128, 0.0]], atol=1e-7)  # column 0 first
    px2 = np.full((2, 2), 200, np.float32)
    px2[1, 1] = 0
    assert np.allclose(one_image(px2, 200, 4)[3][1:, 0], [-1.0])


def test_clipping_at_the_field():
    # a 6 x 6 image of ones in a field of side 4: offsets -3, so columns/rows 1..4 are inside
    px = np.full((6, 6), 9, np.float32)
    keys, rows, bg, feats = one_image(px, 0, 4)
    assert sorted(keys) == list(range(16)) and list(keys) == [x * 4 + y for x in range(4) for y in range(4)]
    assert list(keys) == list(img.codify(px, 0, 4)[0])


@pytest.mark.parametrize("seed,shape,bg,side", [(1, (28, 28), 0, 32), (2, (32, 32, 3), 128, 40), (3, (17, 9, 2), 77, 12),
                                                (4, (14, 10), 200, 16)])
def test_codify_matches_the_oracle_bit_for_bit(seed, shape, bg, side):
    rng = np.random.default_rng(seed)
    px = np.where(rng.random(shape) < 0.3, rng.integers(0, 256, shape), bg).astype(np.float32)
    keys, rows, b, feats = one_image(px, bg, side)
    want = img.codify(px, bg, side)
    assert list(keys) == list(want[0]) and list(rows) == list(want[1]) and b == 0
    assert np.array_equal(feats, want[3]) and len(keys) > 5


def test_distort_jiggles_training_pictures_only():
    h = hostapi()
    rng = np.random.default_rng(5)
    px = np.where(rng.random((12, 12)) < 0.4, 255, 0).astype(np.float32)
    plain = one_image(px, 0, 24)
    same = one_image(px, 0, 24, seed=7, jiggle=2)  # a test batch: unchanged
    assert list(plain[0]) == list(same[0])
    seen = set()
    for seed in range(12):
        moved = one_image(px, 0, 24, seed=seed, batch_type=h.TRAINBATCH, jiggle=2)
        d = np.unique(np.asarray(moved[0]) - np.asarray(plain[0]))
        assert len(d) == 1  # every site moved by the same (dx, dy)
        dx, dy = divmod(int(d[0]) + 2 * 24 + 2, 24)
        assert 0 <= dx <= 4 and 0 <= dy <= 4
        seen.add((dx, dy))
        assert np.array_equal(moved[3], plain[3])
    assert len(seen) > 3


def test_mnist_and_cifar_files(tmp_path):
    h = hostapi()
    rng = np.random.default_rng(6)
    images = rng.integers(0, 256, (5, 7, 6)).astype(np.uint8) * (rng.random((5, 7, 6)) < 0.5)
    labels = np.array([3, 1, 4, 1, 5], np.uint8)
    (tmp_path / "img").write_bytes(struct.pack(">iiii", 2051, 5, 7, 6) + images.astype(np.uint8).tobytes())
    (tmp_path / "lab").write_bytes(struct.pack(">ii", 2049, 5) + labels.tobytes())
    ds = h.Dataset("mnist", 1, 10)
    assert ds.add_mnist_files(tmp_path / "img", tmp_path / "lab") == 5 and len(ds) == 5
    for k in (0, 4):
        keys, rows, bg, feats = ds.codify(k, 12)
        want = img.codify(images[k].astype(np.float32), 0, 12)
        assert list(keys) == list(want[0]) and np.array_equal(feats, want[3])
    ds.close()
    ds = h.Dataset("mnist", 1, 10)
    with pytest.raises(IOError):
        ds.add_mnist_files(tmp_path / "img", tmp_path / "nothing")
    ds.close()
    # CIFAR-10: label byte, then 1024 red, 1024 green, 1024 blue; the picture holds blue, green, red
    rec = []
    planes = rng.integers(0, 256, (2, 3, 32, 32)).astype(np.uint8)
    for k in range(2):
        rec.append(bytes([k + 7]) + planes[k].tobytes())
    (tmp_path / "batch.bin").write_bytes(b"".join(rec))
    ds = h.Dataset("cifar", 3, 10)
    assert ds.add_cifar10_file(tmp_path / "batch.bin") == 2
    keys, rows, bg, feats = ds.codify(1, 36)
    bgr = np.stack([planes[1][2], planes[1][1], planes[1][0]], -1).astype(np.float32)  # [row y][column x][b, g, r]
    want = img.codify(bgr, 128, 36)
    assert list(keys) == list(want[0]) and np.array_equal(feats, want[3])
    ds.close()
    ds = h.Dataset("wrong", 1, 10)
    with pytest.raises(IOError):
        ds.add_cifar10_file(tmp_path / "batch.bin")  # three channels into one feature
    ds.close()
    # CIFAR-100: a coarse and a fine label byte, the fine one is the class
    (tmp_path / "c100.bin").write_bytes(b"".join(bytes([3, 40 + k]) + planes[k].tobytes() for k in range(2)))
    ds = h.Dataset("cifar100", 3, 100)
    assert ds.add_cifar100_file(tmp_path / "c100.bin") == 2
    assert [ds.label(k) for k in range(2)] == [40, 41]
    keys, rows, bg, feats = ds.codify(1, 36)
    assert list(keys) == list(want[0]) and np.array_equal(feats, want[3])
    ds.close()


@pytest.mark.gpu
def test_images_through_a_2d_net(scn):
    import oracle_net
    from sparseconvnet_archived_amd import hostapi as h, synthetic
    rng = np.random.default_rng(13)
    net = h.Net(2, 3, 10, threads=2)
    ora = oracle_net.Net(2, 3, 10)
    for n_ in (net, ora):
        n_.addLeNetLayerMP(32, 3, 1, 2, 2, synthetic.VLEAKYRELU)
        n_.addLeNetLayerMP(64, 2, 1, 2, 2, synthetic.VLEAKYRELU)
        n_.addTerminalPoolingLayer(2)
        n_.addSoftmaxLayer()
    for i, (W, B, pr) in synthetic.he_normal_weights(net.layers(), 5).items():
        net.set_weights(i, W, B, pr)
        ora.set_weights(i, W, B, pr)
    side = net.inputSpatialSize
    ds = h.Dataset("images", 3, 10, h.TESTBATCH)
    pics = []
    for k in range(6):
        shape = (side - 2, side - 2, 3)
        px = np.where(rng.random(shape) < 0.35, rng.integers(0, 256, shape), 128).astype(np.float32)
        pics.append(px)
        ds.add_image(px, 128, k)
    S, K, R, bg, feats, n = [], [], [], [], [], 0
    for k, px in enumerate(pics):
        keys, rows, b, f = img.codify(px, 128, side)
        S += [k] * len(keys)
        K += list(keys)
        R += list(rows + n)
        bg.append(b + n)
        feats.append(f)
        n += len(f)
    want = ora.forward(len(pics), np.array(S, np.int32), np.array(K, np.int64), np.array(R, np.int32),
                       np.array(bg, np.int32), np.concatenate(feats), n, np.arange(len(pics), dtype=np.int32))
    net.begin(ds, len(pics))
    assert net.next_batch()
    out = net.batch_outputs()
    assert_probabilities(out["probabilities"], ora.forward64(want))
    net.end()
    net.close()
