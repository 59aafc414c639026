"""OFF-mesh front-end (OffSurfaceModelPicture) of the host library against the
oracle restatement, hand-computed triangles and geometric invariants.  CPU only,
except the last test, which runs meshes through a 3-D net on the GPU."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import off_picture as off  # noqa: E402
from gpu_util import assert_probabilities


def hostapi():
    from conftest import load_scn
    load_scn()
    from sparseconvnet_archived_amd import hostapi as h
    if not os.path.exists(h.LIB_PATH):
        pytest.skip("libscn_host.so is not built")
    return h


def one_mesh(points, triangles, side, render=8, seed=-1):
    h = hostapi()
    ds = h.Dataset("mesh", 1, 2)
    ds.add_mesh(points, triangles, render, 0)
    out = ds.codify(0, side, seed)
    ds.close()
    return out


def unkey(keys, side):
    keys = np.asarray(keys)
    return np.stack([keys // (side * side), (keys // side) % side, keys % side], 1)


def test_hand_computed_right_triangle():
    # a = 0, u = (3,0,0), v = (0,2,0), lattice of side 8 (origin at voxel 4):
    # rows h = 0, 1, 2 of length 3, 1.5, 0 sampled at unit steps plus the end point
    pts = [(0, 0, 0), (3, 0, 0), (0, 2, 0)]
    want = [(4, 4, 4), (5, 4, 4), (6, 4, 4), (7, 4, 4), (4, 5, 4), (5, 5, 4), (4, 6, 4)]
    want_keys = [(x * 8 + y) * 8 + z for x, y, z in want]
    assert off.draw_triangle(pts[0], pts[1], pts[2], 8)[:4] == want_keys[:4]
    keys, rows, bg, feats = one_mesh(pts, [(0, 1, 2)], 8)
    assert list(keys) == want_keys
    assert list(rows) == list(range(1, 8)) and bg == 0
    assert feats.shape == (8, 1) and feats[0, 0] == 0 and np.all(feats[1:] == 1)
    o = off.codify(pts, [(0, 1, 2)], 8)
    assert list(o[0]) == want_keys


def test_hand_computed_skewed_triangle_with_clamping():
    # a = (-5,0,0), u = (0,0,2.5), v = (0,1,1): u.v = 1, height 1; x = -5 lies outside a lattice of side 6
    # and is clamped onto its face.  h = 0: z = 0, 1, 2, 2.5 -> voxels z = 3, 4, 5, 5; h = 1: the apex (-5,1,1)
    pts = [(-5, 0, 0), (-5, 0, 2.5), (-5, 1, 1)]
    want = [(0, 3, 3), (0, 3, 4), (0, 3, 5), (0, 4, 4)]
    want_keys = [(x * 6 + y) * 6 + z for x, y, z in want]
    keys, rows, bg, feats = one_mesh(pts, [(0, 1, 2)], 6)
    assert list(keys) == want_keys
    assert list(off.codify(pts, [(0, 1, 2)], 6)[0]) == want_keys


def random_mesh(rng, nPoints, nTriangles, spread):
    pts = rng.uniform(-spread, spread, (nPoints, 3))
    tris = np.stack([rng.choice(nPoints, 3, replace=False) for _ in range(nTriangles)])
    return pts, tris.astype(np.int32)


@pytest.mark.parametrize("seed,side,spread", [(1, 16, 6.0), (2, 24, 14.0), (3, 40, 18.0), (4, 12, 9.0)])
def test_codify_matches_the_oracle_bit_for_bit(seed, side, spread):
    rng = np.random.default_rng(seed)
    pts, tris = random_mesh(rng, 30, 40, spread)
    keys, rows, bg, feats = one_mesh(pts, tris, side)
    okeys, orows, obg, ofeats = off.codify(pts, tris, side)
    assert np.array_equal(keys, okeys) and np.array_equal(rows, orows) and bg == obg
    assert np.array_equal(feats, ofeats)


def test_every_voxel_touches_its_triangle_and_the_triangle_is_covered():
    rng = np.random.default_rng(7)
    side = 32
    for _ in range(20):
        P = rng.uniform(-12, 12, (3, 3))
        keys, _, _, _ = one_mesh(P, [(0, 1, 2)], side)
        vox = unkey(keys, side)
        centres = vox + 0.5 - side / 2.0
        # dense barycentric sampling of the triangle
        w = rng.dirichlet((1, 1, 1), 4000)
        samples = w @ P
        d = np.sqrt(((centres[:, None, :] - samples[None, :, :]) ** 2).sum(-1))
        assert d.min(1).max() <= 1.2  # a voxel holds a point of the triangle (up to the sampling density)
        svox = np.floor(samples + side / 2.0).astype(int)
        have = {tuple(v) for v in vox}
        # the net has unit spacing: every point of the triangle is within one step of a drawn voxel
        miss = [s for s in svox if not any((s[0] + a, s[1] + b, s[2] + c) in have
                                           for a in (-1, 0, 1) for b in (-1, 0, 1) for c in (-1, 0, 1))]
        assert not miss


def test_normalize_fits_the_render_cube():
    rng = np.random.default_rng(9)
    pts, tris = random_mesh(rng, 50, 60, 3.0)
    pts[:, 0] *= 5  # longest along x
    n = off.normalize(pts, 20)
    ext = n.max(0) - n.min(0)
    assert abs(ext.max() - 20) < 1e-4 and np.allclose(n.max(0) + n.min(0), 0, atol=1e-9)
    # through distort (rotation + normalize): the drawn voxels span the render cube in some axis, and never more
    keys, _, _, _ = one_mesh(pts, tris, 40, render=20, seed=5)
    vox = unkey(keys, 40)
    span = vox.max(0) - vox.min(0)
    assert 19 <= span.max() <= 21
    # a different seed is a different rotation, the same seed the same one
    again = one_mesh(pts, tris, 40, render=20, seed=5)[0]
    other = one_mesh(pts, tris, 40, render=20, seed=6)[0]
    assert np.array_equal(again, keys) and not np.array_equal(other, keys)


def test_off_files(tmp_path):
    h = hostapi()
    path = tmp_path / "tetra.off"
    path.write_text("OFF\n4 4 6\n0 0 0\n6 0 0\n0 6 0\n0 0 6\n3 0 1 2\n3 0 1 3\n3 0 2 3\n3 1 2 3\n")
    ds = h.Dataset("off", 1, 2)
    ds.add_off_file(path, 10, 1)
    pts = [(0, 0, 0), (6, 0, 0), (0, 6, 0), (0, 0, 6)]
    tris = [(0, 1, 2), (0, 1, 3), (0, 2, 3), (1, 2, 3)]
    ds.add_mesh(pts, tris, 10, 1)
    a, b = ds.codify(0, 16), ds.codify(1, 16)
    assert all(np.array_equal(x, y) for x, y in zip(a[:2], b[:2])) and len(a[0]) > 20
    assert np.array_equal(a[0], off.codify(pts, tris, 16)[0])
    bad = tmp_path / "bad.off"
    bad.write_text("OFF\n3 1 0\n0 0 0\n1 0 0\n")
    with pytest.raises(IOError):
        ds.add_off_file(bad, 10)
    with pytest.raises(IOError):
        ds.add_off_file(tmp_path / "missing.off", 10)
    ds.close()


@pytest.mark.gpu
def test_meshes_through_a_3d_net(scn):
    """Meshes through a small 3-D net.  The voxels codify() produced for the
    unrotated meshes, fed as plain points, must give the oracle's probabilities;
    the mesh pictures themselves (rotated by distort(), as the reference does
    for every batch type) must run end to end."""
    import oracle_net
    from sparseconvnet_archived_amd import hostapi as h, synthetic
    rng = np.random.default_rng(11)
    net = h.Net(3, 1, 5, threads=2)
    ora = oracle_net.Net(3, 1, 5)
    for n_ in (net, ora):
        n_.addLeNetLayerMP(32, 2, 1, 2, 2, synthetic.RELU)
        n_.addLeNetLayerMP(64, 2, 1, 2, 2, synthetic.RELU)
        n_.addTerminalPoolingLayer(2)
        n_.addSoftmaxLayer()
    for i, (W, B, pr) in synthetic.he_normal_weights(net.layers(), 3).items():
        net.set_weights(i, W, B, pr)
        ora.set_weights(i, W, B, pr)
    side = net.inputSpatialSize
    ds = h.Dataset("meshes", 1, 5, h.TESTBATCH)
    meshes = []
    for k in range(6):
        pts, tris = random_mesh(rng, 12, 14, 0.4 * side)
        meshes.append((pts, tris))
        ds.add_mesh(pts, tris, side, k % 5)
    # the oracle's input: every picture codified on the CPU, rows renumbered batch-globally
    S, K, R, bg, feats, n = [], [], [], [], [], 0
    for k, (pts, tris) in enumerate(meshes):
        keys, rows, b, f = off.codify(pts, tris, side)
        S += [k] * len(keys)
        K += list(keys)
        R += list(rows + n)
        bg.append(b + n)
        feats.append(f)
        n += len(f)
    want = ora.forward(len(meshes), np.array(S, np.int32), np.array(K, np.int64), np.array(R, np.int32),
                       np.array(bg, np.int32), np.concatenate(feats), n, np.array([k % 5 for k in range(6)], np.int32))
    ds2 = h.Dataset("points", 1, 5, h.TESTBATCH)
    for k, (pts, tris) in enumerate(meshes):
        keys, rows, b, f = off.codify(pts, tris, side)
        ds2.add_points(3, side, unkey(keys, side), f[1:], k % 5)
    net.begin(ds2, len(meshes))
    assert net.next_batch()
    out = net.batch_outputs()
    assert_probabilities(out["probabilities"], ora.forward64(want))
    net.end()
    # the mesh pictures themselves: a probability row per mesh
    net.begin(ds, len(meshes))
    assert net.next_batch()
    out = net.batch_outputs()
    assert out["probabilities"].shape == (6, 5) and np.allclose(out["probabilities"].sum(1), 1, atol=1e-4)
    net.end()
    net.close()
