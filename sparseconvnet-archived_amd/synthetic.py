"""Seeded synthetic sparse lattices, weights and the five benchmark stacks.

Everything is generated on the host from one seed with numpy's PCG64 and fed
unchanged to whichever implementation is under test, so the GPU path and the
CPU oracle always see identical inputs and weights.
"""
import numpy as np

RELU, VLEAKYRELU, LEAKYRELU, TANH, SOFTMAX, PRELU, SIGMOID = 1, 2, 3, 4, 5, 6, 7


# --------------------------------------------------------------- site patterns
def strokes(rng, size, target, dimension=2):
    """Pen-stroke-like pattern: a few random walks with momentum, unique sites,
    about `target` of them, inside a size^dimension lattice."""
    seen, out = set(), []
    n_strokes = int(rng.integers(3, 6))
    per = max(1, target // n_strokes)
    for s in range(n_strokes):
        pos = rng.uniform(0.15 * size, 0.85 * size, dimension)
        ang = rng.uniform(0, 2 * np.pi)
        got = 0
        budget = (target - len(out)) if s == n_strokes - 1 else per
        guard = 0
        while got < budget and guard < 50 * budget:
            guard += 1
            ang += rng.normal(0, 0.35)
            step = np.array([np.cos(ang), np.sin(ang)] + [0.0] * (dimension - 2))
            pos = pos + step
            for a in range(dimension):  # bounce off the border
                if pos[a] < 0 or pos[a] > size - 1:
                    pos[a] = min(max(pos[a], 0), size - 1)
                    ang += np.pi / 2
            c = tuple(int(round(x)) for x in pos)
            if c not in seen:
                seen.add(c)
                out.append(c)
                got += 1
    return np.array(out, np.int32).reshape(-1, dimension)


def mesh_voxels(rng, size, kind=None):
    """Voxels on the surface of a sphere, torus or perturbed ellipsoid that
    fills most of a size^3 lattice (about 2 % of the sites at size 40)."""
    kind = int(rng.integers(0, 3)) if kind is None else kind
    n = 60000
    u = rng.uniform(0, 2 * np.pi, n)
    v = rng.uniform(0, 2 * np.pi, n)
    c = (size - 1) / 2.0
    if kind == 0:  # sphere
        r = size * rng.uniform(0.22, 0.27)
        w = np.arccos(rng.uniform(-1, 1, n))
        p = np.stack([r * np.sin(w) * np.cos(u), r * np.sin(w) * np.sin(u), r * np.cos(w)], 1)
    elif kind == 1:  # torus
        R, r = size * rng.uniform(0.24, 0.3), size * rng.uniform(0.07, 0.1)
        p = np.stack([(R + r * np.cos(v)) * np.cos(u), (R + r * np.cos(v)) * np.sin(u), r * np.sin(v)], 1)
    else:  # perturbed ellipsoid
        ax = size * rng.uniform(0.15, 0.33, 3)
        w = np.arccos(rng.uniform(-1, 1, n))
        bump = 1 + 0.12 * np.sin(3 * u + rng.uniform(0, 6)) * np.sin(2 * w)
        p = np.stack([ax[0] * np.sin(w) * np.cos(u), ax[1] * np.sin(w) * np.sin(u), ax[2] * np.cos(w)], 1) * bump[:, None]
    # random rotation
    q, _ = np.linalg.qr(rng.standard_normal((3, 3)))
    p = p @ q.T + c
    vox = np.clip(np.rint(p), 0, size - 1).astype(np.int32)
    _, first = np.unique(vox, axis=0, return_index=True)
    return vox[np.sort(first)]  # raster order of the surface sampling, like a mesh renderer


def dense_block(size, block):
    lo = (size - block) // 2
    g = np.arange(lo, lo + block, dtype=np.int32)
    a, b = np.meshgrid(g, g, indexing="ij")
    return np.stack([a.ravel(), b.ravel()], 1)


def moving_blobs(rng, size, target):
    """Blobs moving along smooth random trajectories; axis 0 is time."""
    pts = []
    n_blobs = 6
    per_t = max(1.0, target / (n_blobs * size))
    radius = (3 * per_t / (4 * np.pi)) ** (1 / 3.0) if per_t > 4 else 1.0
    rr = int(np.ceil(radius)) + 1
    offs = np.array([(a, b) for a in range(-rr, rr + 1) for b in range(-rr, rr + 1)], np.int32)
    for _ in range(n_blobs):
        pos = rng.uniform(0.2 * size, 0.8 * size, 2)
        vel = rng.normal(0, 0.6, 2)
        for t in range(size):
            vel = 0.9 * vel + rng.normal(0, 0.25, 2)
            pos = np.clip(pos + vel, rr, size - 1 - rr)
            d2 = ((offs + np.rint(pos) - pos) ** 2).sum(1)
            # a disc per time step: the blob's trace through (t, y, x)
            keep = offs[d2 <= radius * radius * 2.2]
            c = np.rint(pos).astype(np.int32) + keep
            pts.append(np.concatenate([np.full((len(c), 1), t, np.int32), c], 1))
    p = np.concatenate(pts, 0)
    _, first = np.unique(p, axis=0, return_index=True)
    return p[np.sort(first)]


# --------------------------------------------------------------------- configs
class Config:
    def __init__(self, name, dimension, nInputFeatures, nClasses, batch, lattice, stack, headless_top=None):
        self.name, self.dimension, self.nInputFeatures, self.nClasses = name, dimension, nInputFeatures, nClasses
        self.batch, self.lattice, self.stack, self.headless_top = batch, lattice, stack, headless_top

    def build(self, net):
        """Apply the builder calls to anything with the reference's builder API."""
        for call in self.stack:
            getattr(net, call[0])(*call[1:])
        if self.headless_top is not None:
            net.finishHeadless(self.headless_top)
        return net


def config(n, batch=None):
    if n == 1:
        c = Config("c1_single_conv_2d", 2, 32, 1, 16, 64, [("addLeNetLayerMP", 64, 3, 1, 1, 1, RELU)], headless_top=62)
    elif n == 2:
        stack = [("addLeNetLayerMP", 32 * (l + 1), 2, 1, 3, 2, RELU) for l in range(5)]
        stack += [("addLeNetLayerMP", 192, 1, 1, 1, 1, PRELU), ("addTerminalPoolingLayer", 2), ("addSoftmaxLayer",)]
        c = Config("c2_sparse_net_2d", 2, 3, 100, 100, 96, stack)
    elif n == 3:
        stack = [("addLeNetLayerMP", f, 2, 1, 2, 2, RELU) for f in (32, 64, 96, 128)]
        stack += [("addLeNetLayerMP", 128, 1, 1, 1, 1, PRELU), ("addTerminalPoolingLayer", 2), ("addSoftmaxLayer",)]
        c = Config("c3_voxel_net_3d", 3, 1, 40, 32, 40, stack)
    elif n == 4:
        stack = [("addLeNetLayerMP", 160 * (l + 1), 2, 1, 2, 2, RELU) for l in range(5)]
        stack += [("addLeNetLayerMP", 800, 1, 1, 1, 1, RELU), ("addTerminalPoolingLayer", 3), ("addSoftmaxLayer",)]
        c = Config("c4_wide_gemm_2d", 2, 3, 100, 128, 126, stack)
    elif n == 5:
        stack = [("addLeNetLayerMP", 64, 3, 1, 1, 1, RELU), ("addLeNetLayerMP", 64, 3, 1, 2, 2, RELU)]
        c = Config("c5_spatiotemporal_3d", 3, 64, 1, 96, 128, stack, headless_top=62)
    else:
        raise ValueError(n)
    c.number = n
    if batch is not None:
        c.batch = batch
    return c


def make_samples(cfg, seed, batch=None):
    """list of (coords [n x d] int32 in the cfg.lattice frame, features [n x C] float32, label)."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(batch or cfg.batch):
        if cfg.number == 1:
            pts = strokes(rng, cfg.lattice, int(rng.integers(300, 360)))
            f = rng.uniform(-1, 1, (len(pts), 32))
        elif cfg.number == 2:
            pts = strokes(rng, cfg.lattice, int(rng.integers(280, 460)))
            f = rng.uniform(-1, 1, (len(pts), 3))
        elif cfg.number == 3:
            pts = mesh_voxels(rng, cfg.lattice)
            f = np.ones((len(pts), 1))
        elif cfg.number == 4:
            pts = dense_block(cfg.lattice, 32)
            f = rng.standard_normal((len(pts), 3))
        else:
            pts = moving_blobs(rng, cfg.lattice, 10400)
            f = rng.uniform(-1, 1, (len(pts), 64))
        label = int(rng.integers(0, max(cfg.nClasses, 1)))
        out.append((np.ascontiguousarray(pts, np.int32), f.astype(np.float32), label))
    return out


def he_normal_weights(layers, seed):
    """{layer index: (W [K x N], B [N], prelu [N] or None)} for the NiN layers:
    W ~ N(0, 2/K), zero bias, slopes 0.25."""
    rng = np.random.default_rng(seed)
    out = {}
    for i, l in enumerate(layers):
        if l["kind"] not in ("nin", "nin_prelu"):
            continue
        K, N = l["nIn"], l["nOut"]
        W = (rng.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
        B = np.zeros(N, np.float32)
        pr = np.full(N, 0.25, np.float32) if l["kind"] == "nin_prelu" else None
        out[i] = (W, B, pr)
    return out


def codify(samples, dimension, lattice, spatialSize, nFeatures):
    """What BatchProducer + SparsePointsPicture::codifyInputData produce for a
    batch: flat (sample, key, row), backgroundCol per sample, the feature
    matrix [nSpatialSites x nFeatures] and nSpatialSites."""
    shift = int((spatialSize - lattice) / 2)  # toward zero, as the C++ division
    S, K, R, bg, feats = [], [], [], [], []
    n = 0
    for i, (pts, f, _) in enumerate(samples):
        feats.append(np.zeros((1, nFeatures), np.float32))
        bg.append(n)
        n += 1
        c = pts.astype(np.int64) + shift
        inside = np.all((c >= 0) & (c < spatialSize), 1)
        key = np.zeros(len(c), np.int64)
        for a in range(dimension):
            key = key * spatialSize + c[:, a]
        # first occurrence of every key among the points inside the field (a point outside has a key that
        # aliases some other cell's: it must not stand in for that cell)
        idx = np.flatnonzero(inside)
        _, first = np.unique(key[idx], return_index=True)
        keep = np.zeros(len(c), bool)
        keep[idx[first]] = True
        k = key[keep]
        S.append(np.full(len(k), i, np.int32))
        K.append(k)
        R.append(np.arange(n, n + len(k), dtype=np.int32))
        n += len(k)
        feats.append(f[keep])
    return (np.concatenate(S), np.concatenate(K), np.concatenate(R), np.array(bg, np.int32),
            np.concatenate(feats, 0).astype(np.float32), n)
