"""CPU restatement of the reference's pen-stroke front-end (OnlineHandwritingPicture),
TEST INFRASTRUCTURE ONLY: nothing in the product imports this file.

Follows /root/reference/SparseConvNet/OnlineHandwritingPicture.cpp line by line with
numpy scalars of the widths the reference computes in (arma::mat is double; lengths,
alpha, direction and features are float):
  normalize       OnlineHandwritingPicture.cpp:9-25
  constant_speed  OnlineHandwritingPicture.cpp:27-53
  codify          OnlineHandwritingPicture.cpp:77-271 (Simple, Octogram, UndirectedOctogram,
                  SpaceTime3d, VectorSpaceTime3d)
Pins (tests/test_pen_strokes.py): hand-computed characters for every encoding (cell
membership, truncation of negative coordinates toward zero, direction weights at an
angle of pi/8, time axis of the 3-D encodings), closed forms of constant_speed on
straight strokes, invariants on polylines.
The LogSignature encodings are not restated (they need the reference's basis tables,
signature.h:96-514): parity unpinned, and the product refuses them.
distort() draws from std::mt19937 through the reference's RNG class, whose stream is
not restated here: parity unpinned; the tests check what any draw must satisfy.
"""
import numpy as np

f32 = np.float32
SIMPLE, OCTOGRAM, UNDIRECTED_OCTOGRAM, SPACETIME3D, VECTOR_SPACETIME3D = 0, 1, 2, 7, 8
ENCODING_FEATURES = {0: 1, 1: 8, 2: 4, 7: 1, 8: 3}


def normalize(strokes, renderSize):
    strokes = [np.asarray(s, np.float64).reshape(-1, 2) for s in strokes]
    allp = np.concatenate(strokes)
    lo, hi = allp.min(0), allp.max(0)
    scale = f32((hi - lo).max())
    assert scale > 0
    factor = f32(renderSize) / scale  # int / float -> float
    mid = 0.5 * (lo + hi)
    return [(s - mid) * np.float64(factor) for s in strokes]


def constant_speed(stroke, density, multiplier=1):
    stroke = np.asarray(stroke, np.float64).reshape(-1, 2)
    rows = len(stroke)
    density = f32(density)
    lengths = np.zeros(rows, f32)
    for i in range(1, rows):
        d = stroke[i] - stroke[i - 1]
        lengths[i] = f32(np.float64(lengths[i - 1]) + np.sqrt(d[0] ** 2 + d[1] ** 2))
    lTotal = lengths[rows - 1]
    n = int(0.5 + np.float64(lTotal / density)) * multiplier
    r = np.zeros((n + 1, 2), np.float64)
    r[0] = stroke[0]
    j = 0
    for i in range(1, n + 1):
        while j + 2 < rows and f32(n) * lengths[j + 1] < f32(i) * lTotal:
            j += 1
        alpha = (lengths[j + 1] - f32(i) * lTotal / f32(n)) / (lengths[j + 1] - lengths[j])
        a = np.float64(alpha)
        b = np.float64(f32(1) - alpha)
        r[i] = stroke[j] * a + stroke[j + 1] * b
    return r


def codify(strokes, renderSize, enc, spatialSize, penSpeed3d=0.02, offset3d=0.0):
    """(keys in insertion order, rows, background row, features [rows x nFeatures])."""
    nF = ENCODING_FEATURES[enc]
    S = spatialSize
    penSpeed3d, offset3d = f32(penSpeed3d), f32(offset3d)
    piBy4 = f32(3.1415926536 / 4)
    rows_of = {}
    feats = [np.zeros(nF, f32)]  # background row 0
    keys = []
    csp = [constant_speed(s, 0.1) for s in strokes]
    total = sum(len(c) for c in csp)
    volume = enc in (SPACETIME3D, VECTOR_SPACETIME3D)
    direction = enc in (OCTOGRAM, UNDIRECTED_OCTOGRAM, VECTOR_SPACETIME3D)
    z = 0
    with np.errstate(invalid="ignore", divide="ignore"):
        for c in csp:
            last = len(c) - 1 if direction else len(c)
            for j in range(last):
                a0 = int(c[j, 0] + S / 2.0)  # truncation toward zero, as the C conversion
                a1 = int(c[j, 1] + S / 2.0)
                n = a0 * S + a1
                inside = 0 <= a0 < S and 0 <= a1 < S
                if volume:
                    t = f32(z - total // 2) * penSpeed3d + offset3d
                    a2 = int(f32(renderSize) * t + f32(S // 2))
                    z += 1
                    inside = inside and 0 <= a2 < S
                    n = n * S + a2
                if not inside:
                    continue
                if n not in rows_of:
                    rows_of[n] = len(feats)
                    keys.append(n)
                    feats.append(np.zeros(nF, f32))
                f = feats[rows_of[n]]
                if enc in (SIMPLE, SPACETIME3D):
                    f[0] += f32(1)
                    continue
                dx = f32(c[j + 1, 0] - c[j, 0])
                dy = f32(c[j + 1, 1] - c[j, 1])
                m = f32(np.sqrt(f32(dx * dx + dy * dy)))
                dx, dy = f32(dx / m), f32(dy / m)
                if enc == VECTOR_SPACETIME3D:
                    f[0] += f32(1)
                    f[1] += dx
                    f[2] += dy
                    continue
                for k in range(8 if enc == OCTOGRAM else 4):
                    ang = f32(k) * piBy4
                    dot = f32(f32(np.cos(ang)) * dx) + f32(f32(np.sin(ang)) * dy)
                    if enc == UNDIRECTED_OCTOGRAM:
                        dot = np.abs(dot)
                    alpha = f32(1) - f32(np.arccos(f32(dot))) / piBy4
                    if alpha > 0:
                        f[k] += f32(alpha)
    keys = np.array(keys, np.int64)
    return keys, np.arange(1, len(keys) + 1, dtype=np.int32), 0, np.stack(feats)
