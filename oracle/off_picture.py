"""CPU restatement of the reference's OFF-mesh input front-end, for tests only.

Follows Off3DFormatPicture.cpp: mapToGridOFF (:5-8), drawTriangleOFF (:12-50),
OffSurfaceModelPicture::normalize (:73-82) and ::codifyInputData (:107-123).
Single-precision steps are taken with numpy float32 scalars in the reference's
order of operations.  random_rotation (:84-92) draws Q from Armadillo's QR of a
clock-seeded random matrix: parity unpinned (third-party routine, unpinned
version, unseedable RNG); the tests check what any such Q must satisfy.

Pins: two hand-computed triangles (tests/test_off_picture.py) and geometric
invariants (every voxel touches its triangle; the triangle is covered)."""
import numpy as np

f32 = np.float32


def map_to_grid(coord, side):
    # (int)(coord + 0.5 * side): float promoted to double, truncated toward zero, clamped
    return max(0, min(side - 1, int(float(coord) + 0.5 * side)))


def _steps(end):
    """0, 1, 2, ... then `end` itself (`x = min(x + 1, end) + (x == end)`)."""
    x = f32(0)
    while x <= end:
        yield x
        if x == end:
            break
        x = min(f32(x + f32(1)), end)


def draw_triangle(a, u, v, side):
    """Voxel keys in first-touch order of the triangle {a, a+u, a+v} (float32 triples)."""
    a = [f32(x) for x in a]
    u = [f32(x) for x in u]
    v = [f32(x) for x in v]
    with np.errstate(all="ignore"):
        base = f32(np.power(f32(f32(u[0] * u[0] + u[1] * u[1]) + u[2] * u[2]), f32(0.5)))
        u = [f32(x / base) for x in u]
        offset = f32(f32(u[0] * v[0] + u[1] * v[1]) + u[2] * v[2])
        v = [f32(v[k] - f32(offset * u[k])) for k in range(3)]
        height = f32(np.power(f32(f32(v[0] * v[0] + v[1] * v[1]) + v[2] * v[2]), f32(0.5)))
        v = [f32(x / height) for x in v]
        keys = []
        for h in _steps(height):
            length = f32(base * f32(f32(1) - f32(h / height)))
            for b in _steps(length):
                along = f32(b + f32(f32(offset * h) / height))
                p = [f32(f32(a[k] + f32(along * u[k])) + f32(h * v[k])) for k in range(3)]
                keys.append((map_to_grid(p[0], side) * side + map_to_grid(p[1], side)) * side + map_to_grid(p[2], side))
    return keys


def normalize(points, render_size):
    points = np.asarray(points, np.float64)
    lo, hi = points.min(0), points.max(0)
    scale = f32((hi - lo).max())
    factor = f32(f32(render_size) / scale)
    return (points - 0.5 * (lo + hi)) * float(factor)


def codify(points, triangles, side):
    """(keys in insertion order, rows, background row, features [rows x 1])."""
    points = np.asarray(points, np.float64)
    seen, order = set(), []
    for t in np.asarray(triangles).reshape(-1, 3):
        A, B, C = points[t[0]], points[t[1]], points[t[2]]
        for key in draw_triangle(A.astype(f32), (B - A).astype(f32), (C - A).astype(f32), side):
            if key not in seen:
                seen.add(key)
                order.append(key)
    n = len(order)
    feats = np.ones((n + 1, 1), np.float32)
    feats[0] = 0
    return np.array(order, np.int64), np.arange(1, n + 1, dtype=np.int32), 0, feats
