"""Seeded synthetic inputs for the benchmark configurations.

Every generator draws from numpy.random.Generator(PCG64(seed)) and returns
int64 coordinates [n, dim+1] (last column = sample index) in the layout
InputLayer takes.  Points are returned in shuffled order unless order="scan":
a voxelised point cloud reaches the library in no particular order, so nothing
downstream may rely on neighbouring rows being neighbouring sites.
"""
import numpy as np


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _unique_rows(a):
    """Deduplicate keeping first occurrences, preserving order."""
    _, idx = np.unique(a, axis=0, return_index=True)
    return a[np.sort(idx)]


def _rect(axis, pos, lo, hi):
    """All voxels of the axis-aligned rectangle {x[axis]=pos, lo<=others<hi}."""
    others = [d for d in range(3) if d != axis]
    u = np.arange(lo[0], hi[0])
    v = np.arange(lo[1], hi[1])
    uu, vv = np.meshgrid(u, v, indexing="ij")
    out = np.empty((uu.size, 3), np.int64)
    out[:, axis] = pos
    out[:, others[0]] = uu.ravel()
    out[:, others[1]] = vv.ravel()
    return out


def _box_surface(lo, hi):
    """One-voxel-thick surface of the box [lo, hi] (inclusive corners)."""
    faces = []
    for axis in range(3):
        others = [d for d in range(3) if d != axis]
        l2 = (lo[others[0]], lo[others[1]])
        h2 = (hi[others[0]] + 1, hi[others[1]] + 1)
        faces.append(_rect(axis, lo[axis], l2, h2))
        faces.append(_rect(axis, hi[axis], l2, h2))
    return np.concatenate(faces, 0)


def _finish(pts, spatial, batch_idx, rng, order):
    pts = pts[((pts >= 0) & (pts < spatial)).all(1)]
    pts = _unique_rows(pts)
    if order == "shuffled":
        pts = pts[rng.permutation(len(pts))]
    b = np.full((len(pts), 1), batch_idx, np.int64)
    return np.concatenate([pts, b], 1)


def shells_and_planes(seed, spatial=128, target=40000, batch_idx=0, order="shuffled"):
    """One sample of the single-layer configuration: 4-8 voxelised sphere shells and
    axis-aligned rectangles in a spatial^3 grid, about `target` distinct sites."""
    rng = _rng(seed)
    parts = []
    for _ in range(int(rng.integers(4, 9))):
        c = rng.uniform(0.19 * spatial, 0.81 * spatial, 3)
        r = rng.uniform(0.06 * spatial, 0.31 * spatial)
        n = int(40 * r * r)
        u = rng.normal(size=(n, 3))
        u /= np.linalg.norm(u, axis=1, keepdims=True)
        parts.append(np.rint(c + r * u).astype(np.int64))
    for _ in range(int(rng.integers(2, 5))):
        axis = int(rng.integers(0, 3))
        pos = int(rng.integers(0, spatial))
        lo = rng.integers(0, spatial // 2, 2)
        hi = lo + rng.integers(spatial // 4, spatial // 2, 2)
        parts.append(_rect(axis, pos, lo, hi))
    pts = np.concatenate(parts, 0)
    pts = pts[((pts >= 0) & (pts < spatial)).all(1)]
    pts = _unique_rows(pts)
    while len(pts) < target:  # extend with further rectangles
        axis = int(rng.integers(0, 3))
        pos = int(rng.integers(0, spatial))
        lo = rng.integers(0, spatial // 2, 2)
        hi = lo + rng.integers(spatial // 4, spatial // 2, 2)
        pts = _unique_rows(np.concatenate([pts, _rect(axis, pos, lo, hi)], 0))
        pts = pts[((pts >= 0) & (pts < spatial)).all(1)]
    pts = pts[:target]
    return _finish(pts, spatial, batch_idx, rng, order)


def config1(seed=1000, batch=2, spatial=128, target=40000, order="shuffled"):
    """Batch of shells_and_planes samples: coords [N, 4]."""
    return np.concatenate([shells_and_planes(seed + b, spatial, target, b, order)
                           for b in range(batch)], 0)


def _line(p, q):
    """Integer points of a 1-pixel-wide segment p->q (Bresenham-style DDA)."""
    n = int(max(abs(q[0] - p[0]), abs(q[1] - p[1]))) + 1
    t = np.linspace(0.0, 1.0, n)
    return np.stack([np.rint(p[0] + (q[0] - p[0]) * t), np.rint(p[1] + (q[1] - p[1]) * t)],
                    1).astype(np.int64)


def strokes2d(seed=2000, batch=100, canvas=64, spatial=71):
    """2-D pen strokes: per sample 3-10 polylines of 3-6 vertices (steps of at most 12 pixels), one pixel wide, drawn in a
    canvas x canvas window centred in a spatial x spatial grid.  Returns coords [N, 3] grouped
    by sample."""
    out = []
    off = (spatial - canvas) // 2
    for b in range(batch):
        rng = _rng(seed + b)
        pts = []
        for _ in range(int(rng.integers(3, 11))):
            nv = int(rng.integers(3, 7))
            steps = rng.integers(-12, 13, (nv, 2))
            steps[0] = rng.integers(0, canvas, 2)
            v = np.clip(np.cumsum(steps, 0), 0, canvas - 1)
            for a, c in zip(v[:-1], v[1:]):
                pts.append(_line(a, c))
        p = _unique_rows(np.concatenate(pts, 0)) + off
        out.append(np.concatenate([p, np.full((len(p), 1), b, np.int64)], 1))
    return np.concatenate(out, 0)


def room_scene(seed=3000, target=1000000, spatial=4096, n_boxes=50, batch_idx=0,
               order="shuffled", duplicate_fraction=0.0):
    """A room made of one-voxel-thick surfaces: a floor, 2-4 walls and the surfaces of
    `n_boxes` random boxes standing on the floor, scaled so that it has exactly `target`
    distinct sites (when the grid is large enough).  With duplicate_fraction > 0 that share of
    extra points repeats existing sites (for the InputLayer modes that merge duplicates)."""
    rng = _rng(seed)
    # draw the shape parameters once, in units of the floor side, then search the scale
    n_walls = int(rng.integers(2, 5))
    wall_h = rng.uniform(0.25, 0.4, n_walls)
    box_c = rng.uniform(0.08, 0.92, (n_boxes, 2))
    box_s = rng.uniform(0.03, 0.14, (n_boxes, 3))

    def build(side):
        o = (spatial - side) // 2
        z0 = max(1, (spatial - int(0.4 * side)) // 2)
        parts = [_rect(2, z0, (o, o), (o + side, o + side))]
        walls = [(0, o), (1, o), (0, o + side - 1), (1, o + side - 1)]
        for w in range(n_walls):
            axis, pos = walls[w]
            h = max(2, int(wall_h[w] * side))
            if axis == 0:  # others = (1, 2)
                parts.append(_rect(0, pos, (o, z0), (o + side, z0 + h)))
            else:  # axis 1, others = (0, 2)
                parts.append(_rect(1, pos, (o, z0), (o + side, z0 + h)))
        for b in range(n_boxes):
            s = np.maximum(2, (box_s[b] * side).astype(np.int64))
            c = o + (box_c[b] * side).astype(np.int64)
            lo = np.array([c[0] - s[0] // 2, c[1] - s[1] // 2, z0 + 1])
            hi = lo + s
            parts.append(_box_surface(lo, hi))
        pts = np.concatenate(parts, 0)
        pts = pts[((pts >= 0) & (pts < spatial)).all(1)]
        return _unique_rows(pts)

    side = int(min(spatial - 2, max(8, np.sqrt(target / 2.2))))
    pts = build(side)
    for _ in range(12):
        if len(pts) >= target and len(pts) <= 1.03 * target:
            break
        new_side = int(side * np.sqrt(1.015 * target / max(1, len(pts))))
        new_side = int(min(spatial - 2, max(8, new_side if new_side != side else side + 1)))
        if new_side == side:
            break
        side = new_side
        pts = build(side)
    pts = pts[:target]
    out = _finish(pts, spatial, batch_idx, rng, order)
    if duplicate_fraction > 0:
        extra = out[rng.integers(0, len(out), int(duplicate_fraction * len(out)))]
        out = np.concatenate([out, extra], 0)
        out = out[rng.permutation(len(out))]
    return out


def scene_batch(seed, batch, target, spatial=4096, n_boxes=50, order="shuffled",
                duplicate_fraction=0.0):
    return np.concatenate([room_scene(seed + b, target, spatial, n_boxes, b, order,
                                      duplicate_fraction) for b in range(batch)], 0)
