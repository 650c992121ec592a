"""Seeded synthetic inputs for the benchmark configurations: point clouds
sampled on the surfaces of random axis-aligned boxes and ellipsoids, with
Gaussian noise, inside [-1, 1]^3.  NumPy only, so the same seed gives the same
clouds on any machine."""
import numpy as np

CONFIGS = {
    # name: batch, points per cloud, grid, Rs_in, Rs_out, kernel, stride, padding, rotate, shapes
    "cfg1": dict(batch=2, points=1024, grid=32, mult_in=2, mult_out=2, lmax=3, kernel=3, stride=1,
                 padding=1, rotate=False, shapes=(1, 1)),
    "cfg2": dict(batch=32, points=2048, grid=64, mult_in=4, mult_out=8, lmax=3, kernel=3, stride=1,
                 padding=1, rotate=True, shapes=(1, 1)),
    "cfg3": dict(batch=32, points=2048, grid=64, mult_in=8, mult_out=16, lmax=3, kernel=3,
                 stride=2, padding=1, rotate=False, shapes=(1, 1)),
    "cfg5": dict(batch=8, points=16384, grid=128, mult_in=8, mult_out=8, lmax=4, kernel=5,
                 stride=1, padding=2, rotate=False, shapes=(3, 5)),
}


def irreps(mult, lmax):
    """[(mult, 0), (mult, 1), ..., (mult, lmax)]."""
    return [(mult, l) for l in range(lmax + 1)]


def _random_rotation(rng):
    q, r = np.linalg.qr(rng.normal(size=(3, 3)))
    q = q * np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q


def _box_surface(rng, n, half):
    areas = np.array([half[1] * half[2], half[0] * half[2], half[0] * half[1]])
    axis = rng.choice(3, size=n, p=areas / areas.sum())
    pts = rng.uniform(-1.0, 1.0, size=(n, 3)) * half
    side = rng.choice([-1.0, 1.0], size=n)
    pts[np.arange(n), axis] = side * half[axis]
    return pts


def _ellipsoid_surface(rng, n, half):
    v = rng.normal(size=(n, 3))
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    return v * half


def surface_cloud(rng, n_points, rotate=False, shapes=(1, 1), noise=0.01):
    """One cloud [n_points, 3] float32 inside (-1, 1)^3."""
    n_shapes = int(rng.integers(shapes[0], shapes[1] + 1))
    counts = np.full(n_shapes, n_points // n_shapes)
    counts[: n_points - counts.sum()] += 1
    parts = []
    for c in counts:
        half = rng.uniform(0.3, 0.9, size=3)
        centre = np.zeros(3)
        if n_shapes > 1:
            half = half * 0.5
            centre = rng.uniform(-0.45, 0.45, size=3)
        pts = _box_surface(rng, c, half) if rng.integers(2) == 0 else \
            _ellipsoid_surface(rng, c, half)
        parts.append(pts + centre)
    pts = np.concatenate(parts, axis=0)
    if rotate:
        pts = pts @ _random_rotation(rng).T
    pts = pts + rng.normal(scale=noise, size=pts.shape)
    return np.clip(pts, -0.999, 0.999).astype(np.float32)


def make_clouds(batch, points, seed=0, rotate=False, shapes=(1, 1), channels=1):
    """points [B*n, 3] float32, features [B*n, C] float32 ~ N(0,1), batch_ids [B*n] int64."""
    rng = np.random.default_rng(seed)
    pts = np.concatenate([surface_cloud(rng, points, rotate, shapes) for _ in range(batch)], 0)
    feats = rng.normal(size=(batch * points, channels)).astype(np.float32)
    ids = np.repeat(np.arange(batch, dtype=np.int64), points)
    return pts, feats, ids


def config_clouds(name, seed=0):
    c = CONFIGS[name]
    channels = sum(c["mult_in"] * (2 * l + 1) for l in range(c["lmax"] + 1))
    return make_clouds(c["batch"], c["points"], seed, c["rotate"], c["shapes"], channels)


def voxel_indices(points, batch_ids, grid):
    """Sorted unique (b, x, y, z) int32 rows of the occupied voxels of [-1, 1]^3
    cut into grid^3 cells (fp32 arithmetic of the voxeliser: (p + 1) / (2/grid))."""
    unit = np.float32(np.float64(2.0) / grid)
    half = np.float32(0.5) * (np.float32(grid) * unit)
    vox = ((points.astype(np.float32) + half) / unit).astype(np.int32)
    rows = np.concatenate([batch_ids.astype(np.int32)[:, None], vox], axis=1)
    return np.unique(rows, axis=0)
