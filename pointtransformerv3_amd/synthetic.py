"""Seeded synthetic point clouds for tests and benchmarks (numpy, host side).

Every generator returns voxelised scenes with ONE point per occupied voxel — what Pointcept's
GridSample hands to the model and what a submanifold convolution requires.
"""
import numpy as np


def voxelize_unique(points, grid_size):
    """floor((p - min) / grid) and keep the first point of every voxel.
    Returns (grid_coord (M,3) int32, kept point indices (M,))."""
    g = np.floor((points - points.min(0)) / grid_size).astype(np.int64)
    key = (g[:, 0] << 42) | (g[:, 1] << 21) | g[:, 2]
    _, first = np.unique(key, return_index=True)
    first.sort()
    return g[first].astype(np.int32), first


def _box_surface(rng, n, lo, hi):
    """n points uniform on the surface of the axis-aligned box [lo, hi]."""
    size = hi - lo
    areas = np.array([size[1] * size[2], size[1] * size[2], size[0] * size[2], size[0] * size[2],
                      size[0] * size[1], size[0] * size[1]])
    face = rng.choice(6, size=n, p=areas / areas.sum())
    p = lo + rng.random((n, 3)) * size
    axis = face // 2
    side = face % 2
    p[np.arange(n), axis] = np.where(side == 0, lo[axis], hi[axis])
    return p


def room_points(n_points, seed, n_boxes=20, noise=0.005):
    """Points on the six planes of an 8 x 6 x 3 m room plus `n_boxes` random boxes
    (edge U[0.3,1.5] m), area-proportional, with Gaussian noise of `noise` metres."""
    rng = np.random.default_rng(seed)
    room_lo, room_hi = np.zeros(3), np.array([8.0, 6.0, 3.0])
    boxes = []
    for _ in range(n_boxes):
        edge = rng.uniform(0.3, 1.5, size=3)
        lo = np.array([rng.uniform(0, 8.0 - edge[0]), rng.uniform(0, 6.0 - edge[1]), 0.0])
        boxes.append((lo, lo + edge))

    def area(lo, hi):
        s = hi - lo
        return 2 * (s[0] * s[1] + s[1] * s[2] + s[0] * s[2])

    surfaces = [(room_lo, room_hi)] + boxes
    a = np.array([area(lo, hi) for lo, hi in surfaces])
    counts = rng.multinomial(n_points, a / a.sum())
    pts = np.concatenate([_box_surface(rng, c, lo, hi) for c, (lo, hi) in zip(counts, surfaces)])
    pts += rng.normal(0.0, noise, size=pts.shape)
    return pts[rng.permutation(len(pts))]


def room_scene(n_points, seed, grid_size=0.02):
    """One voxelised room: dict(coord (M,3) f32, grid_coord (M,3) i32); M <= n_points."""
    pts = room_points(n_points, seed)
    g, keep = voxelize_unique(pts, grid_size)
    return dict(coord=pts[keep].astype(np.float32), grid_coord=g)


def room_voxels(n_voxels, seed, grid_size=0.02):
    """Exactly `n_voxels` unique voxels from the room generator (over-draw, then cut)."""
    n_draw = int(n_voxels * 1.15) + 1000
    while True:
        sc = room_scene(n_draw, seed, grid_size)
        if len(sc["grid_coord"]) >= n_voxels:
            return dict(coord=sc["coord"][:n_voxels], grid_coord=sc["grid_coord"][:n_voxels])
        n_draw = int(n_draw * 1.3)


def cube_scene(n_voxels, seed, grid_size=0.02, side=5.0):
    """Exactly `n_voxels` unique voxels of points uniform in a cube of `side` metres (a volume, not a
    surface: the plumbing case of the CPU-runnable baseline configuration)."""
    rng = np.random.default_rng(seed)
    pts = rng.random((int(n_voxels * 1.05) + 64, 3)) * side
    while True:
        g, keep = voxelize_unique(pts, grid_size)
        if len(g) >= n_voxels:
            return dict(coord=pts[keep][:n_voxels].astype(np.float32), grid_coord=g[:n_voxels])
        pts = np.concatenate([pts, rng.random((n_voxels, 3)) * side])


def lidar_scene(seed, grid_size=0.05, beams=64, az_step_deg=0.2, max_range=75.0, n_boxes=30):
    """One spinning-LiDAR sweep: `beams` elevations in [-25,+3] deg, azimuth step 0.2 deg
    (115,200 rays), cast against the ground plane z=-1.8 m, random boxes (vehicles, buildings) and
    a ring of walls near 60-70 m that catches the upper beams; returns past `max_range` are
    dropped. Point density falls off with range as for a real sweep."""
    rng = np.random.default_rng(seed)
    elev = np.deg2rad(np.linspace(-25.0, 3.0, beams))
    az = np.deg2rad(np.arange(0.0, 360.0, az_step_deg))
    e, a = np.meshgrid(elev, az, indexing="ij")
    d = np.stack([np.cos(e) * np.cos(a), np.cos(e) * np.sin(a), np.sin(e)], -1).reshape(-1, 3)
    t = np.full(len(d), np.inf)
    down = d[:, 2] < -1e-6
    t[down] = -1.8 / d[down, 2]

    def hit_box(lo, hi):
        with np.errstate(divide="ignore", invalid="ignore"):
            t0, t1 = lo / d, hi / d
        tn, tf = np.minimum(t0, t1).max(1), np.maximum(t0, t1).min(1)
        return np.where((tn <= tf) & (tn > 0), tn, np.inf)

    boxes = []
    for _ in range(n_boxes):
        c = np.array([rng.uniform(-55, 55), rng.uniform(-55, 55)])
        if np.hypot(c[0], c[1]) < 4.0:
            continue
        half = np.array([rng.uniform(0.8, 4.0), rng.uniform(0.8, 4.0)])
        height = rng.uniform(1.5, 6.0)
        boxes.append((np.array([c[0] - half[0], c[1] - half[1], -1.8]), np.array([c[0] + half[0], c[1] + half[1], -1.8 + height])))
    # perimeter: four 12 m high walls at a random distance of 58-68 m
    for axis, sign in ((0, 1), (0, -1), (1, 1), (1, -1)):
        dist = rng.uniform(58, 68)
        lo, hi = np.array([-70.0, -70.0, -1.8]), np.array([70.0, 70.0, 10.2])
        if sign > 0:
            lo[axis], hi[axis] = dist, dist + 1.0
        else:
            lo[axis], hi[axis] = -dist - 1.0, -dist
        boxes.append((lo, hi))
    for lo, hi in boxes:
        t = np.minimum(t, hit_box(lo, hi))
    ok = t < max_range
    pts = d[ok] * t[ok, None] + rng.normal(0, 0.01, size=(int(ok.sum()), 3))
    g, keep = voxelize_unique(pts, grid_size)
    return dict(coord=pts[keep].astype(np.float32), grid_coord=g)


def collate(scenes):
    """Concatenate scenes: grid_coord (N,3) i32, coord (N,3) f32, offset (B,) i64, batch (N,) i64."""
    counts = [len(s["grid_coord"]) for s in scenes]
    return dict(
        grid_coord=np.concatenate([s["grid_coord"] for s in scenes]).astype(np.int32),
        coord=np.concatenate([s["coord"] for s in scenes]).astype(np.float32),
        offset=np.cumsum(counts).astype(np.int64),
        batch=np.repeat(np.arange(len(scenes)), counts).astype(np.int64),
    )


def room_features(coord, seed):
    """6-dim input as in Pointcept's indoor configs: RGB U[0,1] and unit normals (the xyz of a
    point enters the model through coord / grid_coord)."""
    rng = np.random.default_rng(seed)
    nrm = rng.normal(size=(len(coord), 3))
    nrm /= np.linalg.norm(nrm, axis=1, keepdims=True)
    return np.concatenate([rng.random((len(coord), 3)), nrm], 1).astype(np.float32)


def lidar_features(coord, seed):
    """4-dim input: xyz, intensity U[0,1]."""
    rng = np.random.default_rng(seed)
    return np.concatenate([coord, rng.random((len(coord), 1))], 1).astype(np.float32)
