"""Seeded synthetic voxel scenes for the five benchmark workloads.

Every generator returns int32 coordinates ``[N, 4] = (x, y, z, batch)`` whose row
order is a seeded shuffle (never sorted), so site numbering by first appearance is
exercised.  Only numpy is used; nothing here touches a GPU.
"""
import numpy as np


def _box_faces(lo, size):
    """All voxels on the six faces of the axis-aligned box [lo, lo+size)."""
    lo = np.asarray(lo, np.int64)
    hi = lo + np.asarray(size, np.int64) - 1
    out = []
    for ax in range(3):
        a, b = [i for i in range(3) if i != ax]
        ga, gb = np.meshgrid(np.arange(lo[a], hi[a] + 1), np.arange(lo[b], hi[b] + 1), indexing="ij")
        for v in (lo[ax], hi[ax]):
            p = np.empty((ga.size, 3), np.int64)
            p[:, ax] = v
            p[:, a] = ga.ravel()
            p[:, b] = gb.ravel()
            out.append(p)
    return np.concatenate(out, 0)


def _unique_keep_order(p):
    """Unique rows, keeping the first occurrence and the generation order."""
    _, first = np.unique(p, axis=0, return_index=True)
    return p[np.sort(first)]


def _finish(p, n, rng, grid):
    p = p[(p >= 0).all(1) & (p < grid).all(1)]
    p = _unique_keep_order(p)
    if n is not None:
        if len(p) < n:
            raise ValueError("scene generator produced %d < %d voxels" % (len(p), n))
        p = p[:n]
    p = p[rng.permutation(len(p))]
    out = np.zeros((len(p), 4), np.int32)
    out[:, :3] = p
    return out


def boxes_scene(seed=1, n=20000, grid=128, n_boxes=8, lo_rng=(8, 88), size_rng=(12, 32)):
    """Workload 1: faces of random boxes in a small grid, exactly ``n`` voxels."""
    rng = np.random.default_rng(seed)
    parts = []
    for _ in range(n_boxes):
        parts.append(_box_faces(rng.integers(lo_rng[0], lo_rng[1], 3), rng.integers(size_rng[0], size_rng[1], 3)))
    p = np.concatenate(parts, 0)
    total = len(_unique_keep_order(p))
    while total < n:  # add boxes until enough surface exists
        parts.append(_box_faces(rng.integers(lo_rng[0], lo_rng[1], 3), rng.integers(size_rng[0], size_rng[1], 3)))
        p = np.concatenate(parts, 0)
        total = len(_unique_keep_order(p))
    return _finish(p, n, rng, grid)


def planes_boxes_scene(seed=2, n=200000, grid=1024, n_planes=6, n_boxes=20):
    """Workload 2: voxelised random planes plus box faces in a 1024^3 grid."""
    rng = np.random.default_rng(seed)
    parts = []
    for _ in range(n_boxes):
        lo = rng.integers(64, grid - 200, 3)
        parts.append(_box_faces(lo, rng.integers(24, 120, 3)))
    for _ in range(n_planes):
        nrm = rng.normal(size=3)
        nrm /= np.linalg.norm(nrm)
        ax = int(np.argmax(np.abs(nrm)))
        a, b = [i for i in range(3) if i != ax]
        c0 = rng.integers(grid // 4, 3 * grid // 4, 3).astype(np.float64)
        ext = 180
        ga, gb = np.meshgrid(np.arange(-ext, ext), np.arange(-ext, ext), indexing="ij")
        pa = c0[a] + ga.ravel()
        pb = c0[b] + gb.ravel()
        # solve nrm . (p - c0) = 0 for the dominant axis, round to the nearest voxel
        pax = c0[ax] - (nrm[a] * (pa - c0[a]) + nrm[b] * (pb - c0[b])) / nrm[ax]
        p = np.empty((pa.size, 3), np.int64)
        p[:, a] = pa
        p[:, b] = pb
        p[:, ax] = np.rint(pax)
        parts.append(p)
    p = np.concatenate(parts, 0)
    return _finish(p, n, rng, grid)


def _room(rng, origin, dims, n_boxes, side_rng, jitter=True):
    ox, oy, oz = origin
    dx, dy, dz = dims
    parts = []
    gx, gy = np.meshgrid(np.arange(dx), np.arange(dy), indexing="ij")
    floor = np.stack([gx.ravel(), gy.ravel(), np.zeros(gx.size, np.int64)], 1)
    nrm = [np.tile([0, 0, 1], (len(floor), 1))]
    parts.append(floor)
    gz = np.arange(1, dz)
    for x in (0, dx - 1):
        a, b = np.meshgrid(np.arange(dy), gz, indexing="ij")
        parts.append(np.stack([np.full(a.size, x), a.ravel(), b.ravel()], 1))
        nrm.append(np.tile([1, 0, 0], (a.size, 1)))
    for y in (0, dy - 1):
        a, b = np.meshgrid(np.arange(dx), gz, indexing="ij")
        parts.append(np.stack([a.ravel(), np.full(a.size, y), b.ravel()], 1))
        nrm.append(np.tile([0, 1, 0], (a.size, 1)))
    for _ in range(n_boxes):
        side = rng.integers(side_rng[0], side_rng[1], 3)
        lo = np.array([rng.integers(2, dx - side[0] - 2), rng.integers(2, dy - side[1] - 2), 1])
        f = _box_faces(lo, side)
        n_ = np.zeros_like(f)
        hi = lo + side - 1
        for ax in range(3):
            on = (f[:, ax] == lo[ax]) | (f[:, ax] == hi[ax])
            n_[on & (n_ == 0).all(1), ax] = 1
        parts.append(f)
        nrm.append(n_)
    p = np.concatenate(parts, 0).astype(np.int64)
    nv = np.concatenate(nrm, 0).astype(np.int64)
    if jitter:
        # +-1 voxel along the surface normal on a smooth low-frequency pattern, so the
        # surfaces stay connected sheets rather than salt-and-pepper noise
        ph = rng.uniform(0, 6.28, 3)
        s = np.sin(p[:, 0] * 0.11 + ph[0]) + np.sin(p[:, 1] * 0.13 + ph[1]) + np.sin(p[:, 2] * 0.17 + ph[2])
        j = np.where(s > 1.0, 1, np.where(s < -1.0, -1, 0))
        p = p + nv * j[:, None]
    p = p + np.array([ox, oy, oz], np.int64)
    return p


def indoor_scene(seed=3, n=500000, grid=4096, dims=(560, 450, 150), n_boxes=30, side_rng=(15, 60)):
    """Workloads 3/4: a room (floor, four walls, boxes) at 2 cm voxels in a 4096^3 grid."""
    rng = np.random.default_rng(seed)
    p = _room(rng, (1024, 1024, 1024), dims, n_boxes, side_rng)
    extra = 0
    while len(_unique_keep_order(p)) < n and extra < 200:
        side = rng.integers(side_rng[0], side_rng[1], 3)
        lo = np.array([1024 + rng.integers(2, dims[0] - side[0] - 2), 1024 + rng.integers(2, dims[1] - side[1] - 2), 1025])
        p = np.concatenate([p, _box_faces(lo, side)], 0)
        extra += 1
    return _finish(p, n, rng, grid)


def unet_scene(seed=4, n=150000, dup_frac=0.10):
    """Workload 4: 150k-voxel room; points = voxels plus ``dup_frac`` duplicated points.

    Returns (points[P,4] int32, rgb[P,3] float32, voxels[N,4] int32).
    """
    vox = indoor_scene(seed=seed, n=n, dims=(270, 220, 80), n_boxes=30, side_rng=(15, 60))
    rng = np.random.default_rng(seed + 1000)
    dup = vox[rng.integers(0, len(vox), int(dup_frac * len(vox)))]
    pts = np.concatenate([vox, dup], 0)
    pts = pts[rng.permutation(len(pts))]
    rgb = rng.uniform(0, 1, (len(pts), 3)).astype(np.float32)
    return pts, rgb, vox


def sweep_sequence(seed=5, n=150000, frames=50, first_frac=0.2):
    """Workload 5: a sensor sweep over the workload-4 room.

    Frame 0 holds the ``first_frac`` of the voxels nearest a start pose; each later frame
    adds the next voxels in order of distance along the sweep and re-observes 1k-2k already
    seen voxels with RGB perturbed by U[-0.1, 0.1].  The additions are drawn from 3k-8k and
    then scaled so that ``frames`` frames end exactly on ``n`` voxels: 49 unscaled draws would
    add some 270k voxels to a 150k-voxel scene, so with the default arguments a frame really
    adds 1.3k-3.6k voxels (2.4k on average).  ``target_frame`` below is the frame the latency
    target is stated on (5k new voxels onto a scene that then has 150k).
    Returns a list of (points[P,4] int32, rgb[P,3] float32) per frame.
    """
    vox = indoor_scene(seed=4, n=n, dims=(270, 220, 80), n_boxes=30, side_rng=(15, 60))
    rng = np.random.default_rng(seed)
    base_rgb = rng.uniform(0, 1, (len(vox), 3)).astype(np.float32)
    pose = np.array([1024 + 20, 1024 + 20, 1024 + 30], np.float64)
    d = np.linalg.norm(vox[:, :3].astype(np.float64) - pose, axis=1)
    order = np.argsort(d, kind="stable")
    n0 = int(first_frac * len(vox))
    remaining = len(vox) - n0
    adds = rng.integers(3000, 8001, frames - 1).astype(np.float64)
    adds = np.floor(adds * remaining / adds.sum()).astype(np.int64)
    adds[-1] += remaining - adds.sum()
    out = []
    seen = n0
    idx = order[:n0]
    idx = idx[rng.permutation(len(idx))]
    out.append((vox[idx].copy(), base_rgb[idx].copy()))
    for f in range(1, frames):
        new = order[seen:seen + adds[f - 1]]
        k = int(rng.integers(1000, 2001))
        old = order[rng.integers(0, seen, k)]
        idx = np.concatenate([new, old])
        rgb = base_rgb[idx].copy()
        rgb[len(new):] = np.clip(rgb[len(new):] + rng.uniform(-0.1, 0.1, (k, 3)).astype(np.float32), 0, 1)
        perm = rng.permutation(len(idx))
        out.append((vox[idx][perm].copy(), rgb[perm].copy()))
        seen += adds[f - 1]
    return out


def target_frame(seed=6, n=150000, n_new=5000, n_old=1500, old_from="scene"):
    """The frame the latency target is stated on: 5k new voxels onto a 150k-voxel scene.

    The workload-4 room in the order of the sweep (distance from the start pose): the first
    ``n - n_new`` voxels are the scene a full forward has seen (one point per voxel, seeded
    shuffle), and ONE incremental frame then brings exactly ``n_new`` new voxels - the next
    ones along the sweep, i.e. a shell at the scene's frontier, as a moving sensor delivers
    them - plus ``n_old`` re-observed voxels with RGB perturbed by U[-0.1, 0.1], drawn from the
    whole scene (``old_from="scene"``, as in the sweep: the harder case, it dirties every region)
    or from the 10 % of the scene nearest the frontier (``"frontier"``: what a sensor that moves
    on still sees).  This mirrors the reference's usage: one full pass, then a frame with
    increment=True (demo.py:26-38).
    Returns ((scene_points[n - n_new, 4], scene_rgb), (frame_points[n_new + n_old, 4], frame_rgb)).
    """
    vox = indoor_scene(seed=4, n=n, dims=(270, 220, 80), n_boxes=30, side_rng=(15, 60))
    rng = np.random.default_rng(seed)
    base_rgb = rng.uniform(0, 1, (len(vox), 3)).astype(np.float32)
    pose = np.array([1024 + 20, 1024 + 20, 1024 + 30], np.float64)
    d = np.linalg.norm(vox[:, :3].astype(np.float64) - pose, axis=1)
    order = np.argsort(d, kind="stable")
    n0 = n - n_new
    idx0 = order[:n0][rng.permutation(n0)]
    if old_from not in ("scene", "frontier"):
        raise ValueError("old_from must be 'scene' or 'frontier'")
    near = order[:n0] if old_from == "scene" else order[n0 - n0 // 10:n0]
    old = near[rng.permutation(len(near))[:n_old]]
    idx1 = np.concatenate([order[n0:], old])
    rgb1 = base_rgb[idx1].copy()
    rgb1[n_new:] = np.clip(rgb1[n_new:] + rng.uniform(-0.1, 0.1, (n_old, 3)).astype(np.float32), 0, 1)
    perm = rng.permutation(len(idx1))
    return (vox[idx0].copy(), base_rgb[idx0].copy()), (vox[idx1][perm].copy(), rgb1[perm].copy())
