"""Shared helpers of the voxelization tests: seeded point clouds and a second, sort-based
formulation of hard voxelization used to pin the oracle and to check full-size GPU runs."""
import numpy as np


def lidar_like_points(rng, n, features=4, spread=(70.0, 40.0, 3.0), outliers=0.1):
    """x, y, z (+ extra feature columns): most points inside the usual range, some outside."""
    pts = np.empty((n, features), dtype=np.float32)
    pts[:, 0] = rng.uniform(0.0, spread[0], n)
    pts[:, 1] = rng.uniform(-spread[1], spread[1], n)
    pts[:, 2] = rng.uniform(-spread[2], 1.0, n)
    k = int(n * outliers)
    if k:
        sel = rng.choice(n, size=k, replace=False)
        pts[sel, :3] += rng.choice([-1.0, 1.0], size=(k, 3)).astype(np.float32) * 200.0
    for f in range(3, features):
        pts[:, f] = rng.uniform(0, 1, n)
    return pts


def sorted_voxelization(points, voxel_size, coors_range, max_points, max_voxels):
    """Hard voxelization by a stable sort of the cell keys (no search over earlier points)."""
    points = np.asarray(points, dtype=np.float32)
    vs = np.asarray(voxel_size, dtype=np.float32)
    cr = np.asarray(coors_range, dtype=np.float32)
    n, f = points.shape
    grid = np.array([int(np.floor(np.float64((cr[3 + a] - cr[a]) / vs[a]) + 0.5)) for a in range(3)])
    voxels = np.zeros((max_voxels, max_points, f), np.float32)
    coors = np.zeros((max_voxels, 3), np.int32)
    npv = np.zeros((max_voxels,), np.int32)
    if n == 0 or max_points == 0 or max_voxels == 0:
        return voxels, coors, npv, 0
    with np.errstate(invalid="ignore", over="ignore"):
        c = np.floor((points[:, :3] - cr[:3]) / vs)            # float32 arithmetic, columns x, y, z
    ok = np.ones(n, bool)
    for a in range(3):
        ok &= (c[:, a] >= 0) & (c[:, a] < grid[a])
    ids = np.nonzero(ok)[0]
    ci = c[ids].astype(np.int64)
    key = (ci[:, 2] * grid[1] + ci[:, 1]) * grid[0] + ci[:, 0]
    order = np.argsort(key, kind="stable")
    sk = key[order]
    start = np.r_[True, sk[1:] != sk[:-1]]
    seg_first = np.maximum.accumulate(np.where(start, np.arange(sk.size), 0))
    rank = np.empty(ids.size, np.int64)
    rank[order] = np.arange(sk.size) - seg_first
    first_point = np.empty(ids.size, np.int64)
    first_point[order] = ids[order][seg_first]
    is_first = rank == 0
    vid_of_first = np.cumsum(is_first) - 1                     # points are in index order already
    vid = np.full(n, -1, np.int64)
    vid[ids[is_first]] = vid_of_first[is_first]
    v = vid[first_point]
    keep = (v < max_voxels) & (rank < max_points)
    voxels[v[keep], rank[keep]] = points[ids[keep]]
    head = keep & is_first
    coors[v[head]] = ci[head][:, ::-1].astype(np.int32)        # stored (z, y, x)
    np.add.at(npv, v[keep], 1)
    return voxels, coors, npv, int(min(is_first.sum(), max_voxels))
