"""Seeded synthetic voxel sets for the sparse-convolution benchmark configurations.

All generators return int32 coordinates of shape [L, 4] with columns (n, d, h, w),
unique cells, sorted by (n, linear index) -- the order numpy.unique leaves them in.
Pass ``shuffle=True`` to get generation-independent random row order instead.
"""
import numpy as np


def _finish(lin, grid, L, rng, shuffle):
    D, H, W = grid[1:]
    lin = np.asarray(lin, dtype=np.int64)
    n = lin // (D * H * W)
    rem = lin % (D * H * W)
    d = rem // (H * W)
    rem = rem % (H * W)
    h = rem // W
    w = rem % W
    out = np.stack([n, d, h, w], axis=1).astype(np.int32)
    assert out.shape[0] == L
    if shuffle:
        out = out[rng.permutation(L)]
    return out


def uniform_voxels(grid, L, seed, shuffle=False):
    """L distinct cells drawn uniformly from a grid (N, D, H, W)."""
    rng = np.random.default_rng(seed)
    total = int(np.prod(grid))
    lin = rng.choice(total, size=L, replace=False)
    lin.sort()
    return _finish(lin, grid, L, rng, shuffle)


def clustered_voxels(grid, per_batch, seed, n_boxes=200, box_lo=4, box_hi=40,
                     frac_boxes=0.7, shuffle=False):
    """Per batch: ``frac_boxes`` of the cells fall inside ``n_boxes`` random
    axis-aligned boxes (edge box_lo..box_hi per axis, clipped to the grid), the
    rest are uniform.  Duplicates are removed and the set is topped up with
    uniform cells to exactly ``per_batch`` cells per batch."""
    rng = np.random.default_rng(seed)
    N, D, H, W = grid
    vol = D * H * W
    lins = []
    for n in range(N):
        n_in = int(round(per_batch * frac_boxes))
        edges = rng.integers(box_lo, box_hi + 1, size=(n_boxes, 3))
        edges = np.minimum(edges, np.array([D, H, W]))
        origin = np.stack([rng.integers(0, D - edges[:, 0] + 1),
                           rng.integers(0, H - edges[:, 1] + 1),
                           rng.integers(0, W - edges[:, 2] + 1)], axis=1)
        which = rng.integers(0, n_boxes, size=n_in)
        off = (rng.random((n_in, 3)) * edges[which]).astype(np.int64)
        p = origin[which] + off
        cells = (p[:, 0] * H + p[:, 1]) * W + p[:, 2]
        uni = rng.integers(0, vol, size=per_batch - n_in)
        cells = np.unique(np.concatenate([cells, uni]))
        while cells.size < per_batch:
            extra = rng.integers(0, vol, size=(per_batch - cells.size) * 2)
            cells = np.unique(np.concatenate([cells, extra]))
            if cells.size > per_batch:
                drop = rng.choice(cells.size, size=cells.size - per_batch, replace=False)
                cells = np.delete(cells, drop)
        lins.append(cells + n * vol)
    lin = np.concatenate(lins)
    return _finish(lin, grid, per_batch * N, rng, shuffle)


def surface_voxels(grid, L, seed, n_shapes=50, noise_frac=0.05, shuffle=False):
    """Cells on ``n_shapes`` random planes and spheres (voxelised), plus
    ``noise_frac`` uniform cells, single batch index range grid[0]."""
    rng = np.random.default_rng(seed)
    N, D, H, W = grid
    vol = D * H * W
    n_noise = int(round(L * noise_frac))
    target_surface = L - n_noise
    per_shape = int(np.ceil(target_surface / n_shapes * 1.6))
    pts = []
    for s in range(n_shapes):
        n = rng.integers(0, N)
        if s % 2 == 0:  # plane: point + two in-plane directions
            c = rng.random(3) * np.array([D, H, W])
            u = rng.normal(size=3)
            v = rng.normal(size=3)
            u /= np.linalg.norm(u)
            v -= u * (u @ v)
            v /= np.linalg.norm(v)
            ext = rng.uniform(60, 400)
            a = rng.uniform(-ext, ext, size=(per_shape, 1))
            b = rng.uniform(-ext, ext, size=(per_shape, 1))
            p = c + a * u + b * v
        else:  # sphere shell
            r = rng.uniform(10, 60)
            c = rng.random(3) * np.array([D, H, W])
            dirs = rng.normal(size=(per_shape, 3))
            dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
            p = c + r * dirs
        p = np.floor(p).astype(np.int64)
        ok = (p[:, 0] >= 0) & (p[:, 0] < D) & (p[:, 1] >= 0) & (p[:, 1] < H) & \
             (p[:, 2] >= 0) & (p[:, 2] < W)
        p = p[ok]
        pts.append(n * vol + (p[:, 0] * H + p[:, 1]) * W + p[:, 2])
    cells = np.unique(np.concatenate(pts))
    if cells.size > target_surface:
        keep = rng.choice(cells.size, size=target_surface, replace=False)
        cells = cells[np.sort(keep)]
    cells = np.unique(np.concatenate([cells, rng.integers(0, N * vol, size=n_noise)]))
    while cells.size < L:
        extra = rng.integers(0, N * vol, size=(L - cells.size) * 2)
        cells = np.unique(np.concatenate([cells, extra]))
    if cells.size > L:
        drop = rng.choice(cells.size, size=cells.size - L, replace=False)
        cells = np.delete(cells, drop)
    return _finish(cells, grid, L, rng, shuffle)


def scene_voxels(grid, L, seed, sheet_frac=0.6, wall_frac=0.3, shuffle=False):
    """L cells of a driving scene as a voxelizer leaves it, over all batches of ``grid``:
    ``sheet_frac`` of them in filled rectangles one or two cells thick along D (ground, roofs),
    ``wall_frac`` in filled upright rectangles one or two cells thick along H or W (walls,
    vehicles' sides), the rest uniform.  A cell of a filled sheet has 8 to 17 occupied neighbours in
    a 3x3x3 window, which is what the layers of a detection backbone see (against about one for
    cells strewn uniformly)."""
    rng = np.random.default_rng(seed)
    N, D, H, W = grid
    vol = D * H * W
    want_sheet, want_wall = int(L * sheet_frac), int(L * wall_frac)

    def rectangles(quota, upright):
        got, cells = 0, []
        while got < quota:
            n = rng.integers(0, N)
            thick = rng.integers(1, 3)
            if not upright:
                eh, ew = rng.integers(max(4, H // 36), max(6, H // 7) + 1), rng.integers(max(4, W // 36), max(6, W // 7) + 1)
                d0 = rng.integers(0, D - thick + 1)
                h0, w0 = rng.integers(0, H - eh + 1), rng.integers(0, W - ew + 1)
                dd, hh, ww = np.meshgrid(np.arange(d0, d0 + thick), np.arange(h0, h0 + eh),
                                         np.arange(w0, w0 + ew), indexing="ij")
            else:
                ed = rng.integers(min(3, D), min(D, 12) + 1)
                el = rng.integers(max(4, W // 72), max(6, W // 14) + 1)
                d0 = rng.integers(0, D - ed + 1)
                if rng.integers(0, 2):
                    h0, w0 = rng.integers(0, H - thick + 1), rng.integers(0, W - el + 1)
                    dd, hh, ww = np.meshgrid(np.arange(d0, d0 + ed), np.arange(h0, h0 + thick),
                                             np.arange(w0, w0 + el), indexing="ij")
                else:
                    el = min(el, H)
                    h0, w0 = rng.integers(0, H - el + 1), rng.integers(0, W - thick + 1)
                    dd, hh, ww = np.meshgrid(np.arange(d0, d0 + ed), np.arange(h0, h0 + el),
                                             np.arange(w0, w0 + thick), indexing="ij")
            c = n * vol + (dd.ravel() * H + hh.ravel()) * W + ww.ravel()
            cells.append(c)
            got += c.size
        return np.concatenate(cells)

    cells = np.unique(np.concatenate([rectangles(want_sheet, False), rectangles(want_wall, True)]))
    if cells.size > want_sheet + want_wall:
        cells = cells[np.sort(rng.choice(cells.size, size=want_sheet + want_wall, replace=False))]
    while cells.size < L:
        extra = rng.integers(0, N * vol, size=(L - cells.size) + 16)
        cells = np.unique(np.concatenate([cells, extra]))
    if cells.size > L:
        cells = np.delete(cells, rng.choice(cells.size, size=cells.size - L, replace=False))
    return _finish(cells, grid, L, rng, shuffle)


def kaiming_uniform_filters(K_shape, Ci, Co, seed):
    """Weights U(-b, b), b = 1/sqrt(K*Ci), laid out [kd, kh, kw, Ci, Co] (fp32)."""
    rng = np.random.default_rng(seed)
    K = int(np.prod(K_shape))
    b = 1.0 / np.sqrt(K * Ci)
    return rng.uniform(-b, b, size=tuple(K_shape) + (Ci, Co)).astype(np.float32)
