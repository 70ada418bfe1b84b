"""Pins the voxelization oracle (the C restatement of the reference gtest's cpuCompute): cases
worked by hand, a second formulation built on a stable sort instead of the reference's search over
earlier points, and invariants that a dropped cap or a wrong axis order would break."""
import numpy as np
import pytest

import voxelization_oracle as vox
from voxel_cases import lidar_like_points, sorted_voxelization

VS = [0.5, 0.5, 1.0]
CR = [0.0, 0.0, 0.0, 4.0, 4.0, 2.0]      # grid 8 x 8 x 2 (x, y, z)


def test_hand_worked_case():
    pts = np.array([
        [0.1, 0.1, 0.1, 10],    # cell x0 y0 z0 -> voxel 0, slot 0
        [3.9, 0.2, 1.5, 11],    # cell x7 y0 z1 -> voxel 1, slot 0
        [0.2, 0.3, 0.9, 12],    # voxel 0, slot 1
        [4.0, 0.0, 0.0, 13],    # x = 4.0 is outside [0, 4)
        [0.4, 0.4, 0.5, 14],    # voxel 0, third point: over max_points = 2, dropped
        [1.0, 2.6, 0.0, 15],    # cell x2 y5 z0 -> voxel 2
        [-0.1, 1.0, 1.0, 16],   # outside
        [3.6, 0.4, 1.9, 17],    # voxel 1, slot 1
    ], dtype=np.float32)
    voxels, coors, npv, num = vox.voxelization(pts, VS, CR, max_points=2, max_voxels=5)
    assert num == 3
    assert coors[:3].tolist() == [[0, 0, 0], [1, 0, 7], [0, 5, 2]]          # (z, y, x)
    assert npv.tolist() == [2, 2, 1, 0, 0]
    assert voxels[0, :, 3].tolist() == [10, 12] and voxels[1, :, 3].tolist() == [11, 17]
    assert voxels[2, :, 3].tolist() == [15, 0]
    assert not voxels[3:].any() and not coors[3:].any()


def test_voxel_cap_drops_later_cells_and_their_points():
    pts = np.array([[0.1, 0.1, 0.1], [1.1, 0.1, 0.1], [2.1, 0.1, 0.1], [1.2, 0.2, 0.2], [2.2, 0.1, 0.1],
                    [0.2, 0.2, 0.2]], dtype=np.float32)
    voxels, coors, npv, num = vox.voxelization(pts, VS, CR, max_points=4, max_voxels=2)
    assert num == 2 and npv.tolist() == [2, 2]
    assert coors.tolist() == [[0, 0, 0], [0, 0, 2]]
    assert np.array_equal(voxels[0, :2], pts[[0, 5]]) and np.array_equal(voxels[1, :2], pts[[1, 3]])


def test_grid_extent_rounds_half_away_from_zero():
    # (1.25 - 0) / 0.5 = 2.5 -> 3 cells along x: x = 1.3 (cell 2) is inside, x = 1.6 (cell 3) is not
    pts = np.array([[1.3, 0.1, 0.1], [1.6, 0.1, 0.1]], dtype=np.float32)
    _, coors, npv, num = vox.voxelization(pts, [0.5, 0.5, 1.0], [0, 0, 0, 1.25, 4, 2], 3, 3)
    assert num == 1 and coors[0].tolist() == [0, 0, 2]


def test_nan_and_huge_coordinates_are_outside():
    pts = np.array([[np.nan, 0.1, 0.1], [0.1, np.inf, 0.1], [0.1, 0.1, -1e30], [1e30, 0.1, 0.1], [0.1, 0.1, 0.1]],
                   dtype=np.float32)
    _, coors, npv, num = vox.voxelization(pts, VS, CR, 3, 3)
    assert num == 1 and npv.tolist() == [1, 0, 0]


def test_empty_and_zero_caps():
    pts = np.zeros((0, 4), np.float32)
    voxels, coors, npv, num = vox.voxelization(pts, VS, CR, 3, 3)
    assert num == 0 and not voxels.any()
    pts = np.full((5, 3), 0.1, np.float32)
    assert vox.voxelization(pts, VS, CR, 0, 3)[3] == 0
    assert vox.voxelization(pts, VS, CR, 3, 0)[3] == 0


@pytest.mark.parametrize("seed,n,max_points,max_voxels", [(1, 400, 3, 50), (2, 3000, 5, 100000), (3, 3000, 1, 700),
                                                         (4, 6000, 35, 300), (5, 2000, 2, 2000)])
def test_matches_the_sort_based_formulation(seed, n, max_points, max_voxels):
    rng = np.random.default_rng(seed)
    pts = lidar_like_points(rng, n, features=4 + seed % 2, spread=(8.0, 4.0, 2.0))
    vs, cr = [0.4, 0.4, 1.0], [0.0, -4.0, -2.0, 8.0, 4.0, 1.0]
    got = vox.voxelization(pts, vs, cr, max_points, max_voxels)
    want = sorted_voxelization(pts, vs, cr, max_points, max_voxels)
    assert got[3] == want[3]
    for g, w, name in zip(got[:3], want[:3], ("voxels", "coors", "num_points_per_voxel")):
        assert np.array_equal(g, w), name


def test_invariants():
    rng = np.random.default_rng(9)
    pts = lidar_like_points(rng, 5000, spread=(8.0, 4.0, 2.0))
    vs, cr = [0.4, 0.4, 1.0], [0.0, -4.0, -2.0, 8.0, 4.0, 1.0]
    voxels, coors, npv, num = vox.voxelization(pts, vs, cr, 4, 10000)
    assert (npv[:num] >= 1).all() and (npv[:num] <= 4).all() and not npv[num:].any()
    # every stored point lies in the cell its voxel names, cells are distinct
    assert len({tuple(c) for c in coors[:num].tolist()}) == num
    for v in range(0, num, 37):
        for s in range(npv[v]):
            p = voxels[v, s]
            cell = np.floor((p[:3] - np.float32(cr[:3])) / np.float32(vs)).astype(int)
            assert cell[::-1].tolist() == coors[v].tolist()
    # a permutation that keeps the relative order within every cell changes nothing but voxel
    # numbering; doubling max_points never shrinks a voxel
    more = vox.voxelization(pts, vs, cr, 8, 10000)
    assert more[3] == num and np.array_equal(more[1], coors) and (more[2] >= npv).all()
    assert np.array_equal(more[0][:, :4][npv > 0][:, 0], voxels[npv > 0][:, 0])
