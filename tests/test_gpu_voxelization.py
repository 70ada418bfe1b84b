"""mluOpVoxelization through the C ABI against the CPU oracle, bit for bit: every output tensor
including the zero fill of unused voxels.  Sizes the oracle's quadratic search finishes in seconds
are compared with it directly; a full-size cloud is compared with the sort-based formulation the
CPU tests pin against the oracle."""
import numpy as np
import pytest

import voxelization_oracle as vox
from voxel_cases import lidar_like_points, sorted_voxelization

pytestmark = pytest.mark.gpu


def run_gpu(handle, pts, vs, cr, max_points, max_voxels):
    import torch
    import mluop_hip
    out = mluop_hip.voxelization(handle, torch.from_numpy(pts).cuda(),
                                 torch.tensor(vs, dtype=torch.float32).cuda(),
                                 torch.tensor(cr, dtype=torch.float32).cuda(), max_points, max_voxels)
    torch.cuda.synchronize()
    return out[0].cpu().numpy(), out[1].cpu().numpy(), out[2].cpu().numpy(), int(out[3].item())


def assert_same(got, want):
    assert got[3] == want[3], "voxel_num"
    for g, w, name in zip(got[:3], want[:3], ("voxels", "coors", "num_points_per_voxel")):
        assert np.array_equal(g, w), name


CASES = [
    # seed, points, features, max_points, max_voxels
    (1, 1, 3, 1, 1),
    (2, 300, 4, 3, 40),          # both caps bind
    (3, 5000, 4, 5, 100000),     # no cap binds
    (4, 5000, 5, 1, 900),
    (5, 20000, 4, 35, 2000),
    (6, 20000, 7, 2, 20000),
]


@pytest.mark.parametrize("case", CASES)
def test_matches_oracle(gpu_handle, case):
    seed, n, f, max_points, max_voxels = case
    print("voxelization case", case, flush=True)
    rng = np.random.default_rng(seed)
    pts = lidar_like_points(rng, n, features=f, spread=(8.0, 4.0, 2.0))
    vs, cr = [0.4, 0.4, 1.0], [0.0, -4.0, -2.0, 8.0, 4.0, 1.0]
    assert_same(run_gpu(gpu_handle, pts, vs, cr, max_points, max_voxels),
                vox.voxelization(pts, vs, cr, max_points, max_voxels))


def test_special_values_and_all_points_outside(gpu_handle):
    pts = np.array([[np.nan, 0.1, 0.1, 1], [0.1, np.inf, 0.1, 2], [0.1, 0.1, -1e30, 3], [1e30, 0.1, 0.1, 4],
                    [0.1, 0.1, 0.1, 5], [-0.0, 0.0, 0.0, 6]], dtype=np.float32)
    vs, cr = [0.5, 0.5, 1.0], [0.0, 0.0, 0.0, 4.0, 4.0, 2.0]
    assert_same(run_gpu(gpu_handle, pts, vs, cr, 3, 3), vox.voxelization(pts, vs, cr, 3, 3))
    far = np.full((100, 4), 1000.0, np.float32)
    got = run_gpu(gpu_handle, far, vs, cr, 3, 3)
    assert got[3] == 0 and not got[0].any() and not got[1].any() and not got[2].any()


def test_one_crowded_cell(gpu_handle):
    """Thousands of points in one cell: positions past max_points are dropped, order is kept."""
    rng = np.random.default_rng(8)
    pts = np.empty((6000, 4), np.float32)
    pts[:, :3] = rng.uniform(0.0, 0.39, (6000, 3))
    pts[:, 3] = np.arange(6000)
    pts[::7, 0] += 0.4                      # every seventh point goes next door
    vs, cr = [0.4, 0.4, 0.4], [0.0, 0.0, 0.0, 4.0, 4.0, 4.0]
    got = run_gpu(gpu_handle, pts, vs, cr, 10, 50)
    assert_same(got, vox.voxelization(pts, vs, cr, 10, 50))
    assert got[3] == 2 and got[2][:2].tolist() == [10, 10]
    assert got[0][1, :, 3].tolist() == [1, 2, 3, 4, 5, 6, 8, 9, 10, 11]


def test_full_size_cloud_and_repeatability(gpu_handle):
    """1.2 M points, KITTI-like grid (1408 x 1600 x 40 cells): against the sort-based formulation,
    and the same bits on a second run."""
    rng = np.random.default_rng(10)
    pts = lidar_like_points(rng, 1200000, features=4, spread=(70.4, 40.0, 3.0), outliers=0.05)
    vs, cr = [0.05, 0.05, 0.1], [0.0, -40.0, -3.0, 70.4, 40.0, 1.0]
    got = run_gpu(gpu_handle, pts, vs, cr, 5, 150000)
    assert_same(got, sorted_voxelization(pts, vs, cr, 5, 150000))
    again = run_gpu(gpu_handle, pts, vs, cr, 5, 150000)
    assert_same(again, got)


def test_statuses(gpu_handle):
    import torch
    import mluop_hip
    pts = torch.zeros((10, 4), device="cuda")
    vs = torch.ones(3, device="cuda")
    cr = torch.tensor([0, 0, 0, 4, 4, 4.0], device="cuda")
    with pytest.raises(mluop_hip.MluOpError) as e:
        mluop_hip.voxelization(gpu_handle, pts, vs, cr, 3, 3, deterministic=False)
    assert e.value.status == mluop_hip.STATUS_BAD_PARAM
    # zero caps: success, nothing written, no workspace asked for
    out = mluop_hip.voxelization(gpu_handle, pts, vs, cr, 0, 3)
    assert out[0].shape == (3, 0, 4)


def test_points_at_an_odd_address(gpu_handle):
    """A points tensor that is only 4-byte aligned (a view one element into its allocation)."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(12)
    pts = lidar_like_points(rng, 3000, features=4, spread=(8.0, 4.0, 2.0))
    vs, cr = [0.4, 0.4, 1.0], [0.0, -4.0, -2.0, 8.0, 4.0, 1.0]
    flat = torch.empty(pts.size + 8, dtype=torch.float32, device="cuda")
    view = flat[1:1 + pts.size].view(pts.shape)
    view.copy_(torch.from_numpy(pts))
    assert view.data_ptr() % 16 != 0
    expect = vox.voxelization(pts, vs, cr, 5, 2000)
    for skew in (0, 4):   # and a workspace that is only 4-byte aligned
        mluop_hip.WORKSPACE_SKEW = skew
        try:
            out = mluop_hip.voxelization(gpu_handle, view, torch.tensor(vs, dtype=torch.float32).cuda(),
                                         torch.tensor(cr, dtype=torch.float32).cuda(), 5, 2000)
        finally:
            mluop_hip.WORKSPACE_SKEW = 0
        torch.cuda.synchronize()
        got = (out[0].cpu().numpy(), out[1].cpu().numpy(), out[2].cpu().numpy(), int(out[3].item()))
        assert_same(got, expect)


def test_captured_voxelization_replays_bit_exactly():
    """The operator enqueues kernels only (its sort and prefix sums are the library's own: no
    memset node, no wait), so a caller can capture it into a HIP graph.  Three replays with eager
    work and waits between them, on points that change between replays, each against the eager
    result for the same points."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(12)
    n, max_points, max_voxels = 20000, 4, 3000
    vs_np, cr_np = [0.4, 0.4, 1.0], [0.0, -4.0, -2.0, 8.0, 4.0, 1.0]
    clouds = [lidar_like_points(rng, n, features=4, spread=(8.0, 4.0, 2.0)) for _ in range(3)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    guard_bytes, mluop_hip.GUARD_BYTES = mluop_hip.GUARD_BYTES, 0
    try:
        with torch.cuda.stream(side):
            handle = mluop_hip.make_handle_on_current_stream()
            pts = torch.from_numpy(clouds[0]).cuda()
            vs = torch.tensor(vs_np, dtype=torch.float32).cuda()
            cr = torch.tensor(cr_np, dtype=torch.float32).cuda()
            mluop_hip.voxelization(handle, pts, vs, cr, max_points, max_voxels)   # first call outside the capture
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                captured = mluop_hip.voxelization(handle, pts, vs, cr, max_points, max_voxels)
            for cloud in clouds:
                pts.copy_(torch.from_numpy(cloud).cuda())
                for t in captured:
                    t.fill_(-7)
                graph.replay()
                side.synchronize()
                eager = mluop_hip.voxelization(handle, pts, vs, cr, max_points, max_voxels)
                side.synchronize()
                for name, got, want in zip(("voxels", "coors", "num_points_per_voxel", "voxel_num"), captured, eager):
                    assert torch.equal(got, want), name
                got = tuple(t.cpu().numpy() for t in captured[:3]) + (int(captured[3].item()),)
                assert_same(got, vox.voxelization(cloud, vs_np, cr_np, max_points, max_voxels))
        torch.cuda.current_stream().wait_stream(side)
        handle.close()
    finally:
        mluop_hip.GUARD_BYTES = guard_bytes
