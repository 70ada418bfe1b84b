"""mluOpDynamicPointToVoxelForward through the C ABI: the two case files the reference ships
(replayed from their own values), the CPU oracle bit for bit (max and mean: the kernel adds
feats / count in point order, as the sequential definition does), and a full-size cloud."""
import os

import numpy as np
import pytest

import dynamic_point_to_voxel_oracle as dpv

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dynamic_point_to_voxel_forward")


def run_gpu(handle, mode, feats, coors, rows=None):
    import torch
    import mluop_hip
    c = torch.from_numpy(np.ascontiguousarray(coors, dtype=np.int32)).cuda()
    out = mluop_hip.dynamic_point_to_voxel_forward(handle, torch.from_numpy(feats).cuda(), c, mode, rows)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in out[:4]] + [int(out[4].item()), c.cpu().numpy()]


def assert_same(got, want):
    names = ("voxel_feats", "voxel_coors", "point2voxel_map", "voxel_points_count", "voxel_num", "coors")
    for g, w, name in zip(got, want, names):
        assert np.array_equal(g, w), name


@pytest.mark.parametrize("name", ["case_0.prototxt", "case_1.prototxt"])
def test_reference_case_files(gpu_handle, name):
    """Replayed from their own values and compared with their own stored outputs."""
    from mluop_hip import casefile as cf
    res = cf.replay(os.path.join(GOLDEN, name), gpu_handle)
    assert res.passed, res.errors
    node, _ = cf.load(os.path.join(GOLDEN, name))
    outs = [cf.CaseTensor(t) for t in node.all("output")]
    num = int(outs[4].values[0])
    assert res.voxel_num == num
    for t in outs[1:4]:                       # integer outputs: exact
        got, want = res.outputs[t.id], t.values.copy()
        if t is not outs[2]:
            want[num:] = 0
        assert np.array_equal(got, want), t.id
    for tid, func, err, thr in res.errors:   # sums in point order: far inside the file's 3e-3
        assert err <= 1e-6, (tid, func, err)


CASES = [(1, 1, 1, 1, 0.0), (2, 50, 3, 3, 0.1), (3, 5000, 5, 6, 0.05), (4, 5000, 4, 40, 0.0), (5, 300, 1, 2, 0.5),
         (6, 20000, 9, 12, 0.02)]


@pytest.mark.parametrize("mode", ["max", "mean"])
@pytest.mark.parametrize("case", CASES)
def test_matches_oracle(gpu_handle, mode, case):
    seed, n, c, span, neg = case
    print("dynamic_point_to_voxel case", case, mode, flush=True)
    rng = np.random.default_rng(seed)
    feats = rng.uniform(-100, 100, (n, c)).astype(np.float32)
    coors = rng.integers(0, span, (n, 3)).astype(np.int32)
    k = int(n * neg)
    if k:
        coors[rng.choice(n, k, replace=False), rng.integers(0, 3, k)] = -rng.integers(1, 5, k)
    assert_same(run_gpu(gpu_handle, mode, feats, coors), dpv.forward(mode, feats, coors))


@pytest.mark.parametrize("n", [2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 2049, 4095, 4097, 70001])
def test_point_counts_around_the_sort_boundaries(gpu_handle, n):
    """The grouping sort takes 64 pairs a wave at a time, 256 a wave, 1024 a workgroup: point
    counts on both sides of those, with few distinct triples (long runs of equal keys, whose
    points must keep their order for the mean to come out bit for bit) and with many."""
    rng = np.random.default_rng(100 + n)
    feats = rng.uniform(-100, 100, (n, 3)).astype(np.float32)
    for span in (2, 300):
        coors = rng.integers(0, span, (n, 3)).astype(np.int32)
        coors[:: max(n // 7, 1), 2] = -1
        assert_same(run_gpu(gpu_handle, "mean", feats, coors), dpv.forward("mean", feats, coors))
    same = np.full((n, 3), 5, np.int32)   # one voxel holds every point
    assert_same(run_gpu(gpu_handle, "mean", feats, same), dpv.forward("mean", feats, same))


def test_fewer_output_rows_than_voxels_and_all_invalid(gpu_handle):
    rng = np.random.default_rng(7)
    feats = rng.uniform(-1, 1, (400, 3)).astype(np.float32)
    coors = rng.integers(0, 5, (400, 3)).astype(np.int32)
    for mode in ("max", "mean"):
        assert_same(run_gpu(gpu_handle, mode, feats, coors, rows=20), dpv.forward(mode, feats, coors, rows=20))
    bad = -np.ones((64, 3), np.int32)
    got = run_gpu(gpu_handle, "mean", feats[:64], bad)
    assert got[4] == 0 and (got[2] == -1).all() and not got[0].any()


def test_large_coordinates(gpu_handle):
    """The three key widths: triples packed in 32 bits, in 64 bits (17 bits per axis), and three
    separate sorts (coordinates up to 2^31 - 1 need all 32 key bits each)."""
    rng = np.random.default_rng(8)
    feats = rng.uniform(-1, 1, (3000, 2)).astype(np.float32)
    for values in ([0, 1, 2, 900], [0, 1, 70000], [0, 1, 70000, 2 ** 31 - 1]):
        coors = rng.choice(np.array(values, dtype=np.int64), size=(3000, 3)).astype(np.int32)
        coors[::50, 1] = -7
        assert_same(run_gpu(gpu_handle, "max", feats, coors), dpv.forward("max", feats, coors))


def test_full_size_cloud(gpu_handle):
    rng = np.random.default_rng(9)
    n = 1000000
    feats = rng.uniform(-100, 100, (n, 4)).astype(np.float32)
    coors = np.stack([rng.integers(0, 40, n), rng.integers(0, 1600, n), rng.integers(0, 1408, n)], axis=1).astype(
        np.int32)
    coors[rng.choice(n, n // 20, replace=False), 0] = -1
    for mode in ("max", "mean"):
        assert_same(run_gpu(gpu_handle, mode, feats, coors), dpv.forward(mode, feats, coors))


def test_statuses(gpu_handle):
    import torch
    import mluop_hip
    feats = torch.zeros((8, 2), device="cuda")
    coors = torch.zeros((8, 3), dtype=torch.int32, device="cuda")
    with pytest.raises(mluop_hip.MluOpError) as e:
        mluop_hip.dynamic_point_to_voxel_forward(gpu_handle, feats, coors, "sum")
    assert e.value.status == mluop_hip.STATUS_BAD_PARAM


def test_backward_reference_case_file(gpu_handle):
    """The case stores 150 values for grad_voxel_feats [34, 5] (its 30 real voxels); the reader pads."""
    from mluop_hip import casefile as cf
    path = os.path.join(os.path.dirname(GOLDEN), "dynamic_point_to_voxel_backward", "case_1.prototxt")
    res = cf.replay(path, gpu_handle)
    node, _ = cf.load(path)
    want = cf.CaseTensor(node.all("output")[0])
    assert res.passed and np.array_equal(res.outputs[want.id], want.values)


@pytest.mark.parametrize("case", [(1, 200, 4, 3), (2, 5000, 6, 8), (3, 500, 1, 2), (4, 300000, 5, 30)])
def test_backward_matches_oracle_after_gpu_forward(gpu_handle, case):
    """Forward (max) and backward chained on the GPU; ties everywhere (integer features)."""
    import torch
    import mluop_hip
    seed, n, c, span = case
    print("dynamic_point_to_voxel backward case", case, flush=True)
    rng = np.random.default_rng(seed)
    feats = rng.integers(-3, 4, (n, c)).astype(np.float32)
    coors = rng.integers(0, span, (n, 3)).astype(np.int32)
    coors[rng.choice(n, n // 10, replace=False), 0] = -1
    g = rng.standard_normal((n, c)).astype(np.float32)
    tf, tc = torch.from_numpy(feats).cuda(), torch.from_numpy(coors).cuda()
    vf, vc, p2v, cnt, num = mluop_hip.dynamic_point_to_voxel_forward(gpu_handle, tf, tc, "max")
    grad = mluop_hip.dynamic_point_to_voxel_backward(gpu_handle, torch.from_numpy(g).cuda(), tf, vf, p2v, cnt, num)
    torch.cuda.synchronize()
    want = dpv.backward(g, feats, vf.cpu().numpy(), p2v.cpu().numpy(), int(num.item()))
    assert np.array_equal(grad.cpu().numpy(), want)


def test_backward_mean_is_rejected_like_the_reference(gpu_handle):
    import torch
    import mluop_hip
    z = torch.zeros((4, 3), device="cuda")
    i4 = torch.zeros((4,), dtype=torch.int32, device="cuda")
    with pytest.raises(mluop_hip.MluOpError) as e:
        mluop_hip.dynamic_point_to_voxel_backward(gpu_handle, z, z, z, i4, i4, i4[:1], "mean")
    assert e.value.status == mluop_hip.STATUS_BAD_PARAM


def test_inputs_at_odd_addresses(gpu_handle):
    """feats and coors as views one element into their allocations (4-byte aligned only)."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(13)
    n, c = 3000, 5
    feats = rng.uniform(-100, 100, (n, c)).astype(np.float32)
    coors = rng.integers(0, 9, (n, 3)).astype(np.int32)
    ff = torch.empty(feats.size + 8, dtype=torch.float32, device="cuda")
    fv = ff[1:1 + feats.size].view(feats.shape)
    fv.copy_(torch.from_numpy(feats))
    cc = torch.empty(coors.size + 8, dtype=torch.int32, device="cuda")
    cv = cc[1:1 + coors.size].view(coors.shape)
    cv.copy_(torch.from_numpy(coors))
    assert fv.data_ptr() % 16 != 0 and cv.data_ptr() % 16 != 0
    for mode, skew in (("max", 0), ("mean", 0), ("max", 4), ("mean", 12)):   # skew: workspace off alignment too
        cv.copy_(torch.from_numpy(coors))
        mluop_hip.WORKSPACE_SKEW = skew
        try:
            out = mluop_hip.dynamic_point_to_voxel_forward(gpu_handle, fv, cv, mode)
        finally:
            mluop_hip.WORKSPACE_SKEW = 0
        torch.cuda.synchronize()
        got = [t.cpu().numpy() for t in out[:4]] + [int(out[4].item()), cv.cpu().numpy()]
        assert_same(got, dpv.forward(mode, feats, coors))
