"""mluOpExtIndiceConvolutionBackwardFilterNoAlloc against mluOpIndiceConvolutionBackwardFilter.

The entry point keeps its partial sums in an array the library holds on the GPU instead of a
caller's workspace; both run the same kernels, so the results must be the same bits.  Two calls
in a row, the second on a smaller input, show that nothing the first call left in the array
reaches the second result."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(seed, rows, ci, co, ks=(3, 3, 3)):
    import torch
    import mluop_hip
    import sparse_conv_oracle as oracle
    rng = np.random.default_rng(seed)
    space = (16, 48, 48)
    idx = mluop_hip.datagen.uniform_voxels((1,) + space, rows, seed=seed, shuffle=True)
    pairs, _, num, n_out = oracle.get_indice_pairs(idx, 1, [k // 2 for k in ks], [1, 1, 1], [1, 1, 1],
                                                   list(ks), list(space), True)
    feats = torch.from_numpy(rng.standard_normal((rows, ci)).astype(np.float32)).cuda().half()
    dy = torch.from_numpy((rng.standard_normal((n_out, co)) * 0.1).astype(np.float32)).cuda().half()
    return torch.from_numpy(pairs).cuda(), [int(v) for v in num], feats, dy, ks


def _both(handle, case):
    import torch
    import mluop_hip
    pairs, num, feats, dy, ks = case
    want = mluop_hip.indice_conv_backward_filter(handle, feats, dy, pairs, num, ks, True)
    got = torch.full_like(want, float("nan"))
    mluop_hip.indice_conv_backward_filter_no_alloc(handle, feats, dy, pairs, num, ks, True, got)
    torch.cuda.synchronize()
    return got, want


def test_two_calls_in_a_row_match_the_workspace_entry_point(gpu_handle):
    import torch
    big = _case(11, 30000, 64, 64)
    small = _case(12, 700, 32, 16)
    for case in (big, small):
        got, want = _both(gpu_handle, case)
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want)


def test_allocates_nothing(gpu_handle):
    import torch
    import mluop_hip
    case = _case(13, 5000, 32, 32)
    pairs, num, feats, dy, ks = case
    got = torch.empty(tuple(ks) + (32, 32), dtype=torch.float16, device="cuda")
    mluop_hip.indice_conv_backward_filter_no_alloc(gpu_handle, feats, dy, pairs, num, ks, True, got)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        mluop_hip.indice_conv_backward_filter_no_alloc(gpu_handle, feats, dy, pairs, num, ks, True, got)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before


def test_a_shape_whose_usual_slices_do_not_fit_runs_on_fewer(gpu_handle):
    """128 x 128 channels: 795 partial tiles of 64 KiB would be 50 MiB; the entry point cuts the pair
    lists into the 228 slices its 16 MiB hold beside one tile per offset.  Longer slices add up in
    another order, so the result is graded against the workspace entry point like a device result
    against the oracle (diff1, diff2 <= 3e-3), not bit for bit."""
    import torch
    got, want = _both(gpu_handle, _case(14, 30000, 128, 128))
    a, b = got.double(), want.double()
    assert torch.isfinite(a).all()
    diff1 = float((a - b).abs().sum() / (b.abs().sum() + 1e-9))
    diff2 = float(((a - b).square().sum() / (b.square().sum() + 1e-9)).sqrt())
    assert diff1 <= 3e-3 and diff2 <= 3e-3, (diff1, diff2)


def test_shapes_beyond_the_scratch_array_are_refused(gpu_handle):
    """192 x 192 channels run on the generic kernels, whose partial tiles (one per offset and
    4096 rows) cannot be made fewer: 5 x 27 tiles of 144 KiB do not fit."""
    import torch
    import mluop_hip
    pairs, num, feats, dy, ks = _case(15, 20000, 192, 192)
    got = torch.empty(tuple(ks) + (192, 192), dtype=torch.float16, device="cuda")
    with pytest.raises(mluop_hip.MluOpError) as err:
        mluop_hip.indice_conv_backward_filter_no_alloc(gpu_handle, feats, dy, pairs, num, ks, True, got)
    assert err.value.status == mluop_hip.STATUS_NOT_SUPPORTED
