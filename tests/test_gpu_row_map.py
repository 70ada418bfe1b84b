"""Row maps kept across calls (mluOpExtBuildRowMap / mluOpExtUseRowMap): a forward or
backward-data call that is handed the map of its rulebook must give, bit for bit, what the same
call gives when it builds the map itself; the map kernels and the collision check are then not
launched; maps with lost pairs, maps of another direction and unknown buffers are refused."""
import os

import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import out_space, random_voxels, to_torch

pytestmark = pytest.mark.gpu

SHAPES = [
    # (batch, space, L, ks, stride, sub_m, ci, co)
    (2, (10, 12, 12), 1500, (3, 3, 3), (1, 1, 1), True, 64, 64),      # pair-list MFMA kernel
    (1, (8, 8, 8), 400, (3, 3, 3), (1, 1, 1), True, 128, 128),        # dense enough for the register-accumulating kernel
    (2, (10, 12, 12), 1200, (3, 3, 3), (2, 2, 2), False, 32, 64),     # regular, strided
    (1, (6, 8, 8), 200, (1, 3, 3), (1, 1, 1), True, 13, 70),          # generic FMA kernel
    (1, (10, 10, 10), 400, (5, 5, 7), (1, 1, 1), True, 32, 32),       # K = 175: counts in device memory
]


def rulebook(m, handle, idx, batch, space, ks, stride, sub_m):
    import torch
    pad = [k // 2 for k in ks]
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, [1, 1, 1])
    pairs, out_idx, num, n_out = m.get_indice_pairs(handle, torch.from_numpy(idx).cuda(), batch, space, ks, ospace, pad,
                                                    list(stride), [1, 1, 1], sub_m)
    return pairs, num.cpu().tolist(), n_out


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype_name", ["float16", "bfloat16", "float32"])
def test_calls_with_a_map_equal_calls_without(gpu_handle, shape, dtype_name):
    import torch
    import mluop_hip as m
    batch, space, L, ks, stride, sub_m, ci, co = shape
    print("row map case", shape, dtype_name, flush=True)
    rng = np.random.default_rng(51)
    idx = random_voxels(rng, batch, space, L)
    pairs, num, n_out = rulebook(m, gpu_handle, idx, batch, space, ks, stride, sub_m)
    rows = idx.shape[0]
    feats = to_torch(rng.standard_normal((rows, ci)).astype(np.float32), dtype_name, "cuda")
    w = to_torch((rng.standard_normal(ks + (ci, co)) * 0.1).astype(np.float32), dtype_name, "cuda")
    dy = to_torch((rng.standard_normal((n_out, co)) * 0.1).astype(np.float32), dtype_name, "cuda")

    fwd_map = m.RowMap(gpu_handle, pairs, num, n_out, rows, 1)
    bwd_map = m.RowMap(gpu_handle, pairs, num, rows, n_out, 0)
    assert fwd_map.usable and fwd_map.lost_pairs == 0 and bwd_map.usable

    plain_out = m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, sub_m)
    plain_dx = m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, sub_m, ci)
    for _ in range(2):   # a map serves any number of calls
        out = m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, sub_m, row_map=fwd_map)
        dx = m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, sub_m, ci, row_map=bwd_map)
        torch.cuda.synchronize()
        assert torch.equal(out, plain_out) and torch.equal(dx, plain_dx)
    # and the call after an announced one builds its own map again
    again = m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, sub_m)
    torch.cuda.synchronize()
    assert torch.equal(again, plain_out)
    fwd_map.close()
    bwd_map.close()


def test_map_kernels_and_collision_check_are_not_launched(gpu_handle):
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(52)
    idx = random_voxels(rng, 1, (12, 16, 16), 2500)
    pairs, num, n_out = rulebook(m, gpu_handle, idx, 1, (12, 16, 16), (3, 3, 3), (1, 1, 1), True)
    feats = torch.randn(idx.shape[0], 64, device="cuda").half()
    w = (torch.randn(3, 3, 3, 64, 64, device="cuda") * 0.1).half()
    rm = m.RowMap(gpu_handle, pairs, num, n_out, idx.shape[0], 1)

    def kernels(row_map):
        gpu_handle.set_kernel_timing(True)
        m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, True, row_map=row_map)
        names = [k for k, _ in gpu_handle.kernel_timings()]
        gpu_handle.set_kernel_timing(False)
        return names

    # (four cells in five are occupied: left to itself the library takes the kernel for dense rulebooks)
    gpu_handle.set_kernel_choice("dense_tiles", False)
    try:
        assert kernels(None) == ["fillMapPackFilter", "scatterRowMap", "gatherConvMfma", "repairLostPairs"]
        assert kernels(rm) == ["fillMapPackFilter", "gatherConvMfma"]     # the first one only packs the filter here
    finally:
        gpu_handle.set_kernel_choice("dense_tiles", None)
    assert kernels(None) == ["fillMapPackFilter", "scatterRowMap", "gatherConvDense", "repairLostPairs"]
    assert kernels(rm) == ["fillMapPackFilter", "gatherConvDense"]
    rm.close()


def test_unverified_build_needs_the_promise(gpu_handle):
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(56)
    idx = random_voxels(rng, 1, (10, 12, 12), 900)
    pairs, num, n_out = rulebook(m, gpu_handle, idx, 1, (10, 12, 12), (3, 3, 3), (1, 1, 1), True)
    feats = torch.randn(idx.shape[0], 64, device="cuda").half()
    w = (torch.randn(3, 3, 3, 64, 64, device="cuda") * 0.1).half()
    with pytest.raises(m.MluOpError) as e:
        m.RowMap(gpu_handle, pairs, num, n_out, idx.shape[0], 1, verify=False)
    assert e.value.status == m.STATUS_BAD_PARAM
    plain = m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, True)
    gpu_handle.promise_distinct_pairs(True)
    try:
        rm = m.RowMap(gpu_handle, pairs, num, n_out, idx.shape[0], 1, verify=False)
        assert rm.usable and rm.lost_pairs is None
        out = m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, True, row_map=rm)
    finally:
        gpu_handle.promise_distinct_pairs(False)
    torch.cuda.synchronize()
    assert torch.equal(out, plain)
    rm.close()


def test_inverse_layer_with_maps(gpu_handle):
    import torch
    import mluop_hip as m
    gpu_handle.set_extended_modes(True)
    try:
        rng = np.random.default_rng(53)
        idx = random_voxels(rng, 1, (10, 12, 12), 900)
        pairs, num, n_out = rulebook(m, gpu_handle, idx, 1, (10, 12, 12), (3, 3, 3), (2, 2, 2), False)
        rows = idx.shape[0]
        x = torch.randn(n_out, 64, device="cuda").half()          # on the strided layer's outputs
        w = (torch.randn(3, 3, 3, 64, 32, device="cuda") * 0.1).half()
        dy = torch.randn(rows, 32, device="cuda").half()
        fwd_map = m.RowMap(gpu_handle, pairs, num, rows, n_out, 0)     # results on the partner's inputs
        bwd_map = m.RowMap(gpu_handle, pairs, num, n_out, rows, 1)
        out = m.indice_conv_forward(gpu_handle, x, w, m.LAYOUT_ARRAY, pairs, num, rows, False, inverse=1)
        dx = m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, False, 64, inverse=1, rows=n_out)
        out_m = m.indice_conv_forward(gpu_handle, x, w, m.LAYOUT_ARRAY, pairs, num, rows, False, inverse=1,
                                      row_map=fwd_map)
        dx_m = m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, False, 64, inverse=1,
                                           rows=n_out, row_map=bwd_map)
        torch.cuda.synchronize()
        assert torch.equal(out, out_m) and torch.equal(dx, dx_m)
    finally:
        gpu_handle.set_extended_modes(False)


def test_refusals(gpu_handle):
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(54)
    space = (8, 10, 10)
    idx = random_voxels(rng, 1, space, 500, duplicates=60)
    pairs, num, n_out = rulebook(m, gpu_handle, idx, 1, space, (3, 3, 3), (1, 1, 1), True)
    rows = idx.shape[0]
    feats = torch.randn(rows, 32, device="cuda").half()
    w = (torch.randn(3, 3, 3, 32, 32, device="cuda") * 0.1).half()
    # repeated coordinates: several pairs of one offset share a result row, the map loses them
    lossy = m.RowMap(gpu_handle, pairs, num, n_out, rows, 1)
    assert lossy.lost_pairs > 0 and not lossy.usable
    with pytest.raises(m.MluOpError) as e:
        lossy.announce()
    assert e.value.status == m.STATUS_BAD_PARAM
    # the operator without a map still adds every pair (checked against the oracle elsewhere)
    m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, pairs, num, n_out, True)

    idx = random_voxels(rng, 1, space, 500)
    pairs, num, n_out = rulebook(m, gpu_handle, idx, 1, space, (3, 3, 3), (2, 2, 2), False)
    rows = idx.shape[0]
    feats = torch.randn(rows, 32, device="cuda").half()
    dy = torch.randn(n_out, 32, device="cuda").half()
    fwd_map = m.RowMap(gpu_handle, pairs, num, n_out, rows, 1)
    assert fwd_map.usable
    plain = m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, False, 32)
    with pytest.raises(m.MluOpError) as e:      # a forward map announced to backward data
        m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, False, 32, row_map=fwd_map)
    assert e.value.status == m.STATUS_BAD_PARAM
    # the refused call ended the announcement
    after = m.indice_conv_backward_data(gpu_handle, dy, w, m.LAYOUT_ARRAY, pairs, num, False, 32)
    torch.cuda.synchronize()
    assert torch.equal(after, plain)
    other_pairs = pairs.clone()
    with pytest.raises(m.MluOpError):           # the same map with another pair tensor
        m.indice_conv_forward(gpu_handle, feats, w, m.LAYOUT_ARRAY, other_pairs, num, n_out, False, row_map=fwd_map)
    fwd_map.close()
    gone = m.RowMap(gpu_handle, pairs, num, n_out, rows, 1)
    keep, address = gone.buffer, gone.buffer.data_ptr()
    gone.close()
    with pytest.raises(m.MluOpError):           # forgotten
        m.check(m.lib().mluOpExtUseRowMap(gpu_handle.ptr, address))
    del keep
    with pytest.raises(m.MluOpError):           # wrong shape for the column
        m.RowMap(gpu_handle, pairs, num, n_out + 1, rows + 1, 1)


def test_layers_with_known_distinct_coordinates_share_maps(gpu_handle):
    """With share_row_maps on, the caller layer builds one map per rulebook and direction: a tensor declared distinct gives
    the same values and gradients as one that is not (which runs the operators without maps)."""
    import torch
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(55)
    idx = torch.from_numpy(random_voxels(rng, 2, (12, 16, 16), 3000)).cuda()
    feats0 = torch.randn(idx.shape[0], 16, device="cuda")
    torch.manual_seed(0)
    net = torch.nn.ModuleList([spnn.SubMConv3d(16, 32, 3, indice_key="a"), spnn.SubMConv3d(32, 32, 3, indice_key="a"),
                               spnn.SparseConv3d(32, 64, 3, stride=2, padding=1, indice_key="d"),
                               spnn.SubMConv3d(64, 64, 3, indice_key="b")]).cuda().half()

    def run(distinct):
        f = feats0.clone().half().requires_grad_(True)
        x = spnn.SparseTensor(f, idx, (12, 16, 16), 2, distinct=distinct)
        for layer in net:
            x = layer(x)
        for p in net.parameters():
            p.grad = None
        x.features.float().square().sum().backward()
        return x.features.detach(), f.grad.detach(), [p.grad.detach().clone() for p in net.parameters()], x

    spnn.share_row_maps(True)
    try:
        out_a, gin_a, gw_a, x_a = run(False)
        out_b, gin_b, gw_b, x_b = run(True)
    finally:
        spnn.share_row_maps(False)
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b) and torch.equal(gin_a, gin_b)
    for a, b in zip(gw_a, gw_b):
        assert torch.equal(a, b)
    built = [rm for rb in x_b.rulebooks.values() for rm in rb._row_maps.values() if rm is not None]
    assert len(built) >= 4                      # two rulebooks seen so far, two directions each
    # the tensor that was not declared distinct ran its first stage without maps (the strided
    # layer's output never repeats a coordinate, so the stage behind it has them either way)
    assert len(x_a.rulebooks["a"]._row_maps) == 0 and len(x_b.rulebooks["a"]._row_maps) == 2
