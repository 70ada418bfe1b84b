"""Forward and backward data reading the pair lists cut by tile instead of a row map.

The operators take that way when the handle built the rulebook itself (mluOpGetIndicePairs) and,
for the pair column that follows the output rows, when the rulebook's report says the input rows
were in cell order.  Every case builds its rulebook on the GPU, waits for the queue (as the caller
who copies indice_num to the host does), checks through the per-kernel timer which kernels ran, and
grades the results against the CPU oracle like the other operator tests."""
import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import check_close, from_torch, out_space, random_voxels, round_to, to_torch

pytestmark = pytest.mark.gpu

LIST_KERNEL = "packFilterCutPairLists"
MAP_KERNELS = ("fillMapPackFilter", "scatterRowMap", "fillInt32")


def gpu_rulebook(handle, idx, batch, space, ks, pad, stride, dil, sub_m):
    import torch
    import mluop_hip
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    pairs, out_idx, num, n_out = mluop_hip.get_indice_pairs(handle, torch.from_numpy(idx).cuda(), batch, space, ks,
                                                           ospace, pad, stride, dil, sub_m)
    torch.cuda.synchronize()
    return pairs, [int(v) for v in num.cpu().tolist()], n_out


def kernels_of(handle, fn):
    """Runs fn with the per-kernel timer on; returns (result, names of the kernels it launched)."""
    handle.set_kernel_timing(True)
    try:
        res = fn()
        names = [n for n, _ in handle.kernel_timings()]
    finally:
        handle.set_kernel_timing(False)
    return res, names


def run_case(handle, seed, batch, space, L, ks, ci, co, dtype_name, sub_m, shuffle, stride=(1, 1, 1),
             expect_forward_lists=None):
    import torch
    import mluop_hip
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, batch, space, L, shuffle=shuffle)
    pad = [k // 2 for k in ks]
    pairs, num, n_out = gpu_rulebook(handle, idx, batch, space, ks, pad, list(stride), [1, 1, 1], sub_m)
    K = int(np.prod(ks))
    feats = round_to(rng.standard_normal((idx.shape[0], ci)).astype(np.float32), dtype_name)
    b = 1.0 / np.sqrt(K * ci)
    w = round_to(rng.uniform(-b, b, size=tuple(ks) + (ci, co)).astype(np.float32), dtype_name)
    dy = round_to((rng.standard_normal((n_out, co)) * 0.1).astype(np.float32), dtype_name)
    pairs_np = pairs.cpu().numpy()
    w_k = w.reshape(K, ci, co)
    t_f, t_w, t_dy = (to_torch(a, dtype_name, "cuda") for a in (feats, w, dy))

    out, names = kernels_of(handle, lambda: mluop_hip.indice_conv_forward(
        handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, pairs, num, n_out, sub_m))
    torch.cuda.synchronize()
    if expect_forward_lists is None:
        expect_forward_lists = not shuffle
    assert (LIST_KERNEL in names) == expect_forward_lists, names
    check_close(from_torch(out), oracle.forward(feats, w_k, pairs_np, num, n_out), dtype_name, "forward")

    dx, names = kernels_of(handle, lambda: mluop_hip.indice_conv_backward_data(
        handle, t_dy, t_w, mluop_hip.LAYOUT_ARRAY, pairs, num, sub_m, ci))
    torch.cuda.synchronize()
    # the input-row column of a rulebook the handle built ascends whatever the row order
    assert LIST_KERNEL in names and not any(k in names for k in MAP_KERNELS), names
    check_close(from_torch(dx), oracle.backward_data(dy, w_k, pairs_np, num), dtype_name, "backward_data")


SHAPES = [
    # batch, space, rows, kernel, Ci, Co, sub_m
    (1, (10, 30, 30), 3000, (3, 3, 3), 64, 64, True),
    (2, (8, 24, 24), 2500, (3, 3, 3), 32, 64, True),
    (1, (9, 20, 20), 2600, (3, 3, 3), 16, 32, True),
    (1, (8, 16, 16), 1500, (3, 3, 3), 128, 128, True),   # dense enough for the register-accumulating kernel
    (1, (12, 40, 40), 2000, (3, 3, 3), 128, 128, True),  # sparse: two 64-column halves
    (1, (12, 24, 24), 4000, (3, 3, 3), 64, 16, True),
]


@pytest.mark.parametrize("dtype_name", ["float16", "bfloat16", "float32"])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("shuffle", [False, True])
def test_submanifold_layers(gpu_handle, shape, dtype_name, shuffle):
    batch, space, L, ks, ci, co, sub_m = shape
    run_case(gpu_handle, 100 + L + ci, batch, space, L, ks, ci, co, dtype_name, sub_m, shuffle)


@pytest.mark.parametrize("dtype_name", ["float16", "float32"])
@pytest.mark.parametrize("shuffle", [False, True])
def test_strided_layer(gpu_handle, dtype_name, shuffle):
    run_case(gpu_handle, 7, 2, (11, 21, 23), 3500, (3, 3, 3), 32, 64, dtype_name, False, shuffle, stride=(2, 2, 2))
    run_case(gpu_handle, 8, 1, (16, 32, 32), 6000, (2, 2, 2), 64, 64, dtype_name, False, shuffle, stride=(2, 2, 2))


def test_five_wide_kernel_runs_in_several_chunks_of_offsets(gpu_handle):
    """125 offsets: two offsets per lane in the list kernels, five chunks of offsets per tile."""
    run_case(gpu_handle, 9, 1, (12, 24, 24), 3000, (5, 5, 5), 32, 32, "float16", True, False)
    run_case(gpu_handle, 10, 1, (10, 12, 12), 1400, (5, 5, 5), 64, 64, "float16", True, True)


def test_a_layer_whose_last_tile_is_short_and_one_that_is_a_single_tile(gpu_handle):
    run_case(gpu_handle, 11, 1, (6, 12, 12), 129, (3, 3, 3), 64, 64, "float16", True, False)
    run_case(gpu_handle, 12, 1, (6, 12, 12), 5, (3, 3, 3), 64, 64, "float16", True, False)
    run_case(gpu_handle, 13, 1, (6, 12, 12), 864, (3, 3, 3), 64, 64, "float16", True, False)  # every cell active


def test_repeated_coordinates_take_the_row_map(gpu_handle):
    """Repeated input rows are not in strict cell order: forward uses the map and its collision repair;
    backward data still reads the lists (its result rows are the input rows)."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(14)
    idx = random_voxels(rng, 1, (8, 20, 20), 1500, shuffle=False, duplicates=200)
    idx = idx[np.lexsort((idx[:, 3], idx[:, 2], idx[:, 1], idx[:, 0]))]  # sorted, equal rows adjacent
    idx = np.ascontiguousarray(idx)
    pairs, num, n_out = gpu_rulebook(gpu_handle, idx, 1, (8, 20, 20), (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    feats = round_to(rng.standard_normal((idx.shape[0], 32)).astype(np.float32), "float16")
    w = round_to(rng.uniform(-0.1, 0.1, size=(3, 3, 3, 32, 32)).astype(np.float32), "float16")
    out, names = kernels_of(gpu_handle, lambda: mluop_hip.indice_conv_forward(
        gpu_handle, to_torch(feats, "float16", "cuda"), to_torch(w, "float16", "cuda"), mluop_hip.LAYOUT_ARRAY,
        pairs, num, n_out, True))
    torch.cuda.synchronize()
    assert LIST_KERNEL not in names, names
    check_close(from_torch(out), oracle.forward(feats, w.reshape(27, 32, 32), pairs.cpu().numpy(), num, n_out),
                "float16", "forward with repeated rows")


@pytest.mark.parametrize("channels", [(64, 64), (128, 128), (32, 16)])
def test_a_pair_tensor_changed_behind_the_library_is_still_computed_right(gpu_handle, channels):
    """The handle saw a rulebook in order at this address; the caller then writes another rulebook (of
    shuffled rows) into the same tensor.  The operators start on the lists, find them out of order on
    the device and collect every tile's pairs by reading all of them."""
    import torch
    import mluop_hip
    ci, co = channels
    rng = np.random.default_rng(15)
    space, ks = (8, 20, 20), (3, 3, 3)
    idx = random_voxels(rng, 1, space, 1800, shuffle=False)
    pairs, num, n_out = gpu_rulebook(gpu_handle, idx, 1, space, ks, [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    perm = rng.permutation(idx.shape[0])
    idx2 = np.ascontiguousarray(idx[perm])
    rp, _, rn, _ = oracle.get_indice_pairs(idx2, 1, [1, 1, 1], [1, 1, 1], [1, 1, 1], list(ks), list(space), True)
    assert [int(v) for v in rn] == num   # the same cells: the same number of pairs at every offset
    pairs.copy_(torch.from_numpy(rp).cuda())
    feats = round_to(rng.standard_normal((idx.shape[0], ci)).astype(np.float32), "float16")
    w = round_to(rng.uniform(-0.1, 0.1, size=tuple(ks) + (ci, co)).astype(np.float32), "float16")
    out, names = kernels_of(gpu_handle, lambda: mluop_hip.indice_conv_forward(
        gpu_handle, to_torch(feats, "float16", "cuda"), to_torch(w, "float16", "cuda"), mluop_hip.LAYOUT_ARRAY,
        pairs, num, n_out, True))
    torch.cuda.synchronize()
    assert LIST_KERNEL in names, names
    check_close(from_torch(out), oracle.forward(feats, w.reshape(27, ci, co), rp, num, n_out), "float16",
                "forward on lists out of order")
    # entries out of range are refused the same way: every pair list ends early with -1
    broken = rp.copy()
    broken[:, :, 3] = -1
    pairs.copy_(torch.from_numpy(broken).cuda())
    out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats, "float16", "cuda"), to_torch(w, "float16", "cuda"),
                                        mluop_hip.LAYOUT_ARRAY, pairs, num, n_out, True)
    torch.cuda.synchronize()
    check_close(from_torch(out), oracle.forward(feats, w.reshape(27, ci, co), broken, num, n_out), "float16",
                "forward on lists with holes")


def test_a_rulebook_from_elsewhere_takes_the_row_map():
    """A pair tensor the handle did not build (here: the oracle's) is not assumed to be in order.
    (A handle of its own: what an older handle noted about a reused address must not matter here.)"""
    import torch
    import mluop_hip
    gpu_handle = mluop_hip.make_handle_on_current_stream()
    rng = np.random.default_rng(16)
    space, ks = (8, 20, 20), (3, 3, 3)
    idx = random_voxels(rng, 1, space, 1500, shuffle=False)
    rp, _, rn, n_out = oracle.get_indice_pairs(idx, 1, [1, 1, 1], [1, 1, 1], [1, 1, 1], list(ks), list(space), True)
    num = [int(v) for v in rn]
    feats = round_to(rng.standard_normal((idx.shape[0], 32)).astype(np.float32), "float16")
    w = round_to(rng.uniform(-0.1, 0.1, size=tuple(ks) + (32, 32)).astype(np.float32), "float16")
    out, names = kernels_of(gpu_handle, lambda: mluop_hip.indice_conv_forward(
        gpu_handle, to_torch(feats, "float16", "cuda"), to_torch(w, "float16", "cuda"), mluop_hip.LAYOUT_ARRAY,
        torch.from_numpy(rp).cuda(), num, n_out, True))
    torch.cuda.synchronize()
    assert LIST_KERNEL not in names, names
    check_close(from_torch(out), oracle.forward(feats, w.reshape(27, 32, 32), rp, num, n_out), "float16", "forward")
    gpu_handle.close()
