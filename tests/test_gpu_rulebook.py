"""GPU parity of mluOpGetIndicePairs against the CPU oracle: every output tensor must be
bit-exact (reference accuracy rule: diff3 == 0 for indice_pairs, out_indices, indice_num)."""
import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import out_space, random_voxels

pytestmark = pytest.mark.gpu


def run_gpu(handle, idx, batch, space, ks, ospace, pad, stride, dil, sub_m, out_rows=None):
    import torch
    import mluop_hip
    t = torch.from_numpy(idx).cuda()
    pairs, out_idx, num, n_out = mluop_hip.get_indice_pairs(
        handle, t, batch, space, ks, ospace, pad, stride, dil, sub_m, out_rows=out_rows)
    torch.cuda.synchronize()
    return pairs.cpu().numpy(), out_idx.cpu().numpy(), num.cpu().numpy(), n_out


def compare(handle, idx, batch, space, ks, pad, stride, dil, sub_m, out_rows=None):
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    p, o, n, n_out = run_gpu(handle, idx, batch, space, ks, ospace, pad, stride, dil, sub_m, out_rows)
    rows = o.shape[0]
    rp, ro, rn, rn_out = oracle.get_indice_pairs(idx, batch, pad, stride, dil, ks, ospace, sub_m,
                                                 out_rows=rows, exact_count=True)
    assert np.array_equal(n, rn), "indice_num"
    assert np.array_equal(p, rp), "indice_pairs"
    assert np.array_equal(o, ro), "out_indices"
    assert n_out == rn_out
    return p, o, n, n_out


SUBM_CASES = [
    # (batch, space, L, ks, shuffle, duplicates, seed)
    (1, (4, 5, 6), 1, (3, 3, 3), True, 0, 0),
    (1, (4, 5, 6), 60, (3, 3, 3), True, 0, 1),
    (2, (6, 7, 9), 300, (3, 3, 3), True, 0, 2),
    (2, (6, 7, 9), 300, (3, 3, 3), False, 0, 3),
    (3, (8, 8, 8), 700, (3, 3, 3), True, 40, 4),
    (1, (10, 12, 14), 1000, (5, 5, 5), True, 0, 5),
    (1, (9, 9, 9), 400, (1, 3, 5), True, 0, 6),
    (1, (16, 32, 32), 5000, (3, 3, 3), True, 0, 7),
    (1, (5, 5, 5), 125, (3, 3, 3), False, 0, 8),  # full block
    (1, (3, 70, 70), 257, (3, 3, 3), True, 0, 9),
]


@pytest.mark.parametrize("case", SUBM_CASES)
def test_subm_rulebook_matches_oracle(gpu_handle, case):
    batch, space, L, ks, shuffle, dup, seed = case
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, batch, space, L, shuffle=shuffle, duplicates=dup)
    pad = [k // 2 for k in ks]
    print("subm case", case, flush=True)
    p, o, n, n_out = compare(gpu_handle, idx, batch, space, ks, pad, [1, 1, 1], [1, 1, 1], True)
    K = int(np.prod(ks))
    if dup == 0:
        assert n[K // 2] == idx.shape[0]
        assert np.array_equal(n, n[::-1])


SUBM_GEOMETRY_CASES = [
    # (batch, space, L, ks, pad, dil, duplicates, seed): submanifold layers off the 3x3x3 / dilation 1 path
    (2, (9, 9, 40), 900, (3, 3, 3), (1, 1, 1), (1, 1, 1), 60, 22),    # long W rows: runs of 16 cells, duplicates
    (1, (4, 4, 100), 1200, (3, 3, 3), (1, 1, 1), (1, 1, 1), 0, 23),   # 75 % dense: long probe sequences
    (1, (10, 10, 10), 400, (6, 5, 5), (3, 2, 2), (1, 1, 1), 0, 24),   # K = 150 > 128: offsets decoded by division
    (1, (10, 10, 10), 400, (3, 3, 3), (0, 1, 1), (1, 1, 1), 0, 25),   # pad 0 on one axis: asymmetric window
]


@pytest.mark.parametrize("case", SUBM_GEOMETRY_CASES)
def test_subm_rulebook_other_geometries(gpu_handle, case):
    batch, space, L, ks, pad, dil, dup, seed = case
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, batch, space, L, shuffle=True, duplicates=dup)
    print("subm geometry case", case, flush=True)
    compare(gpu_handle, idx, batch, space, ks, list(pad), [1, 1, 1], list(dil), True)


def test_subm_with_dilation_is_rejected_like_the_reference(gpu_handle):
    """Submanifold mode requires stride 1 and dilation 1 (the reference's parameter check)."""
    import mluop_hip
    rng = np.random.default_rng(26)
    idx = random_voxels(rng, 1, (8, 8, 8), 100)
    with pytest.raises(mluop_hip.MluOpError) as e:
        run_gpu(gpu_handle, idx, 1, (8, 8, 8), (3, 3, 3), [8, 8, 8], [2, 2, 2], [1, 1, 1], [2, 2, 2], True)
    assert e.value.status == mluop_hip.STATUS_BAD_PARAM


REGULAR_CASES = [
    # (batch, space, L, ks, pad, stride, dil, seed)
    (1, (6, 6, 6), 40, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1), 0),
    (2, (9, 10, 11), 300, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1), 1),
    (2, (9, 10, 11), 300, (3, 3, 3), (0, 1, 1), (2, 1, 2), (1, 1, 1), 2),
    (1, (12, 12, 12), 500, (3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2), 3),
    (1, (12, 12, 12), 500, (2, 2, 2), (0, 0, 0), (2, 2, 2), (1, 1, 1), 4),
    (3, (8, 16, 16), 1500, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 5),
    (1, (7, 9, 13), 200, (1, 3, 2), (0, 1, 0), (1, 3, 2), (1, 1, 1), 6),
    (1, (16, 40, 40), 6000, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1), 7),
    (1, (10, 10, 10), 300, (3, 1, 3), (1, 0, 2), (1, 2, 1), (1, 1, 2), 8),
]


@pytest.mark.parametrize("case", REGULAR_CASES)
def test_regular_rulebook_matches_oracle(gpu_handle, case):
    batch, space, L, ks, pad, stride, dil, seed = case
    rng = np.random.default_rng(100 + seed)
    idx = random_voxels(rng, batch, space, L, shuffle=True)
    print("regular case", case, flush=True)
    p, o, n, n_out = compare(gpu_handle, idx, batch, space, ks, list(pad), list(stride), list(dil), False)
    K = int(np.prod(ks))
    assert n.sum() < K * idx.shape[0]  # at least one invalid (input, offset): oracle count quirk not hit
    lin_space = out_space(space, ks, pad, stride, dil)
    lin = ((o[:n_out, 0] * lin_space[0] + o[:n_out, 1]) * lin_space[1] + o[:n_out, 2]) * lin_space[2] + o[:n_out, 3]
    assert np.all(np.diff(lin) > 0)


def test_regular_rulebook_in_a_grid_of_many_bitmap_blocks(gpu_handle):
    """2 x 41 x 1024 x 1024 output cells at stride 1: a bitmap of more than 5000 blocks of 256 words,
    whose per-block counts are scanned by a launch of their own instead of summed by every workgroup."""
    rng = np.random.default_rng(131)
    space = (41, 1024, 1024)
    idx = random_voxels(rng, 2, space, 20000, shuffle=True)
    print("regular many blocks", flush=True)
    p, o, n, n_out = compare(gpu_handle, idx, 2, space, (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], False)
    assert n_out > 20000


def test_regular_mode_leaves_the_rows_behind_the_active_outputs_alone(gpu_handle):
    """Like the reference's decode kernel (normal_get_indice_pairs.cpp:1143-1150), which is launched
    over num_act_out rows, the operator writes no row of out_indices from num_act_out on."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(132)
    space, ks = (9, 40, 40), (3, 3, 3)
    idx = random_voxels(rng, 2, space, 900, shuffle=True)
    ospace = out_space(space, ks, (1, 1, 1), (2, 2, 2), (1, 1, 1))
    mine = torch.full((2 * int(np.prod(ospace)), 4), 12345, dtype=torch.int32, device="cuda")
    _, o, _, n_out = mluop_hip.get_indice_pairs(gpu_handle, torch.from_numpy(idx).cuda(), 2, space, ks, ospace,
                                               [1, 1, 1], [2, 2, 2], [1, 1, 1], False, out_indices=mine)
    torch.cuda.synchronize()
    o = o.cpu().numpy()
    _, ro, _, rn_out = oracle.get_indice_pairs(idx, 2, [1, 1, 1], [2, 2, 2], [1, 1, 1], list(ks), ospace, False,
                                               out_rows=o.shape[0], exact_count=True)
    assert n_out == rn_out and 0 < n_out < o.shape[0]
    assert np.array_equal(o[:n_out], ro[:n_out])
    assert np.all(o[n_out:] == 12345)


def test_regular_out_indices_smaller_tensor_is_rejected_cleanly(gpu_handle):
    """A caller-supplied out_indices with fewer rows than active outputs must not be overrun."""
    import mluop_hip
    rng = np.random.default_rng(5)
    idx = random_voxels(rng, 1, (8, 8, 8), 200)
    ospace = out_space((8, 8, 8), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    with pytest.raises(mluop_hip.MluOpError) as e:
        run_gpu(gpu_handle, idx, 1, (8, 8, 8), (3, 3, 3), ospace, [1, 1, 1], [1, 1, 1], [1, 1, 1], False,
                out_rows=10)
    assert e.value.status == mluop_hip.STATUS_BAD_PARAM


def test_config1_subm_rulebook_full_size(gpu_handle):
    """BASELINE config 1: 20 000 uniform voxels in 1x40x400x352, subm 3x3x3."""
    import mluop_hip
    idx = mluop_hip.datagen.uniform_voxels((1, 40, 400, 352), 20000, seed=1)
    compare(gpu_handle, idx, 1, (40, 400, 352), (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)


def test_config4_subm_rulebook_full_size(gpu_handle):
    """BASELINE config 4 (headline): 120 000 clustered voxels in 1x41x1600x1408, sorted and shuffled."""
    import mluop_hip
    for shuffle in (False, True):
        idx = mluop_hip.datagen.clustered_voxels((1, 41, 1600, 1408), 120000, seed=4, shuffle=shuffle)
        print("config4 shuffle", shuffle, flush=True)
        compare(gpu_handle, idx, 1, (41, 1600, 1408), (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)


def test_config3_regular_rulebook_full_size(gpu_handle):
    """BASELINE config 3: 4 x 30 000 clustered voxels in 4x41x1600x1408, 3x3x3 stride 2 pad 1."""
    import mluop_hip
    idx = mluop_hip.datagen.clustered_voxels((4, 41, 1600, 1408), 30000, seed=3)
    compare(gpu_handle, idx, 4, (41, 1600, 1408), (3, 3, 3), [1, 1, 1], [2, 2, 2], [1, 1, 1], False)


@pytest.mark.timeout(600)
def test_largest_accepted_input_one_million_rows(gpu_handle):
    """L = 1 000 000, the most rows the API accepts (INDICE_IN_LARGE_TENSOR_NUM), submanifold and
    regular stride 2, in a grid of 2 x 48 x 512 x 512 cells (density 4 %)."""
    rng = np.random.default_rng(77)
    space = (48, 512, 512)
    idx = random_voxels(rng, 2, space, 1000000)
    print("subm 1M", flush=True)
    compare(gpu_handle, idx, 2, space, (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    print("regular 1M", flush=True)
    compare(gpu_handle, idx, 2, space, (2, 2, 2), [0, 0, 0], [2, 2, 2], [1, 1, 1], False)


@pytest.mark.parametrize("sub_m", [True, False])
def test_indices_that_are_not_16_byte_aligned(gpu_handle, sub_m):
    """The (n, d, h, w) rows are read with one 16-byte load each when the tensor allows it; a tensor
    at an odd address takes the element-wise path and gives the same rulebook."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(51)
    batch, space, ks = 2, (8, 9, 10), (3, 3, 3)
    idx = random_voxels(rng, batch, space, 500)
    pad, stride, dil = [1, 1, 1], ([1, 1, 1] if sub_m else [2, 2, 2]), [1, 1, 1]
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    flat = torch.empty(idx.size + 8, dtype=torch.int32, device="cuda")
    t = flat[1:1 + idx.size].view(idx.shape)
    t.copy_(torch.from_numpy(idx))
    assert t.data_ptr() % 16 != 0
    pairs, out_idx, num, n_out = mluop_hip.get_indice_pairs(gpu_handle, t, batch, space, ks, ospace, pad, stride, dil,
                                                           sub_m)
    torch.cuda.synchronize()
    rp, ro, rn, rn_out = oracle.get_indice_pairs(idx, batch, pad, stride, dil, ks, ospace, sub_m,
                                                 out_rows=out_idx.shape[0], exact_count=True)
    assert n_out == rn_out and np.array_equal(num.cpu().numpy(), rn)
    assert np.array_equal(pairs.cpu().numpy(), rp) and np.array_equal(out_idx.cpu().numpy(), ro)
