"""Submanifold rulebooks from rows in strict cell order, which mluOpGetIndicePairs resolves by
searching the sorted cells instead of a hash table: geometries built to reach every branch of that
way (a wave's span copied to LDS, the per-lane search of waves whose span is too long, the mirrored
offsets of centred kernels, kernels that are not centred, the generic offset-by-offset probe) and
the inputs that must fall back to the table although they look sorted (equal neighbours, one
row a step back).  Everything is compared bit for bit with the CPU oracle."""
import numpy as np
import pytest

from test_gpu_rulebook import compare

pytestmark = pytest.mark.gpu


def sort_rows(idx):
    order = np.lexsort((idx[:, 3], idx[:, 2], idx[:, 1], idx[:, 0]))
    return np.ascontiguousarray(idx[order])


def cells_to_rows(lin, space, n=0):
    D, H, W = space
    lin = np.asarray(lin, dtype=np.int64)
    rem = lin % (D * H * W)
    return np.stack([np.full_like(lin, n), rem // (H * W), (rem % (H * W)) // W, rem % W], axis=1).astype(np.int32)


def thin_rows_next_to_a_dense_slab(rng, space, slab_d):
    """Every cell of plane d = slab_d, a few cells in the planes next to it: the 64 thin rows of a
    wave span a whole plane, and what they look for one plane further is the whole slab."""
    D, H, W = space
    rows = []
    for d in range(D):
        if d == slab_d:
            hh, ww = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
            rows.append(np.stack([np.zeros(H * W), np.full(H * W, d), hh.ravel(), ww.ravel()], axis=1))
        else:
            n = int(rng.integers(20, 70))
            lin = rng.choice(H * W, size=n, replace=False)
            rows.append(np.stack([np.zeros(n), np.full(n, d), lin // W, lin % W], axis=1))
    return sort_rows(np.concatenate(rows).astype(np.int32))


@pytest.mark.parametrize("ks", [(3, 3, 3), (5, 5, 5), (3, 3, 1), (1, 3, 5), (3, 5, 3)])
def test_waves_whose_span_is_longer_than_the_copy(gpu_handle, ks):
    rng = np.random.default_rng(71 + ks[0] + 3 * ks[2])
    space = (6, 40, 48)
    idx = thin_rows_next_to_a_dense_slab(rng, space, slab_d=3)
    pad = [k // 2 for k in ks]
    p, o, n, n_out = compare(gpu_handle, idx, 1, space, ks, pad, [1, 1, 1], [1, 1, 1], True)
    K = int(np.prod(ks))
    assert n[K // 2] == idx.shape[0] and np.array_equal(n, n[::-1])


@pytest.mark.parametrize("L", [1, 2, 63, 64, 65, 255, 256, 257, 4095, 4097, 70001])
def test_row_counts_around_the_wave_and_sample_boundaries(gpu_handle, L):
    rng = np.random.default_rng(72 + L)
    space = (12, 96, 96)
    lin = np.sort(rng.choice(space[0] * space[1] * space[2], size=L, replace=False))
    compare(gpu_handle, cells_to_rows(lin, space), 1, space, (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)


def test_first_and_last_cell_of_the_space(gpu_handle):
    """Rows at cell 0 and at the last cell: the lowest cell a group looks for lies below 0 there."""
    space = (5, 6, 7)
    total = space[0] * space[1] * space[2]
    for ks in [(3, 3, 3), (5, 5, 5), (1, 1, 3)]:
        pad = [k // 2 for k in ks]
        lin = np.array([0, 1, 2, 7, 8, 41, 42, 43, total - 9, total - 2, total - 1])
        compare(gpu_handle, cells_to_rows(lin, space), 1, space, ks, pad, [1, 1, 1], [1, 1, 1], True)
        compare(gpu_handle, cells_to_rows(np.arange(total), space), 1, space, ks, pad, [1, 1, 1], [1, 1, 1], True)


def test_batches_in_order(gpu_handle):
    rng = np.random.default_rng(73)
    space = (6, 20, 20)
    vol = space[0] * space[1] * space[2]
    rows = [cells_to_rows(np.sort(rng.choice(vol, size=700, replace=False)), space, n) for n in range(3)]
    compare(gpu_handle, np.ascontiguousarray(np.concatenate(rows)), 3, space, (3, 3, 3), [1, 1, 1], [1, 1, 1],
            [1, 1, 1], True)


@pytest.mark.parametrize("ks,pad,dil", [
    ((3, 3, 1), (1, 1, 0), (1, 1, 1)),   # one cell wide along w: offsets one by one, mirrored
    ((1, 1, 1), (0, 0, 0), (1, 1, 1)),   # a single offset: the centre alone
    ((2, 2, 2), (1, 1, 1), (1, 1, 1)),   # even edges: nothing to mirror
    ((3, 3, 3), (0, 1, 1), (1, 1, 1)),   # not centred along d
    ((4, 3, 3), (2, 1, 1), (1, 1, 1)),   # even edge along d
    ((3, 3, 5), (1, 1, 2), (1, 1, 1)),
])
def test_kernels_that_are_not_the_centred_cube(gpu_handle, ks, pad, dil):
    rng = np.random.default_rng(74 + ks[0] + pad[0])
    space = (10, 24, 30)
    lin = np.sort(rng.choice(space[0] * space[1] * space[2], size=2500, replace=False))
    compare(gpu_handle, cells_to_rows(lin, space), 1, space, ks, list(pad), [1, 1, 1], list(dil), True)


def test_rows_that_only_look_sorted_take_the_table(gpu_handle):
    """Two equal neighbours, or one row a step back: not in strict cell order, whatever the
    comparison of the other neighbouring rows says."""
    rng = np.random.default_rng(75)
    space = (8, 16, 16)
    lin = np.sort(rng.choice(space[0] * space[1] * space[2], size=900, replace=False))
    idx = cells_to_rows(lin, space)
    twice = np.ascontiguousarray(np.concatenate([idx[:400], idx[399:400], idx[400:]]))   # row 399 twice
    compare(gpu_handle, twice, 1, space, (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    twice_at_end = np.ascontiguousarray(np.concatenate([idx, idx[-1:]]))
    compare(gpu_handle, twice_at_end, 1, space, (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    one_step_back = idx.copy()
    one_step_back[[500, 501]] = one_step_back[[501, 500]]
    compare(gpu_handle, one_step_back, 1, space, (3, 3, 3), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
