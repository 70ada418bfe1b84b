"""Pins of the CPU oracle's rulebook (oracle/sparse_conv_oracle.c, restating reference
zoo/get_indice_pairs/get_indice_pairs.cpp:177-406) that do not reuse its own formulas:

* brute force straight from the definition of a sparse convolution (enumerate every output cell
  and kernel offset, input = output*stride - pad + offset*dilation) on tiny grids;
* closed form on a fully occupied block;
* submanifold symmetry and centre-offset identities;
* regular-mode invariants (ascending out_indices, dense input covers the whole output grid).
"""
import itertools

import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import out_space, random_voxels


def brute_force_rulebook(idx, batch, space, ks, pad, stride, dil, sub_m):
    """Definition-level rulebook: loops over OUTPUT cells and offsets (the oracle loops over inputs)."""
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    L = idx.shape[0]
    K = int(np.prod(ks))
    cell_to_row = {}
    for j, (n, d, h, w) in enumerate(idx.tolist()):
        cell_to_row[(n, d, h, w)] = j  # later rows overwrite earlier ones
    triples = []  # (k, input row, output cell)
    for n in range(batch):
        for od, oh, ow in itertools.product(range(ospace[0]), range(ospace[1]), range(ospace[2])):
            for kd, kh, kw in itertools.product(range(ks[0]), range(ks[1]), range(ks[2])):
                i = (od * stride[0] - pad[0] + kd * dil[0], oh * stride[1] - pad[1] + kh * dil[1],
                     ow * stride[2] - pad[2] + kw * dil[2])
                k = (kd * ks[1] + kh) * ks[2] + kw
                for j, row in enumerate(idx.tolist()):  # every row at that input cell (duplicates too)
                    if tuple(row) == (n,) + i:
                        triples.append((k, j, (n, od, oh, ow)))
    if sub_m:
        triples = [(k, j, cell_to_row[c]) for k, j, c in triples if c in cell_to_row]
        out_rows = idx.copy()
        n_out = L
    else:
        cells = sorted({c for _, _, c in triples})
        rank = {c: r for r, c in enumerate(cells)}
        triples = [(k, j, rank[c]) for k, j, c in triples]
        out_rows = np.array(cells, dtype=np.int32).reshape(-1, 4)
        n_out = len(cells)
    pairs = np.full((K, 2, L), -1, dtype=np.int32)
    num = np.zeros(K, dtype=np.int32)
    for k, j, o in sorted(triples):  # ascending input row inside an offset
        pairs[k, 0, num[k]] = j
        pairs[k, 1, num[k]] = o
        num[k] += 1
    return pairs, out_rows, num, n_out


CASES = []
for seed, (batch, space, L, ks, pad, stride, dil, sub_m) in enumerate([
    (1, (3, 3, 3), 10, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),
    (2, (4, 3, 5), 30, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),
    (1, (4, 4, 4), 20, (1, 3, 5), (0, 1, 2), (1, 1, 1), (1, 1, 1), True),
    (1, (5, 5, 5), 40, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1), False),
    (2, (5, 4, 6), 50, (3, 3, 3), (0, 1, 2), (1, 2, 3), (1, 1, 1), False),
    (1, (6, 6, 6), 60, (3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2), False),
    (1, (6, 5, 4), 45, (2, 2, 2), (0, 0, 0), (2, 2, 2), (1, 1, 1), False),
    (1, (5, 5, 5), 30, (3, 2, 1), (1, 0, 0), (1, 1, 1), (1, 2, 1), False),
    (1, (4, 4, 4), 64, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), False),
    (2, (3, 4, 3), 25, (3, 3, 3), (0, 0, 0), (3, 1, 2), (1, 1, 1), False),
]):
    CASES.append((seed, batch, space, L, ks, pad, stride, dil, sub_m))


@pytest.mark.parametrize("case", CASES)
def test_oracle_matches_definition_level_brute_force(case):
    seed, batch, space, L, ks, pad, stride, dil, sub_m = case
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, batch, space, L)
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    bp, bo, bn, bn_out = brute_force_rulebook(idx, batch, space, ks, pad, stride, dil, sub_m)
    op, oo, on, on_out = oracle.get_indice_pairs(idx, batch, list(pad), list(stride), list(dil), list(ks), ospace,
                                                 sub_m, out_rows=max(bn_out, 1), exact_count=True)
    assert on_out == bn_out
    assert np.array_equal(on, bn)
    assert np.array_equal(op, bp)
    assert np.array_equal(oo[:bn_out], bo[:bn_out])
    if not sub_m and on.sum() < on.size * idx.shape[0]:
        # with at least one invalid (input, offset) the reference's "distinct minus sentinel" count agrees
        _, _, _, quirk = oracle.get_indice_pairs(idx, batch, list(pad), list(stride), list(dil), list(ks), ospace,
                                                 sub_m, out_rows=max(bn_out, 1), exact_count=False)
        assert quirk == bn_out


def test_subm_duplicate_coordinates_last_row_wins():
    idx = np.array([[0, 1, 1, 1], [0, 1, 1, 2], [0, 1, 1, 1]], dtype=np.int32)
    bp, _, bn, _ = brute_force_rulebook(idx, 1, (3, 3, 3), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True)
    op, oo, on, _ = oracle.get_indice_pairs(idx, 1, [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], [3, 3, 3], True)
    assert np.array_equal(op, bp) and np.array_equal(on, bn)
    # centre offset: rows 0 and 2 share a cell, both map to row 2
    assert op[13, 1, :3].tolist() == [2, 1, 2]
    assert np.array_equal(oo, idx)


@pytest.mark.parametrize("block", [(2, 3, 4), (4, 4, 4), (1, 5, 2)])
def test_subm_full_block_closed_form(block):
    """Fully occupied a x b x c block, 3x3x3 pad 1: offset (dz,dy,dx) has (a-|dz|)(b-|dy|)(c-|dx|) pairs."""
    a, b, c = block
    cells = np.array([[0, z, y, x] for z in range(a) for y in range(b) for x in range(c)], dtype=np.int32)
    space = (a + 2, b + 1, c + 3)  # block sits at the corner of a larger grid
    p, o, n, n_out = oracle.get_indice_pairs(cells, 1, [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], list(space), True)
    for kd, kh, kw in itertools.product(range(3), repeat=3):
        expect = max(a - abs(kd - 1), 0) * max(b - abs(kh - 1), 0) * max(c - abs(kw - 1), 0)
        assert n[(kd * 3 + kh) * 3 + kw] == expect
    assert n_out == cells.shape[0]


@pytest.mark.parametrize("seed", range(4))
def test_subm_symmetry_and_centre_identity(seed):
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, 2, (7, 8, 9), 250)
    L = idx.shape[0]
    p, o, n, _ = oracle.get_indice_pairs(idx, 2, [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], [7, 8, 9], True)
    K = 27
    assert n[13] == L
    assert np.array_equal(p[13, 0, :L], np.arange(L)) and np.array_equal(p[13, 1, :L], np.arange(L))
    assert np.array_equal(n, n[::-1])
    for k in range(K):
        fwd = set(zip(p[k, 0, :n[k]].tolist(), p[k, 1, :n[k]].tolist()))
        rev = set(zip(p[K - 1 - k, 1, :n[K - 1 - k]].tolist(), p[K - 1 - k, 0, :n[K - 1 - k]].tolist()))
        assert fwd == rev
        assert np.all(np.diff(p[k, 0, :n[k]]) > 0)
        assert np.all(p[k, :, n[k]:] == -1)
    assert np.array_equal(o, idx)


@pytest.mark.parametrize("stride,pad,ks", [((2, 2, 2), (1, 1, 1), (3, 3, 3)), ((1, 1, 1), (0, 0, 0), (2, 2, 2)),
                                           ((2, 2, 2), (0, 0, 0), (2, 2, 2))])
def test_regular_invariants(stride, pad, ks):
    rng = np.random.default_rng(7)
    space = (8, 9, 10)
    idx = random_voxels(rng, 2, space, 300)
    L = idx.shape[0]
    osp = out_space(space, ks, pad, stride, (1, 1, 1))
    p, o, n, n_out = oracle.get_indice_pairs(idx, 2, list(pad), list(stride), [1, 1, 1], list(ks), osp, False,
                                             exact_count=True)
    lin = ((o[:n_out, 0] * osp[0] + o[:n_out, 1]) * osp[1] + o[:n_out, 2]) * osp[2] + o[:n_out, 3]
    assert np.all(np.diff(lin) > 0)
    assert np.all(o[n_out:] == -1)
    K = int(np.prod(ks))
    used = set()
    for k in range(K):
        assert np.all(np.diff(p[k, 0, :n[k]]) > 0)
        assert np.all((p[k, 1, :n[k]] >= 0) & (p[k, 1, :n[k]] < n_out))
        assert len(set(p[k, 1, :n[k]].tolist())) == n[k]  # one input per output inside an offset
        assert np.all(p[k, :, n[k]:] == -1)
        used.update(p[k, 1, :n[k]].tolist())
    assert used == set(range(n_out))
    # total pair count = number of (input, offset) combinations that land on a valid output cell
    total = 0
    for row in idx.tolist():
        for kk in itertools.product(range(ks[0]), range(ks[1]), range(ks[2])):
            ok = True
            for a in range(3):
                num = row[1 + a] + pad[a] - kk[a]
                if num < 0 or num % stride[a] or num // stride[a] >= osp[a]:
                    ok = False
            total += ok
    assert n.sum() == total


def test_regular_dense_input_covers_output_grid():
    space = (4, 5, 6)
    cells = np.array([[n, z, y, x] for n in range(2) for z in range(4) for y in range(5) for x in range(6)],
                     dtype=np.int32)
    osp = out_space(space, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1))
    p, o, n, n_out = oracle.get_indice_pairs(cells, 2, [1, 1, 1], [2, 2, 2], [1, 1, 1], [3, 3, 3], osp, False,
                                             exact_count=True)
    assert n_out == 2 * osp[0] * osp[1] * osp[2]


def test_reference_count_quirk_when_every_combination_is_valid():
    """1x1x1 kernel, stride 1: every (input, offset) is valid, no sentinel is left in the candidate
    list and the reference's `distinct - 1` (get_indice_pairs.cpp:380) drops the last output."""
    idx = np.array([[0, 0, 0, 0], [0, 1, 1, 1], [0, 2, 2, 2]], dtype=np.int32)
    _, _, _, quirk = oracle.get_indice_pairs(idx, 1, [0, 0, 0], [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], False,
                                             exact_count=False)
    _, _, _, exact = oracle.get_indice_pairs(idx, 1, [0, 0, 0], [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], False,
                                             exact_count=True)
    assert exact == 3 and quirk == 2
