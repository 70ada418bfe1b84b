"""Pins the dynamic point-to-voxel oracle against the two case files the reference ships for the
operator (inputs and expected outputs, bit patterns included) and against numpy.unique."""
import os

import numpy as np
import pytest

import dynamic_point_to_voxel_oracle as dpv

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dynamic_point_to_voxel_forward")


def load_case(name):
    from mluop_hip import casefile as cf
    node, _ = cf.load(os.path.join(GOLDEN, name))
    ins = [cf.CaseTensor(t) for t in node.all("input")]
    outs = [cf.CaseTensor(t) for t in node.all("output")]
    mode = str(node.get("dynamic_point_to_voxel_forward_param").get("reduce_type"))
    return {"REDUCE_MODE_MAX": "max", "REDUCE_MODE_MEAN": "mean"}[mode], ins, outs


@pytest.mark.parametrize("name", ["case_0.prototxt", "case_1.prototxt"])
def test_reference_case_files(name):
    mode, ins, outs = load_case(name)
    rows = outs[0].shape[0]
    vf, vc, p2v, cnt, num, _ = dpv.forward(mode, ins[0].values, ins[1].values, rows=rows)
    want_num = int(outs[4].values[0])
    assert num == want_num
    assert np.array_equal(p2v, outs[2].values)
    assert np.array_equal(vc[:num], outs[1].values[:num])
    assert np.array_equal(cnt[:num], outs[3].values[:num])
    if mode == "max":
        assert np.array_equal(vf[:num], outs[0].values[:num])
    else:
        # the stored means come from another summation: graded as the case file asks (3e-3),
        # and far tighter than that in fact
        ref = outs[0].values[:num].astype(np.float64)
        d1 = np.abs(vf[:num] - ref).sum() / np.abs(ref).sum()
        assert d1 <= 1e-6, d1


def unique_formulation(mode, feats, coors):
    coors = coors.copy()
    bad = (coors < 0).any(axis=1)
    coors[bad] = -1
    uniq, inverse, counts = np.unique(coors, axis=0, return_inverse=True, return_counts=True)
    inverse = inverse.reshape(-1)
    flag = int(uniq[0, 0] == -1)
    p2v = inverse.astype(np.int32) - flag
    vc, cnt = uniq[flag:], counts[flag:]
    num = vc.shape[0]
    vf = np.full((num, feats.shape[1]), -np.inf if mode == "max" else 0.0, np.float32)
    for i in range(feats.shape[0]):
        v = p2v[i]
        if v < 0:
            continue
        if mode == "max":
            vf[v] = np.where(feats[i] >= vf[v], feats[i], vf[v])
        else:
            vf[v] = vf[v] + feats[i] / np.float32(cnt[v])
    return vf, vc.astype(np.int32), p2v, cnt.astype(np.int32), num


@pytest.mark.parametrize("mode", ["max", "mean"])
@pytest.mark.parametrize("seed,n,c,span,neg", [(1, 50, 3, 3, 0.1), (2, 2000, 5, 6, 0.05), (3, 2000, 4, 40, 0.0),
                                               (4, 300, 1, 2, 0.5)])
def test_matches_numpy_unique(mode, seed, n, c, span, neg):
    rng = np.random.default_rng(seed)
    feats = rng.uniform(-100, 100, (n, c)).astype(np.float32)
    coors = rng.integers(0, span, (n, 3)).astype(np.int32)
    k = int(n * neg)
    if k:
        coors[rng.choice(n, k, replace=False), rng.integers(0, 3, k)] = -rng.integers(1, 5, k)
    vf, vc, p2v, cnt, num, coors_after = dpv.forward(mode, feats, coors)
    wf, wc, wp, wcnt, wnum = unique_formulation(mode, feats, coors)
    assert num == wnum and np.array_equal(p2v, wp)
    assert np.array_equal(vc[:num], wc) and np.array_equal(cnt[:num], wcnt)
    assert np.array_equal(vf[:num], wf)                  # same operations in the same order
    # rows past voxel_num keep their fill; negative rows were rewritten in place
    assert not vc[num:].any() and not cnt[num:].any()
    assert np.all(vf[num:] == (-np.inf if mode == "max" else 0.0))
    assert ((coors_after < 0).any(axis=1) == (coors_after == -1).all(axis=1)).all()


def test_all_points_invalid_and_empty():
    feats = np.ones((4, 2), np.float32)
    coors = np.array([[-1, 0, 0], [0, -3, 0], [1, 1, -1], [-2, -2, -2]], np.int32)
    vf, vc, p2v, cnt, num, _ = dpv.forward("mean", feats, coors)
    assert num == 0 and p2v.tolist() == [-1, -1, -1, -1] and not vf.any()
    assert dpv.forward("max", np.zeros((0, 3), np.float32), np.zeros((0, 3), np.int32))[4] == 0


def backward_case_inputs(cf, node):
    """The case file stores grad_voxel_feats [34, 5] with the 150 values of its 30 real voxels only:
    the rows past voxel_num are padded with zeros here."""
    msgs = node.all("input")
    bits = np.array(msgs[0].all("value_i"), dtype=np.int64).astype(np.int32).view(np.float32)
    grad = np.zeros((34, 5), np.float32)
    grad.reshape(-1)[:bits.size] = bits
    return [grad] + [cf.CaseTensor(t).values for t in msgs[1:]]


def test_backward_reference_case_file():
    """tests/golden/dynamic_point_to_voxel_backward/case_1.prototxt: 34 points, 5 features, bit-exact."""
    from mluop_hip import casefile as cf
    node, _ = cf.load(os.path.join(os.path.dirname(GOLDEN), "dynamic_point_to_voxel_backward", "case_1.prototxt"))
    ins = backward_case_inputs(cf, node)
    want = cf.CaseTensor(node.all("output")[0]).values
    got = dpv.backward(ins[0], ins[1], ins[2], ins[3], int(ins[5][0]))
    assert np.array_equal(got, want)
    assert np.count_nonzero(want) > 0


@pytest.mark.parametrize("seed,n,c,span", [(1, 200, 4, 3), (2, 3000, 6, 8), (3, 500, 1, 2)])
def test_backward_round_trip_through_forward(seed, n, c, span):
    """Every (voxel, feature) hands its gradient to exactly one of the voxel's points, the first one
    that attains the maximum; summing grad_feats over a voxel's points gives grad_voxel_feats back."""
    rng = np.random.default_rng(seed)
    feats = rng.integers(-3, 4, (n, c)).astype(np.float32)          # many ties
    coors = rng.integers(0, span, (n, 3)).astype(np.int32)
    coors[rng.choice(n, n // 10, replace=False), 0] = -1
    vf, vc, p2v, cnt, num, _ = dpv.forward("max", feats, coors)
    g = rng.standard_normal((n, c)).astype(np.float32)
    grad = dpv.backward(g, feats, vf, p2v, num)
    assert not grad[p2v < 0].any()
    back = np.zeros((num, c), np.float32)
    np.add.at(back, p2v[p2v >= 0], grad[p2v >= 0])
    assert np.array_equal(back, g[:num])
    # first point attaining the maximum, found independently
    for v in range(0, num, max(1, num // 50)):
        pts = np.nonzero(p2v == v)[0]
        for j in range(c):
            first = pts[np.argmax(feats[pts, j] == vf[v, j])]
            assert grad[first, j] == g[v, j]
