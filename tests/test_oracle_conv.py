"""Pins of the CPU oracle's convolution functions, dtype round trips and diff metrics.

The oracle's forward / backward data / backward filter restate the reference executors' loops
over the rulebook.  They are pinned here against a library routine that knows nothing about
rulebooks: features are scattered into a dense grid, torch.nn.functional.conv3d (fp64) and
torch.autograd compute the dense result, and the active cells are read back.  Adjoint identities
tie the three operators to each other."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import sparse_conv_oracle as oracle
from spconv_cases import out_space, random_voxels


def dense_reference(idx, out_idx, n_out, batch, space, ospace, feats, w, stride, pad, dil, dy=None):
    """Dense fp64 conv3d on the scattered features; returns (out rows, dX rows, dW) like the sparse ops."""
    ci, co = w.shape[3], w.shape[4]
    x = torch.zeros((batch, ci) + tuple(space), dtype=torch.float64)
    f = torch.from_numpy(feats.astype(np.float64))
    ii = torch.from_numpy(idx.astype(np.int64))
    x[ii[:, 0], :, ii[:, 1], ii[:, 2], ii[:, 3]] = f
    x.requires_grad_(True)
    wt = torch.from_numpy(w.astype(np.float64)).permute(4, 3, 0, 1, 2).contiguous().requires_grad_(True)
    y = F.conv3d(x, wt, stride=tuple(stride), padding=tuple(pad), dilation=tuple(dil))
    assert list(y.shape[2:]) == list(ospace)
    oo = torch.from_numpy(out_idx[:n_out].astype(np.int64))
    out_rows = y[oo[:, 0], :, oo[:, 1], oo[:, 2], oo[:, 3]]
    res = [out_rows.detach().numpy()]
    if dy is not None:
        g = torch.zeros_like(y)
        g[oo[:, 0], :, oo[:, 1], oo[:, 2], oo[:, 3]] = torch.from_numpy(dy.astype(np.float64))
        y.backward(g)
        res.append(x.grad[ii[:, 0], :, ii[:, 1], ii[:, 2], ii[:, 3]].numpy())
        res.append(wt.grad.permute(2, 3, 4, 1, 0).contiguous().numpy())  # [kd,kh,kw,ci,co]
    return res


CASES = [
    # (batch, space, L, ks, pad, stride, dil, sub_m, ci, co)
    (1, (5, 6, 7), 60, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True, 4, 5),
    (2, (6, 6, 6), 120, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True, 3, 7),
    (2, (7, 8, 9), 150, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1), False, 5, 4),
    (1, (8, 8, 8), 100, (3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2), False, 2, 3),
    (1, (6, 7, 8), 90, (2, 2, 2), (0, 0, 0), (2, 2, 2), (1, 1, 1), False, 6, 2),
    (1, (5, 9, 6), 80, (1, 3, 2), (0, 1, 0), (1, 2, 1), (1, 1, 1), False, 3, 3),
]


@pytest.mark.parametrize("case", CASES)
def test_oracle_ops_match_dense_conv3d_and_autograd(case):
    batch, space, L, ks, pad, stride, dil, sub_m, ci, co = case
    rng = np.random.default_rng(1)
    idx = random_voxels(rng, batch, space, L)
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, batch, list(pad), list(stride), list(dil), list(ks),
                                                         ospace, sub_m, exact_count=True)
    K = int(np.prod(ks))
    feats = rng.standard_normal((L, ci)).astype(np.float32)
    w = rng.standard_normal(tuple(ks) + (ci, co)).astype(np.float32)
    dy = rng.standard_normal((n_out, co)).astype(np.float32)
    wk = w.reshape(K, ci, co)
    ref_out, ref_dx, ref_dw = dense_reference(idx, out_idx, n_out, batch, space, ospace, feats, w, stride, pad,
                                              dil, dy)
    out = oracle.forward(feats, wk, pairs, num, n_out)
    dx = oracle.backward_data(dy, wk, pairs, num)
    dw = oracle.backward_filter(feats, dy, pairs, num)
    if sub_m:
        # a submanifold conv only evaluates the dense conv at active cells: same numbers there
        pass
    np.testing.assert_allclose(out, ref_out, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(dx, ref_dx, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(dw.reshape(w.shape), ref_dw, rtol=2e-5, atol=2e-4)
    dw_fast = oracle.backward_filter(feats, dy, pairs, num, fast=True)
    assert np.array_equal(dw, dw_fast)  # same summation order per element
    # adjoint identities in fp64: <dY, fwd(X)> = <X, bwd_data(dY)> = <W, bwd_filter(X, dY)>
    a = float(np.sum(dy.astype(np.float64) * out))
    b = float(np.sum(feats.astype(np.float64) * dx))
    c = float(np.sum(wk.astype(np.float64) * dw))
    scale = abs(a) + 1.0
    assert abs(a - b) / scale < 1e-4 and abs(a - c) / scale < 1e-4


INVERSE_CASES = [
    # (batch, space, L, ks, pad, stride, dil, ci of the inverse layer, co of the inverse layer)
    (2, (7, 8, 9), 150, (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1), 5, 4),
    (1, (8, 8, 8), 100, (3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2), 2, 3),
    (1, (6, 7, 8), 90, (2, 2, 2), (0, 0, 0), (2, 2, 2), (1, 1, 1), 6, 2),
    (1, (5, 9, 6), 80, (1, 3, 2), (0, 1, 0), (1, 2, 1), (1, 1, 1), 3, 3),
]


@pytest.mark.parametrize("case", INVERSE_CASES)
def test_inverse_ops_match_dense_conv_transpose3d_and_autograd(case):
    """The inverse convolution runs its partner's rulebook backwards: dense conv_transpose3d of the
    partner's output grid, read back at the partner's input cells, is the same numbers, and its
    autograd gives the two gradients."""
    batch, space, L, ks, pad, stride, dil, ci, co = case
    rng = np.random.default_rng(7)
    idx = random_voxels(rng, batch, space, L)
    ospace = out_space(space, ks, pad, stride, dil)
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, batch, list(pad), list(stride), list(dil), list(ks),
                                                         ospace, False, exact_count=True)
    K = int(np.prod(ks))
    feats = rng.standard_normal((n_out, ci)).astype(np.float32)   # live on the partner's output cells
    w = rng.standard_normal(tuple(ks) + (ci, co)).astype(np.float32)
    dy = rng.standard_normal((L, co)).astype(np.float32)          # gradient at the partner's input cells
    wk = w.reshape(K, ci, co)

    x = torch.zeros((batch, ci) + tuple(ospace), dtype=torch.float64)
    oo = torch.from_numpy(out_idx[:n_out].astype(np.int64))
    ii = torch.from_numpy(idx.astype(np.int64))
    x[oo[:, 0], :, oo[:, 1], oo[:, 2], oo[:, 3]] = torch.from_numpy(feats.astype(np.float64))
    x.requires_grad_(True)
    wt = torch.from_numpy(w.astype(np.float64)).permute(3, 4, 0, 1, 2).contiguous().requires_grad_(True)
    opad = [sp - ((o - 1) * s - 2 * p + d * (k - 1) + 1) for sp, o, s, p, d, k in zip(space, ospace, stride, pad, dil, ks)]
    y = F.conv_transpose3d(x, wt, stride=tuple(stride), padding=tuple(pad), output_padding=tuple(opad),
                           dilation=tuple(dil))
    assert list(y.shape[2:]) == list(space)
    ref_out = y[ii[:, 0], :, ii[:, 1], ii[:, 2], ii[:, 3]].detach().numpy()
    g = torch.zeros_like(y)
    g[ii[:, 0], :, ii[:, 1], ii[:, 2], ii[:, 3]] = torch.from_numpy(dy.astype(np.float64))
    y.backward(g)
    ref_dx = x.grad[oo[:, 0], :, oo[:, 1], oo[:, 2], oo[:, 3]].numpy()
    ref_dw = wt.grad.permute(2, 3, 4, 0, 1).contiguous().numpy()

    out = oracle.forward(feats, wk, pairs, num, L, inverse=True)
    dx = oracle.backward_data(dy, wk, pairs, num, inverse=True, rows=n_out)
    dw = oracle.backward_filter(feats, dy, pairs, num, inverse=True)
    np.testing.assert_allclose(out, ref_out, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(dx, ref_dx, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(dw.reshape(w.shape), ref_dw, rtol=2e-5, atol=2e-4)
    # the inverse forward is the partner's backward data with the filter's channel roles exchanged
    same = oracle.backward_data(feats, np.ascontiguousarray(np.transpose(wk, (0, 2, 1))), pairs, num)
    np.testing.assert_allclose(out, same, rtol=2e-5, atol=2e-5)  # fp32 sums in different orders


def test_forward_skips_negative_pairs_and_respects_indice_num():
    rng = np.random.default_rng(2)
    L, K, ci, co = 6, 2, 3, 2
    feats = rng.standard_normal((L, ci)).astype(np.float32)
    w = rng.standard_normal((K, ci, co)).astype(np.float32)
    pairs = np.full((K, 2, L), -1, dtype=np.int32)
    pairs[0, 0, :3] = [0, 2, 5]
    pairs[0, 1, :3] = [1, 1, -1]       # two inputs into output 1, one negative output (skipped)
    pairs[1, 0, :2] = [4, 3]
    pairs[1, 1, :2] = [0, 2]           # second one lies beyond indice_num[1] = 1
    out = oracle.forward(feats, w, pairs, [3, 1], 3)
    expect = np.zeros((3, co), dtype=np.float64)
    expect[1] = feats[0] @ w[0] + feats[2] @ w[0]
    expect[0] = feats[4] @ w[1]
    np.testing.assert_allclose(out, expect, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("layout,perm", [(3, (4, 0, 1, 2, 3)), (5, (4, 3, 0, 1, 2)), (4, (0, 1, 2, 3, 4))])
def test_filter_layout_transposes(layout, perm):
    rng = np.random.default_rng(3)
    w = rng.standard_normal((2, 3, 2, 5, 4)).astype(np.float32)  # [kd,kh,kw,ci,co]
    src = np.ascontiguousarray(np.transpose(w, perm))
    got = oracle.filters_to_kcico(src, layout, 12, 5, 4)
    assert np.array_equal(got, w.reshape(12, 5, 4))


def test_half_round_trip_matches_ieee_round_to_nearest_even():
    rng = np.random.default_rng(4)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 3,
        rng.standard_normal(2000).astype(np.float32) * 1e-6,   # subnormal half range
        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 2.0 ** -24, 1.5 * 2.0 ** -25, 1.0 + 2.0 ** -11,
                  1.0 + 3 * 2.0 ** -11, np.inf, -np.inf], dtype=np.float32)])
    # The reference's converter (tools.cpp:460-505) is IEEE round-to-nearest-even except that it
    # rounds every non-zero magnitude of at most 2^-25 up to the smallest subnormal instead of to zero.
    tiny = (np.abs(vals) <= 2.0 ** -25) & (vals != 0)
    assert tiny.any()
    assert np.all((oracle.float_to_half_bits(vals[tiny]) & 0x7FFF) == 1)
    vals = vals[~tiny]
    bits = oracle.float_to_half_bits(vals)
    expect = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(bits, expect)
    back = oracle.round_through_half(vals)
    assert np.array_equal(back, vals.astype(np.float16).astype(np.float32))
    # beyond the half range the reference's converter saturates to the largest finite half
    assert oracle.float_to_half_bits(np.array([70000.0], dtype=np.float32))[0] == 0x7BFF
    assert np.isnan(oracle.round_through_half(np.array([np.nan], dtype=np.float32))[0])


def test_bf16_round_trip_is_round_to_nearest_even():
    rng = np.random.default_rng(5)
    vals = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10,
                           np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -2.5, 3.0e38], dtype=np.float32)])
    back = oracle.round_through_bf16(vals)
    expect = torch.from_numpy(vals).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(back, expect)
    assert oracle.float_to_bf16_bits(np.array([np.nan], dtype=np.float32))[0] == 0x7FC0


def test_diff_metrics_closed_forms():
    rng = np.random.default_rng(6)
    b = rng.standard_normal(1000).astype(np.float32) + 3.0
    assert oracle.diff1(b, b) == 0.0 and oracle.diff2(b, b) == 0.0 and oracle.diff3(b, b) == 0.0
    eps = 1e-3
    a = (b.astype(np.float64) * (1 + eps)).astype(np.float32)
    assert abs(oracle.diff1(a, b) - eps) < 1e-5
    assert abs(oracle.diff2(a, b) - eps) < 1e-5
    assert abs(oracle.diff3(a, b) - eps) < 1e-5
    # explicit small case: a-b = [1, -2], b = [2, 4]
    a2, b2 = np.array([3.0, 2.0], dtype=np.float32), np.array([2.0, 4.0], dtype=np.float32)
    assert abs(oracle.diff1(a2, b2) - 3.0 / 6.0) < 1e-9
    assert abs(oracle.diff2(a2, b2) - np.sqrt(5.0 / 20.0)) < 1e-9
    assert abs(oracle.diff3(a2, b2) - 0.5) < 1e-9
    # below the absolute-error threshold diff3 switches to the absolute error
    assert abs(oracle.diff3(np.array([1e-7], dtype=np.float32), np.array([0.0], dtype=np.float32)) - 1e-7) < 1e-12
