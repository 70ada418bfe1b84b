"""The PyTorch caller layer (mluop_hip.nn) against dense torch.conv3d + autograd in float64 on the
CPU: a submanifold layer, a second one sharing its rulebook through `indice_key`, and a strided
regular layer, forward values and the gradients of features and weights."""
import numpy as np
import pytest

from spconv_cases import random_voxels

pytestmark = pytest.mark.gpu


def dense_reference(idx, feats, weights, space, batch):
    """Runs the same three layers densely in float64; returns (out rows at out cells, grads)."""
    import torch
    import torch.nn.functional as F
    D, H, W = space
    x = torch.tensor(feats, dtype=torch.float64, requires_grad=True)
    ws = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in weights]
    ii = torch.from_numpy(idx.astype(np.int64))
    dense = torch.zeros((batch, D, H, W, feats.shape[1]), dtype=torch.float64)
    dense = dense.index_put((ii[:, 0], ii[:, 1], ii[:, 2], ii[:, 3]), x)
    mask = torch.zeros((batch, 1, D, H, W), dtype=torch.float64)
    mask[ii[:, 0], 0, ii[:, 1], ii[:, 2], ii[:, 3]] = 1.0
    t = dense.permute(0, 4, 1, 2, 3)

    def conv(t, w, stride, pad):
        return F.conv3d(t, w.permute(4, 3, 0, 1, 2), stride=stride, padding=pad)

    t = conv(t, ws[0], 1, 1) * mask          # submanifold: outputs only on active inputs
    t = conv(t, ws[1], 1, 1) * mask
    t = conv(t, ws[2], 2, 1)                 # regular: every reached cell is active
    reach = conv(mask, torch.ones((3, 3, 3, 1, 1), dtype=torch.float64), 2, 1) > 0
    return x, ws, t, reach[:, 0]


def test_layers_match_dense_autograd(gpu_handle):
    import torch
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(21)
    batch, space, L, ci, cm, co = 2, (8, 10, 12), 300, 16, 32, 16
    idx = random_voxels(rng, batch, space, L)
    feats = rng.standard_normal((L, ci)).astype(np.float32)
    torch.manual_seed(3)
    l1 = spnn.SubMConv3d(ci, cm, 3, indice_key="subm1").cuda()
    l2 = spnn.SubMConv3d(cm, cm, 3, indice_key="subm1").cuda()
    l3 = spnn.SparseConv3d(cm, co, 3, stride=2, padding=1).cuda()
    x = torch.from_numpy(feats).cuda().requires_grad_(True)
    st = spnn.SparseTensor(x, torch.from_numpy(idx).cuda(), space, batch)
    y1 = l1(st)
    assert len(st.rulebooks) == 1
    y2 = l2(y1)
    assert len(st.rulebooks) == 1 and y2.rulebooks is st.rulebooks   # second layer reused the rulebook
    y3 = l3(y2)
    out_idx = y3.indices.cpu().numpy().astype(np.int64)
    g = rng.standard_normal(tuple(y3.features.shape)).astype(np.float32)
    (y3.features * torch.from_numpy(g).cuda()).sum().backward()
    torch.cuda.synchronize()

    weights = [l.weight.detach().cpu().numpy() for l in (l1, l2, l3)]
    rx, rws, rt, reach = dense_reference(idx, feats, weights, space, batch)
    # same active output cells, in ascending linear order
    ref_cells = np.argwhere(reach.numpy())
    assert np.array_equal(out_idx, ref_cells)
    oi = torch.from_numpy(out_idx)
    ref_rows = rt.permute(0, 2, 3, 4, 1)[oi[:, 0], oi[:, 1], oi[:, 2], oi[:, 3]]
    (ref_rows * torch.from_numpy(g).double()).sum().backward()

    def close(a, b, what):
        a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
        d1 = np.abs(a - b).sum() / (np.abs(b).sum() + 1e-9)
        d2 = np.sqrt(((a - b) ** 2).sum() / ((b ** 2).sum() + 1e-9))
        assert d1 <= 1e-5 and d2 <= 1e-5, "%s diff1=%.3e diff2=%.3e" % (what, d1, d2)

    close(y3.features.detach().cpu().numpy(), ref_rows.detach().numpy(), "forward")
    close(x.grad.cpu().numpy(), rx.grad.numpy(), "grad features")
    for layer, rw, name in zip((l1, l2, l3), rws, ("w1", "w2", "w3")):
        close(layer.weight.grad.cpu().numpy(), rw.grad.numpy(), "grad " + name)


def test_sequential_plans_all_rulebooks_first_and_matches_the_layers_one_by_one(gpu_handle, monkeypatch):
    """SparseSequential builds the rulebooks of all its convolutions before the first layer runs (keyed
    layers share one, keyless strided layers get theirs planned, the inverse layer finds its partner's)
    and gives the bits of the same layers applied one by one."""
    import torch
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(23)
    batch, space, L = 2, (8, 10, 12), 400
    idx = random_voxels(rng, batch, space, L)
    feats = torch.from_numpy(rng.standard_normal((L, 16)).astype(np.float32)).cuda()
    torch.manual_seed(5)
    layers = [spnn.SubMConv3d(16, 16, 3, indice_key="a"), torch.nn.ReLU(),
              spnn.SubMConv3d(16, 32, 3, indice_key="a"), torch.nn.ReLU(),
              spnn.SparseConv3d(32, 32, 3, stride=2, padding=1, indice_key="down"),
              spnn.SparseSequential(spnn.SubMConv3d(32, 32, 3), torch.nn.ReLU(),
                                    spnn.SparseConv3d(32, 64, 3, stride=2, padding=1)),
              spnn.SubMConv3d(64, 64, 3)]
    net = spnn.SparseSequential(*layers).cuda()
    indices = torch.from_numpy(idx).cuda()

    built, order = [], []
    real = spnn.get_indice_pairs
    monkeypatch.setattr(spnn, "get_indice_pairs", lambda *a, **k: (built.append(1), real(*a, **k))[1])
    real_apply = spnn._IndiceConv.apply
    x1 = feats.clone().requires_grad_(True)
    hooks = [m.register_forward_pre_hook(lambda mod, inp: order.append(len(built)))
             for m in net.modules() if isinstance(m, spnn._ConvBase)]
    y = net(spnn.SparseTensor(x1, indices, space, batch))
    for h in hooks:
        h.remove()
    # six convolutions, five rulebooks (two layers share "a"), all of them there before the first layer ran
    assert len(built) == 5 and order == [5] * 6
    y.features.square().sum().backward()

    x2 = feats.clone().requires_grad_(True)
    grads1 = [p.grad.clone() for p in net.parameters()]
    for p in net.parameters():
        p.grad = None
    t = spnn.SparseTensor(x2, indices, space, batch)
    flat = layers[:5] + list(layers[5]) + layers[6:]
    for m in flat:
        t = m(t) if isinstance(m, spnn._ConvBase) else t.replace_features(m(t.features))
    t.features.square().sum().backward()
    torch.cuda.synchronize()
    assert torch.equal(y.indices, t.indices) and torch.equal(y.features, t.features)
    assert torch.equal(x1.grad, x2.grad)
    for g1, p in zip(grads1, net.parameters()):
        assert torch.equal(g1, p.grad)


def test_half_precision_layer_runs_mfma_path(gpu_handle):
    """fp16 features through SubMConv3d(64, 64): graded at the fp16 threshold against float64."""
    import torch
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(22)
    batch, space, L = 1, (10, 12, 12), 700
    idx = random_voxels(rng, batch, space, L)
    feats = torch.from_numpy(rng.standard_normal((L, 64)).astype(np.float32)).half()
    layer = spnn.SubMConv3d(64, 64, 3).cuda()
    with torch.no_grad():
        layer.weight.copy_(layer.weight.half().float())
    st = spnn.SparseTensor(feats.cuda(), torch.from_numpy(idx).cuda(), space, batch)
    y = layer(st).features.detach().float().cpu().numpy()
    rb = next(iter([layer._rulebook(st)]))
    pairs = rb.pairs.cpu().numpy()
    w = layer.weight.detach().cpu().double().numpy().reshape(27, 64, 64)
    ref = np.zeros((L, 64))
    f64 = feats.double().numpy()
    for k in range(27):
        n = rb.indice_num[k]
        np.add.at(ref, pairs[k, 1, :n], f64[pairs[k, 0, :n]] @ w[k])
    d1 = np.abs(y - ref).sum() / (np.abs(ref).sum() + 1e-9)
    assert d1 <= 3e-3, d1


def test_points_to_voxels_to_submanifold_layer(gpu_handle):
    """points -> Voxelization -> mean features -> SparseTensor -> SubMConv3d: voxel coordinates are
    distinct cells of the grid, and the layer's output equals the dense convolution of the voxel
    grid at those cells."""
    import torch
    import torch.nn.functional as F
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(23)
    pts = np.empty((4000, 4), np.float32)
    pts[:, 0] = rng.uniform(0, 6.4, 4000)
    pts[:, 1] = rng.uniform(-3.2, 3.2, 4000)
    pts[:, 2] = rng.uniform(-1, 1, 4000)
    pts[:, 3] = rng.uniform(0, 1, 4000)
    vox = spnn.Voxelization([0.4, 0.4, 0.5], [0, -3.2, -1, 6.4, 3.2, 1], max_num_points=8, max_voxels=5000).cuda()
    space = vox.grid_shape()
    assert space == (4, 16, 16)
    voxels, coors, npv = vox(torch.from_numpy(pts).cuda())
    V = voxels.shape[0]
    c = coors.cpu().numpy()
    assert V == len({tuple(r) for r in c.tolist()}) and (c >= 0).all() and (c < np.array(space)).all()
    assert int(npv.sum().item()) <= 4000 and int(npv.min().item()) >= 1
    feats = spnn.mean_voxel_features(voxels, npv)
    torch.manual_seed(5)
    layer = spnn.SubMConv3d(4, 16, 3).cuda()
    dense = torch.zeros((1, 4) + space, dtype=torch.float64)
    ci = torch.from_numpy(c.astype(np.int64))
    dense[0, :, ci[:, 0], ci[:, 1], ci[:, 2]] = feats.cpu().double().t()
    w = layer.weight.detach().cpu().double().permute(4, 3, 0, 1, 2)
    full = F.conv3d(dense, w, padding=1)[0]
    # The voxelizer numbers voxels by first point; the sparse tensor puts them in cell order, so
    # the layer's rulebook needs no hash table and its forward no row map.
    handle = spnn._handle()
    for order_by_cell in (True, False):
        st = spnn.sparse_tensor_from_voxels(feats, coors, space, order_by_cell=order_by_cell)
        rows = st.indices[:, 1:].cpu().numpy().astype(np.int64)
        assert sorted(map(tuple, rows.tolist())) == sorted(map(tuple, c.tolist()))
        if order_by_cell:
            lin = (rows[:, 0] * space[1] + rows[:, 1]) * space[2] + rows[:, 2]
            assert (np.diff(lin) > 0).all()
        handle.set_kernel_timing(True)
        y = layer(st).features.detach().cpu().double()
        names = [n for n, _ in handle.kernel_timings()]
        handle.set_kernel_timing(False)
        assert any(n.startswith("gatherConv") for n in names), names
        took_the_map = [n for n in names if n in ("scatterRowMap", "fillMapPackFilter", "fillInt32")]
        assert (not took_the_map) == order_by_cell, names
        ref = full[:, rows[:, 0], rows[:, 1], rows[:, 2]].t()
        d1 = (y - ref).abs().sum() / ref.abs().sum()
        assert d1 <= 1e-5, float(d1)


def test_small_channel_counts_are_padded_for_the_matrix_cores(gpu_handle):
    """5 -> 12 channels (padded to 16 -> 16 inside the layer): values and gradients against the
    rulebook-driven float64 formula."""
    import torch
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(24)
    batch, space, L = 1, (9, 10, 11), 400
    idx = random_voxels(rng, batch, space, L)
    feats = torch.from_numpy(rng.standard_normal((L, 5)).astype(np.float32)).cuda().requires_grad_(True)
    torch.manual_seed(7)
    layer = spnn.SubMConv3d(5, 12, 3).cuda()
    st = spnn.SparseTensor(feats, torch.from_numpy(idx).cuda(), space, batch)
    y = layer(st).features
    assert tuple(y.shape) == (L, 12)
    g = torch.from_numpy(rng.standard_normal((L, 12)).astype(np.float32)).cuda()
    (y * g).sum().backward()
    rb = layer._rulebook(st)
    pairs = rb.pairs.cpu().numpy()
    w = layer.weight.detach().cpu().double().numpy().reshape(27, 5, 12)
    x64, g64 = feats.detach().cpu().double().numpy(), g.cpu().double().numpy()
    ref, dx, dw = np.zeros((L, 12)), np.zeros((L, 5)), np.zeros((27, 5, 12))
    for k in range(27):
        n = rb.indice_num[k]
        i, o = pairs[k, 0, :n], pairs[k, 1, :n]
        np.add.at(ref, o, x64[i] @ w[k])
        np.add.at(dx, i, g64[o] @ w[k].T)
        dw[k] = x64[i].T @ g64[o]
    for got, want, what in ((y.detach().cpu().numpy(), ref, "forward"), (feats.grad.cpu().numpy(), dx, "grad x"),
                            (layer.weight.grad.cpu().numpy().reshape(27, 5, 12), dw, "grad w")):
        d1 = np.abs(got - want).sum() / np.abs(want).sum()
        assert d1 <= 1e-5, (what, d1)


def test_inverse_layer_returns_to_the_partner_layers_cells(gpu_handle):
    """SparseConv3d (stride 2) followed by the SparseInverseConv3d that shares its rulebook, against
    dense conv3d -> conv_transpose3d in float64 read at the first layer's input cells, with the
    gradients of features and both filters."""
    import torch
    import torch.nn.functional as F
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(23)
    batch, space, L, ci, cm, co = 2, (8, 10, 12), 300, 16, 32, 16
    idx = random_voxels(rng, batch, space, L)
    feats = rng.standard_normal((L, ci)).astype(np.float32)
    torch.manual_seed(5)
    down = spnn.SparseConv3d(ci, cm, 3, stride=2, padding=1, indice_key="down").cuda()
    up = spnn.SparseInverseConv3d(cm, co, 3, indice_key="down").cuda()
    x = torch.from_numpy(feats).cuda().requires_grad_(True)
    st = spnn.SparseTensor(x, torch.from_numpy(idx).cuda(), space, batch)
    mid = down(st)
    y = up(mid)
    assert y.spatial_shape == tuple(space) and torch.equal(y.indices, st.indices)
    assert tuple(y.features.shape) == (L, co)
    g = rng.standard_normal((L, co)).astype(np.float32)
    (y.features * torch.from_numpy(g).cuda()).sum().backward()
    torch.cuda.synchronize()

    D, H, W = space
    rx = torch.tensor(feats, dtype=torch.float64, requires_grad=True)
    w1 = torch.tensor(down.weight.detach().cpu().numpy(), dtype=torch.float64, requires_grad=True)
    w2 = torch.tensor(up.weight.detach().cpu().numpy(), dtype=torch.float64, requires_grad=True)
    ii = torch.from_numpy(idx.astype(np.int64))
    dense = torch.zeros((batch, D, H, W, ci), dtype=torch.float64).index_put(
        (ii[:, 0], ii[:, 1], ii[:, 2], ii[:, 3]), rx).permute(0, 4, 1, 2, 3)
    t = F.conv3d(dense, w1.permute(4, 3, 0, 1, 2), stride=2, padding=1)
    opad = [s - ((o - 1) * 2 - 2 + 2 + 1) for s, o in zip(space, t.shape[2:])]
    t = F.conv_transpose3d(t, w2.permute(3, 4, 0, 1, 2), stride=2, padding=1, output_padding=opad)
    assert tuple(t.shape[2:]) == tuple(space)
    rows = t[ii[:, 0], :, ii[:, 1], ii[:, 2], ii[:, 3]]
    (rows * torch.from_numpy(g.astype(np.float64))).sum().backward()
    np.testing.assert_allclose(y.features.detach().cpu().numpy(), rows.detach().numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(x.grad.cpu().numpy(), rx.grad.numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(down.weight.grad.cpu().numpy(), w1.grad.numpy(), rtol=1e-4, atol=2e-4)
    np.testing.assert_allclose(up.weight.grad.cpu().numpy(), w2.grad.numpy(), rtol=1e-4, atol=2e-4)


def test_repeated_coordinates_through_the_layers(gpu_handle):
    """A tensor whose coordinates repeat (not marked distinct): the submanifold layer adds every
    pair, as the dense reference does when the repeated rows' features are summed per cell... which
    is not what a last-writer-wins rulebook means, so the reference here is the CPU oracle; and a
    tensor marked distinct skips the operators' collision check."""
    import torch
    import mluop_hip
    import sparse_conv_oracle as oracle
    from mluop_hip import nn as spnn
    rng = np.random.default_rng(25)
    batch, space, L, ci, co = 1, (8, 9, 10), 300, 16, 32
    idx = random_voxels(rng, batch, space, L, duplicates=60)
    feats = rng.standard_normal((idx.shape[0], ci)).astype(np.float32)
    layer = spnn.SubMConv3d(ci, co, 3).cuda()
    st = spnn.SparseTensor(torch.from_numpy(feats).cuda(), torch.from_numpy(idx).cuda(), space, batch)
    assert not st.distinct
    out = layer(st).features
    torch.cuda.synchronize()
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, batch, [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3],
                                                         list(space), True, exact_count=True)
    w = layer.weight.detach().cpu().numpy().reshape(27, ci, co)
    ref = oracle.forward(feats, w, pairs, num, n_out)
    np.testing.assert_allclose(out.detach().cpu().numpy(), ref, rtol=1e-4, atol=1e-5)

    h = spnn._handle()
    clean = random_voxels(rng, batch, space, L)
    x = torch.from_numpy(rng.standard_normal((L, ci)).astype(np.float32)).cuda()
    for distinct, expect_check in ((False, True), (True, False)):
        st = spnn.SparseTensor(x, torch.from_numpy(clean).cuda(), space, batch, distinct=distinct)
        h.set_kernel_timing(True)
        y = layer(st)
        names = [n for n, _ in h.kernel_timings()]
        h.set_kernel_timing(False)
        assert ("repairLostPairs" in names) == expect_check
        assert y.distinct == distinct
    down = spnn.SparseConv3d(ci, co, 3, stride=2, padding=1).cuda()
    assert down(spnn.SparseTensor(x, torch.from_numpy(clean).cuda(), space, batch)).distinct
