"""Seeded random sweeps through the C ABI against the CPU oracles: geometries, channel counts,
dtypes, filter layouts, repeated coordinates, inverse convolutions, and the upstream operators'
parameters are drawn at random (small sizes, a few hundred cases, a few seconds).  A sweep of this
kind found what the hand-written cases had missed: pairs of one offset sharing a result row.
Rulebooks and the upstream operators are compared bit for bit, convolutions at the reference's
thresholds."""
import numpy as np
import pytest

import dynamic_point_to_voxel_oracle as dpv
import sparse_conv_oracle as oracle
import voxelization_oracle as vox
from spconv_cases import THRESH, from_torch, out_space, random_voxels, round_to, to_torch

pytestmark = pytest.mark.gpu

CHANNELS = [16, 32, 64, 128, 8, 24, 48, 5, 96]


def draw_geometry(rng):
    batch = int(rng.integers(1, 4))
    space = tuple(int(v) for v in rng.integers(3, 14, size=3))
    ks = tuple(int(v) for v in rng.integers(1, 5, size=3))
    sub_m = bool(rng.integers(0, 2))
    if sub_m:
        ks = tuple(k | 1 for k in ks)
        stride, dil, pad = [1, 1, 1], [1, 1, 1], [k // 2 for k in ks]
    else:
        stride = [int(v) for v in rng.integers(1, 4, size=3)]
        # the reference refuses stride and dilation above 1 on the same axis
        dil = [int(v) if st == 1 else 1 for v, st in zip(rng.integers(1, 3, size=3), stride)]
        pad = [int(v) for v in rng.integers(0, 3, size=3)]
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    return batch, space, ks, sub_m, stride, dil, pad, ospace


@pytest.mark.parametrize("block", range(6))
def test_rulebook_and_convolutions(gpu_handle, block):
    import torch
    import mluop_hip as m
    gpu_handle.set_extended_modes(True)
    try:
        done = 0
        for case in range(40):
            seed = 7000 + block * 100 + case
            rng = np.random.default_rng(seed)
            batch, space, ks, sub_m, stride, dil, pad, ospace = draw_geometry(rng)
            if min(ospace) < 1:
                continue
            cells = batch * space[0] * space[1] * space[2]
            L = int(rng.integers(1, min(cells, 3000) + 1))
            dup = int(rng.integers(0, 3)) * int(rng.integers(0, 20))
            idx = random_voxels(rng, batch, space, L, shuffle=bool(rng.integers(0, 2)), duplicates=dup)
            ci, co = int(rng.choice(CHANNELS)), int(rng.choice(CHANNELS))
            dtype_name = str(rng.choice(["float32", "float16", "bfloat16"]))
            inverse = (not sub_m) and bool(rng.integers(0, 3) == 0)
            what = "seed %d: %s" % (seed, dict(batch=batch, space=space, ks=ks, sub_m=sub_m, stride=stride, dil=dil,
                                                pad=pad, rows=idx.shape[0], ci=ci, co=co, dtype=dtype_name,
                                                inverse=inverse))
            print(what, flush=True)
            K = int(np.prod(ks))
            pairs_o, out_o, num_o, n_out_o = oracle.get_indice_pairs(idx, batch, pad, stride, dil, list(ks), ospace,
                                                                     sub_m, exact_count=True)
            try:
                pairs, out_idx, num, n_out = m.get_indice_pairs(gpu_handle, torch.from_numpy(idx).cuda(), batch, space,
                                                                ks, ospace, pad, stride, dil, sub_m)
            except m.MluOpError:
                continue   # a geometry the reference's checks refuse as well
            torch.cuda.synchronize()
            assert n_out == n_out_o and np.array_equal(pairs.cpu().numpy(), pairs_o), what
            assert np.array_equal(num.cpu().numpy(), num_o), what
            assert np.array_equal(out_idx.cpu().numpy()[:n_out], out_o[:n_out]), what
            if n_out == 0:
                continue
            rows = idx.shape[0]
            num_host = [int(v) for v in num_o]
            w = round_to((rng.standard_normal(ks + (ci, co)) / np.sqrt(K * ci)).astype(np.float32), dtype_name)
            wk = w.reshape(K, ci, co)
            thr = THRESH[dtype_name]

            def grade(dev, ref, name):
                ref = round_to(ref, dtype_name)
                assert np.isfinite(dev).all(), what + " " + name
                assert oracle.diff1(dev, ref) <= thr and oracle.diff2(dev, ref) <= thr, what + " " + name

            x_rows, y_rows = (n_out, rows) if inverse else (rows, n_out)
            x = round_to(rng.standard_normal((x_rows, ci)).astype(np.float32), dtype_name)
            dy = round_to((rng.standard_normal((y_rows, co)) * 0.1).astype(np.float32), dtype_name)
            xt, dyt = to_torch(x, dtype_name, "cuda"), to_torch(dy, dtype_name, "cuda")
            try:
                if inverse:
                    wt = to_torch(w, dtype_name, "cuda")
                    out = m.indice_conv_forward(gpu_handle, xt, wt, m.LAYOUT_ARRAY, pairs, num_host, rows, False,
                                                inverse=1)
                    dx = m.indice_conv_backward_data(gpu_handle, dyt, wt, m.LAYOUT_ARRAY, pairs, num_host, False, ci,
                                                     inverse=1, rows=n_out)
                    dw = m.indice_conv_backward_filter(gpu_handle, xt, dyt, pairs, num_host, ks, False, inverse=1)
                    dw_k = from_torch(dw).reshape(K, ci, co)
                else:
                    lay = int(rng.choice([m.LAYOUT_ARRAY, m.LAYOUT_NDHWC, m.LAYOUT_NCDHW]))
                    perm = {m.LAYOUT_ARRAY: (0, 1, 2, 3, 4), m.LAYOUT_NDHWC: (4, 0, 1, 2, 3),
                            m.LAYOUT_NCDHW: (4, 3, 0, 1, 2)}[lay]
                    wt = to_torch(np.ascontiguousarray(np.transpose(w, perm)), dtype_name, "cuda")
                    out = m.indice_conv_forward(gpu_handle, xt, wt, lay, pairs, num_host, n_out, sub_m)
                    dx = m.indice_conv_backward_data(gpu_handle, dyt, wt, lay, pairs, num_host, sub_m, ci)
                    dw = m.indice_conv_backward_filter(gpu_handle, xt, dyt, pairs, num_host, ks, sub_m, grad_layout=lay)
                    dw_k = np.ascontiguousarray(np.transpose(from_torch(dw), tuple(np.argsort(perm)))).reshape(K, ci, co)
            except m.MluOpError:
                continue   # e.g. more pairs in an offset than output_grad has rows: refused as in the reference
            torch.cuda.synchronize()
            # with the rulebook's row maps kept across calls the operators must give the same bits
            # (a map that lost pairs, as repeated coordinates make it, is refused and not tried)
            fwd_map = m.RowMap(gpu_handle, pairs, num_host, y_rows, x_rows, 0 if inverse else 1)
            bwd_map = m.RowMap(gpu_handle, pairs, num_host, x_rows, y_rows, 1 if inverse else 0)
            # (repeated coordinates collide in the map whose rows are the outputs, not in the other)
            assert dup > 0 or (fwd_map.usable and bwd_map.usable), what
            if fwd_map.usable:
                if inverse:
                    out2 = m.indice_conv_forward(gpu_handle, xt, wt, m.LAYOUT_ARRAY, pairs, num_host, rows, False,
                                                 inverse=1, row_map=fwd_map)
                else:
                    out2 = m.indice_conv_forward(gpu_handle, xt, wt, lay, pairs, num_host, n_out, sub_m,
                                                 row_map=fwd_map)
                torch.cuda.synchronize()
                assert torch.equal(out2, out), what + " forward with its row map"
            if bwd_map.usable:
                if inverse:
                    dx2 = m.indice_conv_backward_data(gpu_handle, dyt, wt, m.LAYOUT_ARRAY, pairs, num_host, False, ci,
                                                      inverse=1, rows=n_out, row_map=bwd_map)
                else:
                    dx2 = m.indice_conv_backward_data(gpu_handle, dyt, wt, lay, pairs, num_host, sub_m, ci,
                                                      row_map=bwd_map)
                torch.cuda.synchronize()
                assert torch.equal(dx2, dx), what + " backward data with its row map"
            fwd_map.close()
            bwd_map.close()
            grade(from_torch(out), oracle.forward(x, wk, pairs_o, num_o, y_rows, inverse=inverse), "forward")
            grade(from_torch(dx), oracle.backward_data(dy, wk, pairs_o, num_o, inverse=inverse, rows=x_rows)
                  if inverse else oracle.backward_data(dy, wk, pairs_o, num_o), "backward data")
            grade(dw_k, oracle.backward_filter(x, dy, pairs_o, num_o, fast=True, inverse=inverse), "backward filter")
            done += 1
        assert done >= 20   # the sweep compared something
    finally:
        gpu_handle.set_extended_modes(False)


@pytest.mark.parametrize("block", range(3))
def test_voxelization(gpu_handle, block):
    import torch
    import mluop_hip as m
    done = 0
    for case in range(60):
        seed = 8000 + block * 100 + case
        rng = np.random.default_rng(seed)
        npts, f = int(rng.integers(0, 3000)), int(rng.integers(3, 9))
        max_points, max_voxels = int(rng.integers(1, 12)), int(rng.integers(1, 2000))
        vs = [float(v) for v in rng.choice([0.1, 0.25, 0.4, 0.5, 1.0, 2.0], size=3)]
        lo = [float(v) for v in rng.uniform(-5, 1, size=3)]
        cells = [int(rng.integers(1, 40)) for _ in range(3)]
        cr = lo + [lo[a] + vs[a] * cells[a] for a in range(3)]
        pts = rng.uniform(-8, 45, (npts, f)).astype(np.float32)
        inside = rng.random(npts) < 0.7
        for a in range(3):
            pts[inside, a] = rng.uniform(cr[a], cr[3 + a], inside.sum()).astype(np.float32)
        if npts and rng.integers(0, 4) == 0:
            pts[rng.integers(0, npts), rng.integers(0, 3)] = rng.choice([np.nan, np.inf, -np.inf, 1e30, -1e30])
        if npts > 10 and rng.integers(0, 2) == 0:           # repeated points: crowded cells
            pts[npts // 2:] = pts[rng.integers(0, npts // 2, npts - npts // 2)]
        what = "seed %d: %d points x %d, max_points %d, max_voxels %d, cells %s" % (seed, npts, f, max_points,
                                                                                 max_voxels, cells)
        print(what, flush=True)
        try:
            out = m.voxelization(gpu_handle, torch.from_numpy(pts).cuda(), torch.tensor(vs, dtype=torch.float32).cuda(),
                                 torch.tensor(cr, dtype=torch.float32).cuda(), max_points, max_voxels)
        except m.MluOpError:
            continue   # e.g. no points: refused as in the reference
        torch.cuda.synchronize()
        want = vox.voxelization(pts, vs, cr, max_points, max_voxels)
        assert int(out[3].item()) == want[3], what
        for got, ref in zip(out[:3], want[:3]):
            assert np.array_equal(got.cpu().numpy(), ref, equal_nan=True), what
        done += 1
    assert done >= 40


@pytest.mark.parametrize("block", range(3))
def test_dynamic_point_to_voxel(gpu_handle, block):
    import torch
    import mluop_hip as m
    for case in range(60):
        seed = 9000 + block * 100 + case
        rng = np.random.default_rng(seed)
        npts, c, span = int(rng.integers(1, 4000)), int(rng.integers(1, 12)), int(rng.integers(1, 30))
        mode = str(rng.choice(["max", "mean"]))
        whole = bool(rng.integers(0, 2))                       # whole numbers: ties in the maximum
        feats = (rng.integers(-3, 4, (npts, c)) if whole else rng.uniform(-100, 100, (npts, c))).astype(np.float32)
        huge = bool(rng.integers(0, 5) == 0)                   # coordinates up to 2^31 - 1: 64-bit keys
        coors = rng.integers(0, 2 ** 31 - 1 if huge else span, (npts, 3)).astype(np.int32)
        k = int(npts * rng.choice([0.0, 0.1, 0.5]))
        if k:
            coors[rng.choice(npts, k, replace=False), rng.integers(0, 3, k)] = -rng.integers(1, 5, k)
        rows = None if rng.integers(0, 3) else int(rng.integers(1, npts + 1))
        what = "seed %d: %d points x %d, span %d, %s, rows %s" % (seed, npts, c, span, mode, rows)
        print(what, flush=True)
        tf, tc = torch.from_numpy(feats).cuda(), torch.from_numpy(coors.copy()).cuda()
        out = m.dynamic_point_to_voxel_forward(gpu_handle, tf, tc, mode, rows)
        torch.cuda.synchronize()
        got = [t.cpu().numpy() for t in out[:4]] + [int(out[4].item()), tc.cpu().numpy()]
        for g, ref in zip(got, dpv.forward(mode, feats, coors, rows)):
            assert np.array_equal(g, ref), what
        if mode == "max" and rows is None:
            grad_out = rng.standard_normal((npts, c)).astype(np.float32)
            grad = m.dynamic_point_to_voxel_backward(gpu_handle, torch.from_numpy(grad_out).cuda(), tf, out[0], out[2],
                                                     out[3], out[4])
            torch.cuda.synchronize()
            assert np.array_equal(grad.cpu().numpy(), dpv.backward(grad_out, feats, got[0], got[2], got[4])), what
