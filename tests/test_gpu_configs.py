"""BASELINE configs 2, 3 and 5 at full size through the C ABI (configs 1 and 4 live beside the
per-operator tests).  Rulebooks are compared bit-exactly with the CPU oracle.  Convolutions are
compared with the oracle where it finishes in seconds; for config 5 (1e11 multiply-adds) a
seeded sample of result rows is recomputed in float64 from the rulebook itself and graded at
the same diff1/diff2 thresholds."""
import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import THRESH, check_close, from_torch, out_space, random_voxels, round_to, to_torch

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


def gpu_rulebook(handle, idx, batch, space, ks, pad, stride, dil, sub_m):
    import torch
    import mluop_hip
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    t = torch.from_numpy(idx).cuda()
    pairs, out_idx, num, n_out = mluop_hip.get_indice_pairs(handle, t, batch, space, ks, ospace, pad, stride,
                                                           dil, sub_m)
    torch.cuda.synchronize()
    return pairs, out_idx, num, n_out, ospace


def assert_rulebook_exact(pairs, out_idx, num, n_out, idx, batch, ks, pad, stride, dil, ospace, sub_m):
    rp, ro, rn, rn_out = oracle.get_indice_pairs(idx, batch, pad, stride, dil, ks, ospace, sub_m,
                                                 out_rows=out_idx.shape[0], exact_count=True)
    assert np.array_equal(num.cpu().numpy(), rn), "indice_num"
    assert n_out == rn_out
    assert np.array_equal(out_idx.cpu().numpy(), ro), "out_indices"
    assert np.array_equal(pairs.cpu().numpy(), rp), "indice_pairs"


def sampled_rows_reference(feats, w_k, pairs_np, num, rows):
    """float64 forward result for the output rows `rows` only, straight from the rulebook."""
    n_rows_total = int(pairs_np[:, 1, :].max()) + 1
    pos = np.full(max(n_rows_total, int(rows.max()) + 1), -1, dtype=np.int64)
    pos[rows] = np.arange(rows.size)
    out = np.zeros((rows.size, w_k.shape[2]), dtype=np.float64)
    f64 = feats.astype(np.float64)
    for k in range(w_k.shape[0]):
        n = int(num[k])
        if n == 0:
            continue
        o = pairs_np[k, 1, :n]
        i = pairs_np[k, 0, :n]
        where = pos[o]
        sel = where >= 0
        if sel.any():
            np.add.at(out, where[sel], f64[i[sel]] @ w_k[k].astype(np.float64))
    return out


def grade_sample(dev_rows, ref_rows, dtype_name, what):
    ref = round_to(ref_rows.astype(np.float32), dtype_name)
    d1, d2 = oracle.diff1(dev_rows, ref), oracle.diff2(dev_rows, ref)
    assert np.isfinite(dev_rows).all(), what
    assert d1 <= THRESH[dtype_name] and d2 <= THRESH[dtype_name], "%s diff1=%.3e diff2=%.3e" % (what, d1, d2)


def test_config2_subm_two_batches_fp16(gpu_handle):
    """Config 2: 2 x 60 000 clustered voxels in 2x41x1600x1408, subm 3x3x3, Ci=Co=32 fp16."""
    import mluop_hip
    space, ks = (41, 1600, 1408), (3, 3, 3)
    idx = mluop_hip.datagen.clustered_voxels((2,) + space, 60000, seed=2)
    pairs, out_idx, num, n_out, ospace = gpu_rulebook(gpu_handle, idx, 2, space, ks, [1, 1, 1], [1, 1, 1],
                                                      [1, 1, 1], True)
    assert_rulebook_exact(pairs, out_idx, num, n_out, idx, 2, ks, [1, 1, 1], [1, 1, 1], [1, 1, 1], ospace, True)
    rng = np.random.default_rng(2)
    feats = round_to(rng.standard_normal((idx.shape[0], 32)).astype(np.float32), "float16")
    w = round_to(mluop_hip.datagen.kaiming_uniform_filters(ks, 32, 32, seed=2), "float16")
    num_host = num.cpu().tolist()
    out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats, "float16", "cuda"),
                                        to_torch(w, "float16", "cuda"), mluop_hip.LAYOUT_ARRAY, pairs,
                                        num_host, n_out, True)
    ref = oracle.forward(feats, w.reshape(27, 32, 32), pairs.cpu().numpy(), num_host, n_out)
    check_close(from_torch(out), ref, "float16", "config2 forward")


def test_config3_regular_stride2_bf16_forward(gpu_handle):
    """Config 3: 4 x 30 000 clustered voxels, regular 3x3x3 stride 2 pad 1, Ci=Co=64 bf16; the forward
    consumes the rulebook and num_act_out the library produced."""
    import mluop_hip
    space, ks = (41, 1600, 1408), (3, 3, 3)
    idx = mluop_hip.datagen.clustered_voxels((4,) + space, 30000, seed=3)
    pairs, out_idx, num, n_out, ospace = gpu_rulebook(gpu_handle, idx, 4, space, ks, [1, 1, 1], [2, 2, 2],
                                                      [1, 1, 1], False)
    assert ospace == [21, 800, 704]
    rng = np.random.default_rng(3)
    feats = round_to(rng.standard_normal((idx.shape[0], 64)).astype(np.float32), "bfloat16")
    w = round_to(mluop_hip.datagen.kaiming_uniform_filters(ks, 64, 64, seed=3), "bfloat16")
    num_host = num.cpu().tolist()
    out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats, "bfloat16", "cuda"),
                                        to_torch(w, "bfloat16", "cuda"), mluop_hip.LAYOUT_ARRAY, pairs,
                                        num_host, n_out, False)
    assert out.shape[0] == n_out
    ref = oracle.forward(feats, w.reshape(27, 64, 64), pairs.cpu().numpy(), num_host, n_out)
    check_close(from_torch(out), ref, "bfloat16", "config3 forward")


@pytest.fixture(scope="module")
def config5_voxels():
    import mluop_hip
    return mluop_hip.datagen.surface_voxels((1, 64, 1024, 1024), 400000, seed=5)


def test_config5a_subm_5x5x5_rulebook_and_forward(gpu_handle, config5_voxels):
    """Config 5a: 400 000 surface voxels in 1x64x1024x1024, subm 5x5x5 pad 2, Ci=Co=128, fp16 (MFMA
    path, five chunks of offsets) and fp32; indice_pairs alone is 400 MB."""
    import torch
    import mluop_hip
    idx = config5_voxels
    space, ks, pad = (64, 1024, 1024), (5, 5, 5), [2, 2, 2]
    pairs, out_idx, num, n_out, ospace = gpu_rulebook(gpu_handle, idx, 1, space, ks, pad, [1, 1, 1], [1, 1, 1],
                                                      True)
    assert_rulebook_exact(pairs, out_idx, num, n_out, idx, 1, ks, pad, [1, 1, 1], [1, 1, 1], ospace, True)
    num_host = num.cpu().tolist()
    assert num_host[62] == idx.shape[0]  # centre offset pairs every row with itself
    pairs_np = pairs.cpu().numpy()
    rng = np.random.default_rng(5)
    rows = np.sort(rng.choice(n_out, size=3000, replace=False))
    feats32 = rng.standard_normal((idx.shape[0], 128)).astype(np.float32)
    w32 = mluop_hip.datagen.kaiming_uniform_filters(ks, 128, 128, seed=5)
    for dtype_name in ("float16", "float32"):
        print("config5a forward", dtype_name, "pairs", int(sum(num_host)), flush=True)
        feats, w = round_to(feats32, dtype_name), round_to(w32, dtype_name)
        out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats, dtype_name, "cuda"),
                                            to_torch(w, dtype_name, "cuda"), mluop_hip.LAYOUT_ARRAY, pairs,
                                            num_host, n_out, True)
        torch.cuda.synchronize()
        ref = sampled_rows_reference(feats, w.reshape(125, 128, 128), pairs_np, num_host, rows)
        grade_sample(from_torch(out[torch.from_numpy(rows).cuda()]), ref, dtype_name, "config5a " + dtype_name)
        del out

    # backward data and backward filter on the same rulebook, fp16: input-gradient rows of a sample
    # (the forward sum with the pair columns swapped and every filter slice transposed), and the filter
    # gradient of four offsets (centre, both ends, one in between) as X[in]^T dY[out] over their pairs
    print("config5a backward data", flush=True)
    dy = round_to((rng.standard_normal((n_out, 128)) * 0.1).astype(np.float32), "float16")
    w = round_to(w32, "float16")
    feats = round_to(feats32, "float16")
    t_dy, t_w, t_f = (to_torch(a, "float16", "cuda") for a in (dy, w, feats))
    dx = mluop_hip.indice_conv_backward_data(gpu_handle, t_dy, t_w, mluop_hip.LAYOUT_ARRAY, pairs, num_host, True,
                                             128)
    torch.cuda.synchronize()
    swapped = np.ascontiguousarray(pairs_np[:, ::-1, :])
    w_t = np.ascontiguousarray(w.reshape(125, 128, 128).transpose(0, 2, 1))
    ref = sampled_rows_reference(dy, w_t, swapped, num_host, rows)
    grade_sample(from_torch(dx[torch.from_numpy(rows).cuda()]), ref, "float16", "config5a backward data")
    del dx
    print("config5a backward filter", flush=True)
    dw = mluop_hip.indice_conv_backward_filter(gpu_handle, t_f, t_dy, pairs, num_host, ks, True)
    torch.cuda.synchronize()
    dw_np = from_torch(dw).reshape(125, 128, 128)
    for k in (0, 37, 62, 124):
        n = num_host[k]
        ref_k = feats[pairs_np[k, 0, :n]].astype(np.float64).T @ dy[pairs_np[k, 1, :n]].astype(np.float64)
        grade_sample(dw_np[k], ref_k, "float16", "config5a backward filter, offset %d" % k)


def test_config5a_rows_out_of_order_take_the_row_map_in_chunks(gpu_handle, config5_voxels):
    """The same 400 000 voxels in shuffled row order: forward cannot read the pair lists by result
    row and builds row maps, 64 MiB (131 072 rows of 125 offsets) at a time: four chunks."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(55)
    idx = np.ascontiguousarray(config5_voxels[rng.permutation(config5_voxels.shape[0])])
    space, ks, pad = (64, 1024, 1024), (5, 5, 5), [2, 2, 2]
    pairs, out_idx, num, n_out, ospace = gpu_rulebook(gpu_handle, idx, 1, space, ks, pad, [1, 1, 1], [1, 1, 1],
                                                      True)
    num_host = num.cpu().tolist()
    feats = round_to(rng.standard_normal((idx.shape[0], 128)).astype(np.float32), "float16")
    w = round_to(mluop_hip.datagen.kaiming_uniform_filters(ks, 128, 128, seed=5), "float16")
    gpu_handle.set_kernel_timing(True)
    try:
        out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats, "float16", "cuda"),
                                            to_torch(w, "float16", "cuda"), mluop_hip.LAYOUT_ARRAY, pairs, num_host,
                                            n_out, True)
        names = [n for n, _ in gpu_handle.kernel_timings()]
    finally:
        gpu_handle.set_kernel_timing(False)
    assert names.count("scatterRowMap") == 4 and names.count("repairLostPairs") == 4, names
    rows = np.sort(rng.choice(n_out, size=3000, replace=False))
    ref = sampled_rows_reference(feats, w.reshape(125, 128, 128), pairs.cpu().numpy(), num_host, rows)
    grade_sample(from_torch(out[torch.from_numpy(rows).cuda()]), ref, "float16", "config5a, shuffled rows")


def test_config5b_regular_2x2x2_stride2_on_5a_outputs(gpu_handle, config5_voxels):
    """Config 5b: regular 2x2x2 stride 2 pad 0 over the rows 5a leaves (a submanifold layer keeps
    its input coordinates), out 1x32x512x512, Ci=Co=128, fp16 and fp32."""
    import torch
    import mluop_hip
    idx = config5_voxels
    space, ks, pad = (64, 1024, 1024), (2, 2, 2), [0, 0, 0]
    pairs, out_idx, num, n_out, ospace = gpu_rulebook(gpu_handle, idx, 1, space, ks, pad, [2, 2, 2], [1, 1, 1],
                                                      False)
    assert ospace == [32, 512, 512]
    assert_rulebook_exact(pairs, out_idx, num, n_out, idx, 1, ks, pad, [2, 2, 2], [1, 1, 1], ospace, False)
    num_host = num.cpu().tolist()
    assert sum(num_host) == idx.shape[0]  # stride = kernel edge: every input row lands in exactly one pair
    rng = np.random.default_rng(6)
    feats32 = rng.standard_normal((idx.shape[0], 128)).astype(np.float32)
    w32 = mluop_hip.datagen.kaiming_uniform_filters(ks, 128, 128, seed=6)
    rows = np.sort(rng.choice(n_out, size=3000, replace=False))
    pairs_np = pairs.cpu().numpy()
    for dtype_name in ("float16", "float32"):
        print("config5b forward", dtype_name, flush=True)
        feats, w = round_to(feats32, dtype_name), round_to(w32, dtype_name)
        out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats, dtype_name, "cuda"),
                                            to_torch(w, dtype_name, "cuda"), mluop_hip.LAYOUT_ARRAY, pairs, num_host,
                                            n_out, False)
        torch.cuda.synchronize()
        ref = sampled_rows_reference(feats, w.reshape(8, 128, 128), pairs_np, num_host, rows)
        grade_sample(from_torch(out[torch.from_numpy(rows).cuda()]), ref, dtype_name, "config5b " + dtype_name)
        del out

@pytest.mark.timeout(600)
def test_convolutions_at_one_million_rows(gpu_handle):
    """The most rows the API accepts (1 000 000), submanifold 3x3x3 at 64 channels fp16, checked
    through properties that need no CPU pass over the whole tensor: a filter that is the identity at
    the centre offset and zero elsewhere returns its input bit for bit (forward and backward data);
    a random filter is compared with numpy on 2 000 sampled rows; the centre slice of the filter
    gradient is the dense product X^T dY, computed by torch in fp32."""
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(91)
    space, L, C, ks = (48, 512, 512), 1000000, 64, (3, 3, 3)
    idx = random_voxels(rng, 2, space, L)
    print("rulebook 1M", flush=True)
    pairs, out_idx, num, n_out = m.get_indice_pairs(gpu_handle, torch.from_numpy(idx).cuda(), 2, space, ks, list(space),
                                                    [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    num_host = num.cpu().tolist()
    assert n_out == L and num_host[13] == L
    x = torch.randn(L, C, device="cuda").half()
    dy = (torch.randn(L, C, device="cuda") * 0.1).half()
    eye = torch.zeros(ks + (C, C), device="cuda", dtype=torch.float16)
    eye[1, 1, 1] = torch.eye(C, device="cuda", dtype=torch.float16)
    print("identity filter", flush=True)
    out = m.indice_conv_forward(gpu_handle, x, eye, m.LAYOUT_ARRAY, pairs, num_host, L, True)
    dx = m.indice_conv_backward_data(gpu_handle, dy, eye, m.LAYOUT_ARRAY, pairs, num_host, True, C)
    torch.cuda.synchronize()
    assert torch.equal(out, x) and torch.equal(dx, dy)

    print("random filter, sampled rows", flush=True)
    w = (torch.randn(ks + (C, C), device="cuda") / np.sqrt(27 * C)).half()
    out = m.indice_conv_forward(gpu_handle, x, w, m.LAYOUT_ARRAY, pairs, num_host, L, True)
    dw = m.indice_conv_backward_filter(gpu_handle, x, dy, pairs, num_host, ks, True)
    torch.cuda.synchronize()
    rows = rng.choice(L, size=2000, replace=False)
    pn = pairs.cpu().numpy()
    xf, wf = x.float().cpu().numpy(), w.float().cpu().numpy().reshape(27, C, C)
    ref = np.zeros((2000, C), np.float64)
    pos = {int(r): i for i, r in enumerate(rows)}
    for k in range(27):
        o = pn[k, 1, :num_host[k]]
        sel = np.nonzero(np.isin(o, rows))[0]
        for p in sel:
            ref[pos[int(o[p])]] += xf[pn[k, 0, p]].astype(np.float64) @ wf[k]
    got = out[torch.from_numpy(rows).cuda()].float().cpu().numpy()
    check_close(got, ref.astype(np.float32), "float16", "forward, sampled rows")
    centre = (x.float().t() @ dy.float()).cpu().numpy()
    check_close(dw[1, 1, 1].float().cpu().numpy(), centre, "float16", "backward filter, centre offset")
