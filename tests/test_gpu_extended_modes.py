"""GPU parity of the modes the reference rejects and this library offers behind a handle switch
(mluOpExtSetSparseConvExtendedModes): inverse = 1 for the three indice-convolution operators and
filters_grad written in its tagged layout.

The oracle's inverse functions run the partner layer's rulebook backwards; they are pinned on the
CPU against dense conv_transpose3d (test_oracle_conv.py).  Inputs and grading are those of
test_gpu_conv.py: seeded values rounded through the tensor dtype, diff1/diff2 at the reference's
thresholds."""

import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import check_close, from_torch, out_space, random_voxels, round_to, to_torch

pytestmark = pytest.mark.gpu


@pytest.fixture()
def extended_handle(gpu_handle):
    gpu_handle.set_extended_modes(True)
    yield gpu_handle
    gpu_handle.set_extended_modes(False)


def inverse_case(seed, batch, space, L, ks, stride, ci, co):
    """A strided layer's rulebook and tensors of its inverse partner: features on the strided
    layer's output cells (ci channels), results on its input cells (co channels)."""
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, batch, space, L)
    pad = [k // 2 for k in ks]
    ospace = out_space(space, ks, pad, stride, [1, 1, 1])
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, batch, pad, list(stride), [1, 1, 1], list(ks), ospace,
                                                         False, exact_count=True)
    K = int(np.prod(ks))
    b = 1.0 / np.sqrt(K * ci)
    return dict(pairs=pairs, num=num, L=idx.shape[0], n_out=n_out, K=K, ks=ks, ci=ci, co=co,
                feats=rng.standard_normal((n_out, ci)).astype(np.float32),
                w=rng.uniform(-b, b, size=tuple(ks) + (ci, co)).astype(np.float32),
                dy=(rng.standard_normal((idx.shape[0], co)) * 1e-1).astype(np.float32))


INVERSE_SHAPES = [
    # (batch, space, L, ks, stride, ci, co)
    (1, (8, 8, 8), 300, (3, 3, 3), (2, 2, 2), 32, 16),
    (2, (8, 10, 10), 500, (3, 3, 3), (2, 2, 2), 64, 32),
    (1, (10, 12, 12), 900, (3, 3, 3), (2, 2, 2), 64, 64),
    (1, (8, 8, 8), 400, (3, 3, 3), (1, 1, 1), 128, 128),     # stride 1: dense enough for the register-accumulating kernel
    (1, (8, 8, 8), 300, (2, 2, 2), (2, 2, 2), 128, 64),
    (1, (6, 6, 6), 100, (1, 3, 3), (1, 2, 1), 13, 70),        # odd channel counts -> SIMT
    (1, (10, 10, 10), 400, (5, 5, 7), (2, 2, 2), 32, 32),     # K = 175: counts in device memory
]


@pytest.mark.parametrize("shape", INVERSE_SHAPES)
@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_inverse_ops_match_oracle(extended_handle, shape, dtype_name):
    import torch
    import mluop_hip
    print("inverse conv case", shape, dtype_name, flush=True)
    c = inverse_case(21, *shape)
    feats_r, w_r, dy_r = (round_to(c[k], dtype_name) for k in ("feats", "w", "dy"))
    w_k = w_r.reshape(c["K"], c["ci"], c["co"])
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    feats_t, w_t, dy_t = (to_torch(a, dtype_name, "cuda") for a in (feats_r, w_r, dy_r))
    h = extended_handle
    out = mluop_hip.indice_conv_forward(h, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host, c["L"], False,
                                        inverse=1)
    dx = mluop_hip.indice_conv_backward_data(h, dy_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host, False,
                                             c["ci"], inverse=1, rows=c["n_out"])
    dw = mluop_hip.indice_conv_backward_filter(h, feats_t, dy_t, pairs_t, num_host, c["ks"], False, inverse=1)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (c["L"], c["co"]) and tuple(dx.shape) == (c["n_out"], c["ci"])
    check_close(from_torch(out), oracle.forward(feats_r, w_k, c["pairs"], c["num"], c["L"], inverse=True),
                dtype_name, "inverse forward")
    check_close(from_torch(dx),
                oracle.backward_data(dy_r, w_k, c["pairs"], c["num"], inverse=True, rows=c["n_out"]),
                dtype_name, "inverse backward_data")
    ref_dw = oracle.backward_filter(feats_r, dy_r, c["pairs"], c["num"], fast=True, inverse=True)
    check_close(from_torch(dw).reshape(ref_dw.shape), ref_dw, dtype_name, "inverse backward_filter")


@pytest.mark.parametrize("dtype_name", ["float32", "float16"])
def test_inverse_forward_is_partner_backward_data(extended_handle, dtype_name):
    """Bit for bit: the inverse forward gathers and multiplies exactly what the partner layer's
    backward data does when handed the filter with its channel roles exchanged."""
    import torch
    import mluop_hip
    c = inverse_case(22, 1, (10, 12, 12), 900, (3, 3, 3), (2, 2, 2), 64, 32)
    feats_t = to_torch(round_to(c["feats"], dtype_name), dtype_name, "cuda")
    w_r = round_to(c["w"], dtype_name)
    w_t = to_torch(w_r, dtype_name, "cuda")
    w_swapped = to_torch(np.ascontiguousarray(np.swapaxes(w_r, 3, 4)), dtype_name, "cuda")  # [kd,kh,kw,co,ci]
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    out = mluop_hip.indice_conv_forward(extended_handle, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host,
                                        c["L"], False, inverse=1)
    same = mluop_hip.indice_conv_backward_data(extended_handle, feats_t, w_swapped, mluop_hip.LAYOUT_ARRAY, pairs_t,
                                               num_host, False, c["co"])
    torch.cuda.synchronize()
    assert torch.equal(out, same)


def test_inverse_is_rejected_without_the_switch(gpu_handle):
    """A fresh handle answers inverse = 1 as the reference does."""
    import torch
    import mluop_hip
    c = inverse_case(23, 1, (8, 8, 8), 200, (3, 3, 3), (2, 2, 2), 16, 16)
    feats_t = to_torch(c["feats"], "float32", "cuda")
    w_t = to_torch(c["w"], "float32", "cuda")
    dy_t = to_torch(c["dy"], "float32", "cuda")
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    with pytest.raises(mluop_hip.MluOpError) as e:
        mluop_hip.indice_conv_forward(gpu_handle, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host, c["L"],
                                      False, inverse=1)
    assert e.value.status == mluop_hip.STATUS_NOT_SUPPORTED
    with pytest.raises(mluop_hip.MluOpError) as e:
        mluop_hip.indice_conv_backward_data(gpu_handle, dy_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host, False,
                                            c["ci"], inverse=1, rows=c["n_out"])
    assert e.value.status == mluop_hip.STATUS_NOT_SUPPORTED
    with pytest.raises(mluop_hip.MluOpError) as e:
        mluop_hip.indice_conv_backward_filter(gpu_handle, feats_t, dy_t, pairs_t, num_host, c["ks"], False,
                                              inverse=1)
    assert e.value.status == mluop_hip.STATUS_BAD_PARAM


GRAD_LAYOUT_SHAPES = [
    # (ks, ci, co, force the SIMT path)
    ((3, 3, 3), 32, 64, False),
    ((3, 3, 3), 64, 16, False),
    ((3, 3, 3), 32, 64, True),
    ((1, 3, 3), 13, 70, False),
]


@pytest.mark.parametrize("shape", GRAD_LAYOUT_SHAPES)
@pytest.mark.parametrize("layout_name", ["NDHWC", "NCDHW", "ARRAY"])
@pytest.mark.parametrize("dtype_name", ["float32", "float16"])
def test_filters_grad_in_its_tagged_layout(extended_handle, shape, layout_name, dtype_name):
    import torch
    import mluop_hip
    ks, ci, co, simt = shape
    rng = np.random.default_rng(24)
    idx = random_voxels(rng, 1, (8, 8, 8), 300)
    pad = [k // 2 for k in ks]
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, 1, pad, [1, 1, 1], [1, 1, 1], list(ks),
                                                         out_space((8, 8, 8), ks, pad, [1, 1, 1], [1, 1, 1]), False,
                                                         exact_count=True)
    feats_r = round_to(rng.standard_normal((300, ci)).astype(np.float32), dtype_name)
    dy_r = round_to((rng.standard_normal((n_out, co)) * 1e-1).astype(np.float32), dtype_name)
    code = {"NDHWC": mluop_hip.LAYOUT_NDHWC, "NCDHW": mluop_hip.LAYOUT_NCDHW, "ARRAY": mluop_hip.LAYOUT_ARRAY}[
        layout_name]
    extended_handle.set_kernel_choice("gather_simt", True if simt else None)
    try:
        dw = mluop_hip.indice_conv_backward_filter(extended_handle, to_torch(feats_r, dtype_name, "cuda"),
                                                   to_torch(dy_r, dtype_name, "cuda"), torch.from_numpy(pairs).cuda(),
                                                   [int(v) for v in num], ks, False, grad_layout=code)
        torch.cuda.synchronize()
    finally:
        extended_handle.set_kernel_choice("gather_simt", None)
    got = from_torch(dw)
    K = int(np.prod(ks))
    # back to [K, Ci, Co] with the oracle's own layout transpose (the one the forward tests pin)
    got_k = oracle.filters_to_kcico(np.ascontiguousarray(got), code, K, ci, co)
    ref = oracle.backward_filter(feats_r, dy_r, pairs, num, fast=True)
    check_close(got_k, ref, dtype_name, "backward_filter " + layout_name)
    if layout_name != "ARRAY":
        assert got.shape[0] == co and got.shape[-1 if layout_name == "NDHWC" else 1] == ci
