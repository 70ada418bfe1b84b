"""GPU parity of the three indice-convolution operators against the CPU oracle.

Inputs are seeded fp32 values rounded through the tensor dtype (so device and oracle see the
same numbers), the oracle accumulates in fp32 and its result is rounded through the output
dtype, then diff1/diff2 are graded at the reference's thresholds (spconv_cases.THRESH)."""

import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import check_close, from_torch, out_space, random_voxels, round_to, to_torch

pytestmark = pytest.mark.gpu


def build_rulebook(idx, batch, space, ks, pad, stride, dil, sub_m):
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, batch, pad, stride, dil, ks, ospace, sub_m,
                                                         exact_count=True)
    return pairs, num, n_out


def conv_case(seed, batch, space, L, ks, ci, co, sub_m, stride=(1, 1, 1)):
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, batch, space, L)
    pad = [k // 2 for k in ks]
    pairs, num, n_out = build_rulebook(idx, batch, space, ks, pad, list(stride), [1, 1, 1], sub_m)
    K = int(np.prod(ks))
    feats = rng.standard_normal((idx.shape[0], ci)).astype(np.float32)
    b = 1.0 / np.sqrt(K * ci)
    w = rng.uniform(-b, b, size=tuple(ks) + (ci, co)).astype(np.float32)
    dy = (rng.standard_normal((n_out, co)) * 1e-1).astype(np.float32)
    return dict(idx=idx, pairs=pairs, num=num, n_out=n_out, feats=feats, w=w, dy=dy, K=K, ks=ks,
                ci=ci, co=co, sub_m=sub_m)


def run_all_ops(handle, c, dtype_name, force_simt=False, check=("fwd", "bwd_data", "bwd_filter")):
    import torch
    import mluop_hip
    handle.set_kernel_choice("gather_simt", True if force_simt else None)
    try:
        dev = "cuda"
        feats_r = round_to(c["feats"], dtype_name)
        w_r = round_to(c["w"], dtype_name)
        dy_r = round_to(c["dy"], dtype_name)
        w_k = w_r.reshape(c["K"], c["ci"], c["co"])
        pairs_t = torch.from_numpy(c["pairs"]).cuda()
        num_host = [int(v) for v in c["num"]]
        feats_t = to_torch(feats_r, dtype_name, dev)
        w_t = to_torch(w_r, dtype_name, dev)
        dy_t = to_torch(dy_r, dtype_name, dev)
        res = {}
        if "fwd" in check:
            out = mluop_hip.indice_conv_forward(handle, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host,
                                                c["n_out"], c["sub_m"])
            torch.cuda.synchronize()
            ref = oracle.forward(feats_r, w_k, c["pairs"], c["num"], c["n_out"])
            res["fwd"] = check_close(from_torch(out), ref, dtype_name, "forward")
        if "bwd_data" in check:
            dx = mluop_hip.indice_conv_backward_data(handle, dy_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host,
                                                     c["sub_m"], c["ci"])
            torch.cuda.synchronize()
            ref = oracle.backward_data(dy_r, w_k, c["pairs"], c["num"])
            res["bwd_data"] = check_close(from_torch(dx), ref, dtype_name, "backward_data")
        if "bwd_filter" in check:
            dw = mluop_hip.indice_conv_backward_filter(handle, feats_t, dy_t, pairs_t, num_host, c["ks"],
                                                       c["sub_m"])
            torch.cuda.synchronize()
            ref = oracle.backward_filter(feats_r, dy_r, c["pairs"], c["num"], fast=True)
            res["bwd_filter"] = check_close(from_torch(dw).reshape(ref.shape), ref, dtype_name,
                                            "backward_filter")
        return res
    finally:
        handle.set_kernel_choice("gather_simt", None)


SHAPES = [
    # (batch, space, L, ks, ci, co, sub_m, stride)
    (1, (6, 6, 6), 50, (3, 3, 3), 16, 16, True, (1, 1, 1)),
    (2, (8, 9, 10), 400, (3, 3, 3), 32, 32, True, (1, 1, 1)),
    (2, (8, 9, 10), 400, (3, 3, 3), 16, 32, True, (1, 1, 1)),     # 16 reduction channels: half-filled fragments for fp16/bf16
    (1, (8, 8, 8), 300, (3, 3, 3), 32, 16, False, (2, 2, 2)),
    (1, (10, 12, 12), 900, (3, 3, 3), 64, 64, True, (1, 1, 1)),
    (2, (8, 10, 10), 500, (3, 3, 3), 64, 32, False, (2, 2, 2)),
    (1, (8, 8, 8), 300, (3, 3, 3), 32, 128, True, (1, 1, 1)),
    (1, (8, 8, 8), 300, (3, 3, 3), 128, 64, False, (1, 1, 1)),
    (1, (8, 8, 8), 300, (3, 3, 3), 128, 128, True, (1, 1, 1)),     # dense: whole 128-column tiles
    (1, (20, 20, 20), 300, (3, 3, 3), 128, 128, True, (1, 1, 1)),  # sparse: two 64-column halves
    (1, (6, 6, 6), 100, (3, 3, 3), 21, 10, True, (1, 1, 1)),   # odd channel counts -> SIMT
    (1, (6, 6, 6), 100, (1, 3, 3), 13, 70, False, (1, 2, 1)),
    (1, (6, 6, 6), 120, (3, 3, 3), 260, 300, True, (1, 1, 1)),   # wider than any matrix-core instance
    (1, (10, 10, 10), 400, (5, 5, 7), 32, 32, True, (1, 1, 1)),   # K = 175: counts in device memory, seven chunks of offsets
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_conv_ops_match_oracle(gpu_handle, shape, dtype_name):
    batch, space, L, ks, ci, co, sub_m, stride = shape
    print("conv case", shape, dtype_name, flush=True)
    c = conv_case(11, batch, space, L, ks, ci, co, sub_m, stride)
    run_all_ops(gpu_handle, c, dtype_name)


@pytest.mark.parametrize("dtype_name", ["float16", "bfloat16"])
def test_simt_path_matches_oracle_on_mfma_shapes(gpu_handle, dtype_name):
    c = conv_case(12, 2, (8, 9, 10), 400, (3, 3, 3), 64, 64, True)
    run_all_ops(gpu_handle, c, dtype_name, force_simt=True, check=("fwd", "bwd_data"))


DENSE_SHAPES = [
    # the register-accumulating kernel takes 16 to 128 result columns; (8, 8, 8) with 300 voxels is dense
    (1, (8, 8, 8), 300, (3, 3, 3), 16, 16, True, (1, 1, 1)),      # half a reduction fragment in fp16
    (2, (8, 8, 8), 500, (3, 3, 3), 16, 32, True, (1, 1, 1)),
    (1, (8, 8, 8), 300, (3, 3, 3), 32, 16, False, (1, 1, 1)),
    (1, (10, 10, 10), 700, (3, 3, 3), 32, 32, True, (1, 1, 1)),   # 700 rows: three tiles of 256
    (1, (9, 9, 9), 500, (3, 3, 3), 16, 128, False, (2, 2, 2)),
    (1, (8, 8, 8), 300, (3, 3, 3), 64, 64, True, (1, 1, 1)),
    (1, (8, 8, 8), 300, (3, 3, 3), 128, 128, True, (1, 1, 1)),
    (2, (8, 8, 8), 500, (3, 3, 3), 32, 128, True, (1, 1, 1)),
    (1, (8, 8, 8), 300, (3, 3, 3), 128, 64, False, (1, 1, 1)),
    (1, (6, 6, 6), 150, (5, 5, 7), 64, 128, True, (1, 1, 1)),     # K = 175: six chunks of offsets
    (1, (20, 20, 20), 130, (3, 3, 3), 64, 64, True, (1, 1, 1)),    # sparse input through the dense kernel
]


@pytest.mark.parametrize("shape", DENSE_SHAPES)
@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_dense_kernel_matches_oracle(gpu_handle, shape, dtype_name):
    """The same operators with the dense-rulebook kernel forced on (and, for comparison, off)."""
    batch, space, L, ks, ci, co, sub_m, stride = shape
    print("dense conv case", shape, dtype_name, flush=True)
    c = conv_case(12, batch, space, L, ks, ci, co, sub_m, stride)
    for force in (True, False):
        gpu_handle.set_kernel_choice("dense_tiles", force)
        try:
            run_all_ops(gpu_handle, c, dtype_name, check=("fwd", "bwd_data"))
        finally:
            gpu_handle.set_kernel_choice("dense_tiles", None)


@pytest.mark.parametrize("shape", [
    # (space, L, ks, ci, co, sub_m, stride): slices of several chunks of row indices, ragged ends
    ((14, 20, 20), 4000, (3, 3, 3), 128, 128, True, (1, 1, 1)),
    ((14, 20, 20), 3100, (3, 3, 3), 64, 32, True, (1, 1, 1)),
    ((12, 30, 30), 5000, (3, 3, 3), 32, 128, False, (2, 2, 2)),
    ((6, 6, 6), 150, (5, 5, 5), 64, 64, True, (1, 1, 1)),      # 125 offsets, short lists
])
@pytest.mark.parametrize("dtype_name", ["float16", "bfloat16"])
def test_backward_filter_kernels_agree(gpu_handle, shape, dtype_name):
    """2-byte types of 32 to 128 channels: the kernel that reads its operand fragments with the
    transposing LDS read against the oracle, and bit for bit against the kernel that transposes with
    element-sized stores (same products, same order of sums)."""
    import torch
    import mluop_hip
    space, L, ks, ci, co, sub_m, stride = shape
    print("backward filter case", shape, dtype_name, flush=True)
    c = conv_case(14, 1, space, L, ks, ci, co, sub_m, stride)
    feats_t = to_torch(round_to(c["feats"], dtype_name), dtype_name, "cuda")
    dy_t = to_torch(round_to(c["dy"], dtype_name), dtype_name, "cuda")
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    got = {}
    for stores in (False, True):
        gpu_handle.set_kernel_choice("filter_stores", True if stores else None)
        try:
            gpu_handle.set_kernel_timing(True)
            dw = mluop_hip.indice_conv_backward_filter(gpu_handle, feats_t, dy_t, pairs_t, num_host, c["ks"], sub_m)
            torch.cuda.synchronize()
            names = [k for k, _ in gpu_handle.kernel_timings()]
            gpu_handle.set_kernel_timing(False)
        finally:
            gpu_handle.set_kernel_choice("filter_stores", None)
        assert names[0] == ("backwardFilterMfma" if stores else "backwardFilterMfmaTr")
        got[stores] = dw
    ref = oracle.backward_filter(round_to(c["feats"], dtype_name), round_to(c["dy"], dtype_name), c["pairs"],
                                 c["num"], fast=True)
    check_close(from_torch(got[False]).reshape(ref.shape), ref, dtype_name, "backward_filter")
    assert torch.equal(got[False], got[True])


def test_backward_filter_short_steps_on_long_slices(gpu_handle):
    """Below 128 x 128 channels, slices of 2048 pairs and more are multiplied in steps of 32 pairs
    (another instance of the transposing-read kernel).  3.4 million pairs of a nearly full grid: bit
    for bit against the storing kernel, and a sample of offsets against a float64 product on the host."""
    import torch
    import mluop_hip
    from spconv_cases import random_voxels, to_torch
    rng = np.random.default_rng(61)
    space, ks, ci, co = (32, 64, 64), (3, 3, 3), 64, 32
    idx = random_voxels(rng, 1, space, 125000, shuffle=False)
    pairs, _, num, n_out = mluop_hip.get_indice_pairs(gpu_handle, torch.from_numpy(idx).cuda(), 1, space, ks, space,
                                                      [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    num_host = [int(v) for v in num.cpu()]
    assert sum(num_host) >= 1024 * 2048
    feats = torch.from_numpy(rng.standard_normal((idx.shape[0], ci)).astype(np.float32)).cuda().half()
    dy = torch.from_numpy((rng.standard_normal((n_out, co)) * 0.1).astype(np.float32)).cuda().half()
    got = {}
    for stores in (False, True):
        gpu_handle.set_kernel_choice("filter_stores", True if stores else None)
        try:
            got[stores] = mluop_hip.indice_conv_backward_filter(gpu_handle, feats, dy, pairs, num_host, ks, True)
            torch.cuda.synchronize()
        finally:
            gpu_handle.set_kernel_choice("filter_stores", None)
    assert torch.equal(got[False], got[True])
    dw = got[False].float().reshape(27, ci, co)
    for k in (0, 13, 26):
        n = num_host[k]
        x_k = feats[pairs[k, 0, :n].long()].double()
        dy_k = dy[pairs[k, 1, :n].long()].double()
        ref = x_k.t() @ dy_k
        err = (dw[k].double() - ref).abs().sum() / ref.abs().sum()
        assert float(err) <= 3e-3, (k, float(err))


@pytest.mark.parametrize("layout_name", ["NDHWC", "NCDHW", "ARRAY"])
@pytest.mark.parametrize("dtype_name", ["float32", "float16"])
def test_forward_filter_layouts(gpu_handle, layout_name, dtype_name):
    import torch
    import mluop_hip
    c = conv_case(13, 1, (8, 8, 8), 300, (3, 3, 3), 32, 64, True)
    feats_r = round_to(c["feats"], dtype_name)
    w_r = round_to(c["w"], dtype_name)  # [kd,kh,kw,ci,co]
    if layout_name == "NDHWC":
        w_l, code = np.transpose(w_r, (4, 0, 1, 2, 3)), mluop_hip.LAYOUT_NDHWC
    elif layout_name == "NCDHW":
        w_l, code = np.transpose(w_r, (4, 3, 0, 1, 2)), mluop_hip.LAYOUT_NCDHW
    else:
        w_l, code = w_r, mluop_hip.LAYOUT_ARRAY
    w_l = np.ascontiguousarray(w_l)
    # the oracle's own layout transpose must land on the [K, Ci, Co] tensor
    w_k = oracle.filters_to_kcico(w_l, code, c["K"], c["ci"], c["co"])
    assert np.array_equal(w_k, w_r.reshape(c["K"], c["ci"], c["co"]))
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    out = mluop_hip.indice_conv_forward(gpu_handle, to_torch(feats_r, dtype_name, "cuda"),
                                        to_torch(w_l, dtype_name, "cuda"), code, pairs_t, num_host, c["n_out"], True)
    dx = mluop_hip.indice_conv_backward_data(gpu_handle, to_torch(round_to(c["dy"], dtype_name), dtype_name, "cuda"),
                                             to_torch(w_l, dtype_name, "cuda"), code, pairs_t, num_host, True, c["ci"])
    torch.cuda.synchronize()
    check_close(from_torch(out), oracle.forward(feats_r, w_k, c["pairs"], c["num"], c["n_out"]), dtype_name,
                "forward " + layout_name)
    check_close(from_torch(dx), oracle.backward_data(round_to(c["dy"], dtype_name), w_k, c["pairs"], c["num"]),
                dtype_name, "backward_data " + layout_name)


def test_reference_case0_shape_backward_data(gpu_handle):
    """Shapes of the reference's only in-tree case (zoo/indice_convolution_backward_data/test_case/
    case_0.prototxt): L=10, 3x3 HWCN filter, Ci=210... here Ci=21, Co=10 4-D filter, identity pairs."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(3)
    L, K, ci, co = 10, 9, 21, 10
    pairs = np.full((K, 2, L), -1, dtype=np.int32)
    for k in range(K):
        pairs[k, 0, :] = np.arange(L)
        pairs[k, 1, :] = np.arange(L)
    num = [L] * K
    dy = rng.standard_normal((L, co)).astype(np.float32)
    w = rng.standard_normal((3, 3, ci, co)).astype(np.float32)
    handle = gpu_handle
    lib = mluop_hip.lib()
    import ctypes
    d_dy = mluop_hip.TensorDescriptor(mluop_hip.LAYOUT_ARRAY, mluop_hip.DTYPE_FLOAT, [L, co])
    d_w = mluop_hip.TensorDescriptor(mluop_hip.LAYOUT_HWCN, mluop_hip.DTYPE_FLOAT, [3, 3, ci, co])
    d_p = mluop_hip.TensorDescriptor(mluop_hip.LAYOUT_ARRAY, mluop_hip.DTYPE_INT32, [K, 2, L])
    d_dx = mluop_hip.TensorDescriptor(mluop_hip.LAYOUT_ARRAY, mluop_hip.DTYPE_FLOAT, [L, ci])
    counts = (ctypes.c_int64 * K)(*num)
    size = ctypes.c_size_t(0)
    mluop_hip.check(lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(
        handle.ptr, d_dy.ptr, d_w.ptr, d_p.ptr, d_dx.ptr, counts, 0, ctypes.byref(size)))
    ws = torch.empty(max(size.value, 1), dtype=torch.uint8, device="cuda")
    t_dy, t_w, t_p = torch.from_numpy(dy).cuda(), torch.from_numpy(w).cuda(), torch.from_numpy(pairs).cuda()
    t_dx = torch.empty((L, ci), dtype=torch.float32, device="cuda")
    mluop_hip.check(lib.mluOpIndiceConvolutionBackwardData(
        handle.ptr, d_dy.ptr, t_dy.data_ptr(), d_w.ptr, t_w.data_ptr(), d_p.ptr, t_p.data_ptr(), counts, 0, 0,
        ws.data_ptr(), size.value, d_dx.ptr, t_dx.data_ptr()))
    torch.cuda.synchronize()
    ref = oracle.backward_data(dy, w.reshape(K, ci, co), pairs, num)
    check_close(t_dx.cpu().numpy(), ref, "float32", "case_0 shape")


def test_config1_forward_full_size(gpu_handle):
    """BASELINE config 1: 20 000 uniform voxels, Ci=Co=16 fp32, subm 3x3x3, rulebook built on the GPU."""
    import torch
    import mluop_hip
    idx = mluop_hip.datagen.uniform_voxels((1, 40, 400, 352), 20000, seed=1)
    rng = np.random.default_rng(1)
    feats = rng.standard_normal((20000, 16)).astype(np.float32)
    w = mluop_hip.datagen.kaiming_uniform_filters((3, 3, 3), 16, 16, seed=1)
    t_idx = torch.from_numpy(idx).cuda()
    pairs, out_idx, num, n_out = mluop_hip.get_indice_pairs(gpu_handle, t_idx, 1, (40, 400, 352), (3, 3, 3),
                                                           (40, 400, 352), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    num_host = num.cpu().tolist()
    out = mluop_hip.indice_conv_forward(gpu_handle, torch.from_numpy(feats).cuda(), torch.from_numpy(w).cuda(),
                                        mluop_hip.LAYOUT_ARRAY, pairs, num_host, n_out, True)
    torch.cuda.synchronize()
    ref = oracle.forward(feats, w.reshape(27, 16, 16), pairs.cpu().numpy(), num_host, n_out)
    check_close(out.cpu().numpy(), ref, "float32", "config1 forward")


def test_config4_all_ops_full_size(gpu_handle):
    """BASELINE config 4 (headline): 120 000 clustered voxels, Ci=Co=64 fp16, subm 3x3x3: forward,
    backward data and backward filter (dY ~ N(0, 1e-2), filter gradient accumulated in fp32)."""
    import torch
    import mluop_hip
    L = 120000
    idx = mluop_hip.datagen.clustered_voxels((1, 41, 1600, 1408), L, seed=4)
    rng = np.random.default_rng(4)
    feats = round_to(rng.standard_normal((L, 64)).astype(np.float32), "float16")
    w = round_to(mluop_hip.datagen.kaiming_uniform_filters((3, 3, 3), 64, 64, seed=4), "float16")
    dy = round_to((rng.standard_normal((L, 64)) * 1e-1).astype(np.float32), "float16")
    t_idx = torch.from_numpy(idx).cuda()
    pairs, out_idx, num, n_out = mluop_hip.get_indice_pairs(gpu_handle, t_idx, 1, (41, 1600, 1408), (3, 3, 3),
                                                           (41, 1600, 1408), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    num_host = num.cpu().tolist()
    pairs_np = pairs.cpu().numpy()
    c = dict(pairs=pairs_np, num=np.array(num_host), n_out=n_out, feats=feats, w=w, dy=dy, K=27, ks=(3, 3, 3),
             ci=64, co=64, sub_m=True)
    print("config4 ops", flush=True)
    run_all_ops(gpu_handle, c, "float16")


# --- pairs of one offset that share a result row -------------------------------------------------
# Repeated input coordinates make mluOpGetIndicePairs list several inputs for one (offset, output
# row); made-up pair tensors (test case files) can repeat anything.  The reference adds every pair.

COLLISION_SHAPES = [
    # (space, L, duplicated rows, ks, ci, co, sub_m, stride, force dense kernel)
    ((8, 9, 10), 400, 60, (3, 3, 3), 64, 64, True, (1, 1, 1), False),       # pair-list MFMA kernel
    ((8, 8, 8), 300, 80, (3, 3, 3), 128, 128, True, (1, 1, 1), True),       # register-accumulating kernel
    ((8, 10, 10), 500, 100, (3, 3, 3), 32, 16, False, (2, 2, 2), False),    # regular, strided
    ((6, 6, 6), 100, 40, (3, 3, 3), 21, 10, True, (1, 1, 1), False),        # generic FMA kernel
    ((10, 10, 10), 300, 50, (5, 5, 7), 32, 32, True, (1, 1, 1), False),     # K = 175
    ((32, 8, 35), 5000, 3000, (3, 3, 5), 128, 32, True, (1, 1, 1), False),  # more lost pairs than the repair pool has rows
]


@pytest.mark.parametrize("shape", COLLISION_SHAPES)
@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_repeated_coordinates_are_all_added(gpu_handle, shape, dtype_name):
    space, L, dup, ks, ci, co, sub_m, stride, dense = shape
    print("collision case", shape, dtype_name, flush=True)
    rng = np.random.default_rng(41)
    idx = random_voxels(rng, 2, space, L, duplicates=dup)
    pad = [k // 2 for k in ks]
    pairs, num, n_out = build_rulebook(idx, 2, space, ks, pad, list(stride), [1, 1, 1], sub_m)
    K = int(np.prod(ks))
    # at least one offset lists one output row twice: the case this test is about
    assert any(len(np.unique(pairs[k, 1, :num[k]])) < num[k] for k in range(K))
    b = 1.0 / np.sqrt(K * ci)
    c = dict(idx=idx, pairs=pairs, num=num, n_out=n_out, K=K, ks=ks, ci=ci, co=co, sub_m=sub_m,
             feats=rng.standard_normal((idx.shape[0], ci)).astype(np.float32),
             w=rng.uniform(-b, b, size=tuple(ks) + (ci, co)).astype(np.float32),
             dy=(rng.standard_normal((n_out, co)) * 1e-1).astype(np.float32))
    if dense:
        gpu_handle.set_kernel_choice("dense_tiles", True)
    try:
        run_all_ops(gpu_handle, c, dtype_name)
    finally:
        gpu_handle.set_kernel_choice("dense_tiles", None)


@pytest.mark.parametrize("case", [
    # (space, L, duplicated rows, ks, ci, co, sub_m, stride, kernel choice switched on)
    ((16, 30, 30), 9000, 0, (3, 3, 3), 64, 64, True, (1, 1, 1), None),
    ((16, 30, 30), 9000, 700, (3, 3, 3), 64, 64, True, (1, 1, 1), None),
    ((16, 24, 24), 6000, 500, (3, 3, 3), 128, 128, True, (1, 1, 1), "dense_tiles"),
    ((16, 48, 48), 9000, 400, (3, 3, 3), 32, 16, False, (2, 2, 2), None),
    ((12, 20, 20), 4500, 300, (3, 3, 3), 21, 10, True, (1, 1, 1), None),          # generic FMA kernel
    ((12, 20, 20), 4500, 300, (5, 5, 7), 32, 32, True, (1, 1, 1), None),          # K = 175
])
@pytest.mark.parametrize("dtype_name", ["float16", "float32"])
def test_row_maps_built_a_chunk_of_rows_at_a_time(gpu_handle, case, dtype_name):
    """The library's own row map covers at most 64 MiB worth of result rows; more rows are done
    chunk after chunk (fill, scatter, gather, repair per chunk).  With chunks of 2048 rows switched
    on, inputs of a few thousand rows take that way: graded against the oracle, and equal bit for
    bit to the one-chunk results where no pairs collide."""
    import torch
    import mluop_hip
    space, L, dup, ks, ci, co, sub_m, stride, choice = case
    rng = np.random.default_rng(45)
    idx = random_voxels(rng, 2, space, L, duplicates=dup)
    pad = [k // 2 for k in ks]
    pairs, num, n_out = build_rulebook(idx, 2, space, ks, pad, list(stride), [1, 1, 1], sub_m)
    K = int(np.prod(ks))
    assert n_out > 4096 and idx.shape[0] > 4096      # several chunks in both directions
    b = 1.0 / np.sqrt(K * ci)
    c = dict(idx=idx, pairs=pairs, num=num, n_out=n_out, K=K, ks=ks, ci=ci, co=co, sub_m=sub_m,
             feats=rng.standard_normal((idx.shape[0], ci)).astype(np.float32),
             w=rng.uniform(-b, b, size=tuple(ks) + (ci, co)).astype(np.float32),
             dy=(rng.standard_normal((n_out, co)) * 1e-1).astype(np.float32))
    t_pairs = torch.from_numpy(pairs).cuda()
    num_host = [int(v) for v in num]
    t_f, t_w = (to_torch(round_to(c[k], dtype_name), dtype_name, "cuda") for k in ("feats", "w"))
    if choice:
        gpu_handle.set_kernel_choice(choice, True)
    try:
        whole = mluop_hip.indice_conv_forward(gpu_handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, t_pairs, num_host, n_out,
                                              sub_m)
        gpu_handle.set_kernel_choice("small_map_chunks", True)
        run_all_ops(gpu_handle, c, dtype_name, check=("fwd", "bwd_data"))
        chunked = mluop_hip.indice_conv_forward(gpu_handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, t_pairs, num_host,
                                                n_out, sub_m)
        torch.cuda.synchronize()
    finally:
        gpu_handle.set_kernel_choice("small_map_chunks", None)
        if choice:
            gpu_handle.set_kernel_choice(choice, None)
    if dup == 0:
        as_int = torch.int16 if dtype_name != "float32" else torch.int32
        assert torch.equal(whole.view(as_int), chunked.view(as_int))


def test_a_hundred_thousand_repeated_coordinates_finish_in_bounded_time(gpu_handle):
    """300 000 rows of which 100 000 repeat the coordinates of another row (a cloud that was
    never made unique): about a million pairs lose their map slot.  Their repair is spread over
    windows of result rows, each with a workgroup of its own, and must not take the queue for
    longer than a second; forward and backward data are graded against the oracle."""
    import time
    import torch
    import mluop_hip
    rng = np.random.default_rng(43)
    space, ks, ci, co = (24, 96, 96), (3, 3, 3), 32, 32
    idx = random_voxels(rng, 1, space, 200000, duplicates=100000)
    pairs, num, n_out = build_rulebook(idx, 1, space, ks, [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    lost = sum(int(num[k]) - len(np.unique(pairs[k, 1, :num[k]])) for k in range(27))
    print("pairs", int(num.sum()), "of which lose their slot in forward:", lost, flush=True)
    assert lost > 500000
    feats = round_to(rng.standard_normal((idx.shape[0], ci)).astype(np.float32), "float16")
    w = round_to(rng.uniform(-0.05, 0.05, size=ks + (ci, co)).astype(np.float32), "float16")
    dy = round_to((rng.standard_normal((n_out, co)) * 0.1).astype(np.float32), "float16")
    t_pairs = torch.from_numpy(pairs).cuda()
    num_host = [int(v) for v in num]
    t_f, t_w, t_dy = (to_torch(a, "float16", "cuda") for a in (feats, w, dy))
    w_k = w.reshape(27, ci, co)
    for _ in range(2):   # the second call is the timed one
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = mluop_hip.indice_conv_forward(gpu_handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, t_pairs, num_host, n_out,
                                            True)
        torch.cuda.synchronize()
        fwd_s = time.perf_counter() - t0
    print("forward with repairs: %.1f ms" % (fwd_s * 1e3), flush=True)
    assert fwd_s < 1.0
    check_close(from_torch(out), oracle.forward(feats, w_k, pairs, num, n_out), "float16", "forward")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dx = mluop_hip.indice_conv_backward_data(gpu_handle, t_dy, t_w, mluop_hip.LAYOUT_ARRAY, t_pairs, num_host, True,
                                             ci)
    torch.cuda.synchronize()
    assert time.perf_counter() - t0 < 1.0
    check_close(from_torch(dx), oracle.backward_data(dy, w_k, pairs, num), "float16", "backward_data")


def test_pairs_outside_their_tensors_do_not_start_the_repair_scan(gpu_handle):
    """Pairs that name a row outside the tensors are skipped (the reference would read out of
    bounds); the map can never hold them, and the check for lost pairs must not take them for
    collisions: the repair kernel returns as fast as it does for a clean rulebook."""
    import torch
    import mluop_hip
    rng = np.random.default_rng(44)
    space, ks, ci, co, L = (16, 40, 40), (3, 3, 3), 32, 32, 20000
    idx = random_voxels(rng, 1, space, L)
    pairs, num, n_out = build_rulebook(idx, 1, space, ks, [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    broken = pairs.copy()
    for k in range(27):
        n = int(num[k])
        where = rng.choice(n, size=min(n, 50), replace=False)
        broken[k, 1, where[:25]] = n_out + 5          # result row outside
        broken[k, 0, where[25:]] = -7                 # gathered row outside
    feats = round_to(rng.standard_normal((L, ci)).astype(np.float32), "float16")
    w = round_to(rng.uniform(-0.05, 0.05, size=ks + (ci, co)).astype(np.float32), "float16")
    t_f, t_w = to_torch(feats, "float16", "cuda"), to_torch(w, "float16", "cuda")
    num_host = [int(v) for v in num]
    times = {}
    for name, tensor in (("clean", pairs), ("broken", broken)):
        t_pairs = torch.from_numpy(tensor).cuda()
        mluop_hip.indice_conv_forward(gpu_handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, t_pairs, num_host, n_out, True)
        gpu_handle.set_kernel_timing(True)
        try:
            out = mluop_hip.indice_conv_forward(gpu_handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, t_pairs, num_host,
                                                n_out, True)
            times[name] = dict(gpu_handle.kernel_timings())["repairLostPairs"]
        finally:
            gpu_handle.set_kernel_timing(False)
    valid = broken.copy()                              # the oracle's view: those pairs do not exist
    keep_num = num.copy()
    for k in range(27):
        n = int(num[k])
        ok = (broken[k, 1, :n] < n_out) & (broken[k, 0, :n] >= 0)
        valid[k, :, :n] = -1
        valid[k, :, :int(ok.sum())] = broken[k][:, :n][:, ok]
        keep_num[k] = int(ok.sum())
    check_close(from_torch(out), oracle.forward(feats, w.reshape(27, ci, co), valid, keep_num, n_out), "float16",
                "forward")
    print("repairLostPairs ms:", times, flush=True)
    assert times["broken"] < 5 * times["clean"] + 0.02


@pytest.mark.parametrize("ci,co", [(64, 64), (13, 70)])
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_made_up_pairs_with_repeats_everywhere(gpu_handle, ci, co, dtype_name):
    """Uniformly random pair tensors, as a case file's random_data gives them: the same output row
    many times per offset, the same input row many times per offset, identical pairs twice, and
    more touched rows than the repair pool holds at once."""
    rng = np.random.default_rng(42)
    K, L, n_out = 9, 6000, 6200          # output_grad needs at least as many rows as an offset has pairs
    pairs = np.full((K, 2, L), -1, dtype=np.int32)
    num = rng.integers(L // 2, L + 1, size=K)
    for k in range(K):
        pairs[k, 0, :num[k]] = rng.integers(0, L, size=num[k])
        pairs[k, 1, :num[k]] = rng.integers(0, n_out, size=num[k])
    pairs[0, :, 1] = pairs[0, :, 0]                       # an identical pair, twice
    c = dict(pairs=pairs, num=num, n_out=n_out, K=K, ks=(1, 3, 3), ci=ci, co=co, sub_m=False,
             feats=rng.standard_normal((L, ci)).astype(np.float32),
             w=(rng.standard_normal((1, 3, 3, ci, co)) / np.sqrt(K * ci)).astype(np.float32),
             dy=(rng.standard_normal((n_out, co)) * 1e-1).astype(np.float32))
    run_all_ops(gpu_handle, c, dtype_name)


def test_distinct_pairs_promise_skips_the_check(gpu_handle):
    """With the promise the check kernel is not launched (one kernel fewer per call) and a rulebook
    with distinct pairs gives the same bits; the default handle launches it."""
    import torch
    import mluop_hip
    c = conv_case(43, 2, (8, 9, 10), 400, (3, 3, 3), 64, 64, True)
    feats_t = to_torch(round_to(c["feats"], "float16"), "float16", "cuda")
    w_t = to_torch(round_to(c["w"], "float16"), "float16", "cuda")
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]

    def forward_and_kernels():
        gpu_handle.set_kernel_timing(True)
        out = mluop_hip.indice_conv_forward(gpu_handle, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host,
                                            c["n_out"], True)
        names = [name for name, _ in gpu_handle.kernel_timings()]
        gpu_handle.set_kernel_timing(False)
        return out, names

    checked, names = forward_and_kernels()
    assert names[-1] == "repairLostPairs"
    gpu_handle.promise_distinct_pairs(True)
    try:
        promised, names_promised = forward_and_kernels()
    finally:
        gpu_handle.promise_distinct_pairs(False)
    assert "repairLostPairs" not in names_promised and len(names_promised) == len(names) - 1
    assert torch.equal(checked, promised)


def _offset_view(torch, t, elements=1):
    """The same values at an address `elements` past a fresh allocation: not 16-byte aligned."""
    flat = torch.empty(t.numel() + 8, dtype=t.dtype, device=t.device)
    view = flat[elements:elements + t.numel()].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 16 != 0
    return view


@pytest.mark.parametrize("dtype_name", ["float32", "float16"])
def test_tensors_that_are_not_16_byte_aligned(gpu_handle, dtype_name):
    """Feature, gradient, filter and pair tensors at odd addresses: the kernels that move rows with
    16-byte accesses step aside for the generic ones, and the numbers stay the same."""
    import torch
    import mluop_hip
    c = conv_case(44, 2, (8, 9, 10), 400, (3, 3, 3), 64, 64, True)
    feats_r, w_r, dy_r = (round_to(c[k], dtype_name) for k in ("feats", "w", "dy"))
    w_k = w_r.reshape(c["K"], c["ci"], c["co"])
    feats_t = _offset_view(torch, to_torch(feats_r, dtype_name, "cuda"))
    w_t = _offset_view(torch, to_torch(w_r, dtype_name, "cuda"))
    dy_t = _offset_view(torch, to_torch(dy_r, dtype_name, "cuda"))
    pairs_t = _offset_view(torch, torch.from_numpy(c["pairs"]).cuda())
    num_host = [int(v) for v in c["num"]]
    out = mluop_hip.indice_conv_forward(gpu_handle, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host,
                                        c["n_out"], True)
    dx = mluop_hip.indice_conv_backward_data(gpu_handle, dy_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host, True,
                                             c["ci"])
    dw = mluop_hip.indice_conv_backward_filter(gpu_handle, feats_t, dy_t, pairs_t, num_host, c["ks"], True)
    torch.cuda.synchronize()
    check_close(from_torch(out), oracle.forward(feats_r, w_k, c["pairs"], c["num"], c["n_out"]), dtype_name, "forward")
    check_close(from_torch(dx), oracle.backward_data(dy_r, w_k, c["pairs"], c["num"]), dtype_name, "backward_data")
    ref = oracle.backward_filter(feats_r, dy_r, c["pairs"], c["num"], fast=True)
    check_close(from_torch(dw).reshape(ref.shape), ref, dtype_name, "backward_filter")


@pytest.mark.parametrize("case", [
    # (space, L, ks, ci, co)
    ((41, 400, 352), 40000, (3, 3, 3), 64, 64),   # centre offset: hundreds of slices, the others a few
    ((20, 40, 40), 20000, (3, 3, 3), 32, 16),     # offsets between 17 and 128 slices next to thin ones
    ((12, 12, 12), 1500, (5, 5, 5), 128, 128),    # 125 offsets of one or two slices: the shape the flat grid is for
    ((8, 8, 8), 300, (3, 3, 3), 16, 16),          # one 256-element chunk per offset
])
@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_flat_slice_sum_gives_the_bits_of_the_grid_one(gpu_handle, case, dtype_name):
    """Backward filter adds an offset's partial tiles with one of two kernels, chosen by the size of
    the grid; both add the slices in the same order and tree, so the filter gradient must not
    depend on the choice.  Also graded against the oracle."""
    import torch
    import mluop_hip
    space, L, ks, ci, co = case
    print("slice sum case", case, dtype_name, flush=True)
    c = conv_case(23, 1, space, L, ks, ci, co, True)
    feats_t = to_torch(round_to(c["feats"], dtype_name), dtype_name, "cuda")
    dy_t = to_torch(round_to(c["dy"], dtype_name), dtype_name, "cuda")
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    got = {}
    try:
        for mode in ("1", "0"):
            gpu_handle.set_kernel_choice("flat_slice_sum", mode == "1")
            if mode == "1":
                run_all_ops(gpu_handle, c, dtype_name, check=("bwd_filter",))
            dw = mluop_hip.indice_conv_backward_filter(gpu_handle, feats_t, dy_t, pairs_t, num_host, c["ks"], True)
            torch.cuda.synchronize()
            got[mode] = dw.view(torch.int16 if dtype_name != "float32" else torch.int32).cpu()
    finally:
        gpu_handle.set_kernel_choice("flat_slice_sum", None)
    assert torch.equal(got["1"], got["0"])


@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[3], SHAPES[4], SHAPES[5],
                                   (1, (30, 30, 30), 40, (3, 3, 3), 32, 32, True, (1, 1, 1))])  # offsets without pairs
@pytest.mark.parametrize("dtype_name", ["float32", "float16"])
def test_flat_row_map_scatter_gives_the_same_results(gpu_handle, shape, dtype_name):
    """The row map of a gather convolution is written by one of two kernels, chosen by the size of
    the grid; with distinct coordinates every map slot has one writer, so forward and backward
    data must not depend on the choice.  Also graded against the oracle."""
    import torch
    import mluop_hip
    batch, space, L, ks, ci, co, sub_m, stride = shape
    print("flat scatter case", shape, dtype_name, flush=True)
    c = conv_case(31, batch, space, L, ks, ci, co, sub_m, stride)
    feats_t = to_torch(round_to(c["feats"], dtype_name), dtype_name, "cuda")
    w_t = to_torch(round_to(c["w"], dtype_name), dtype_name, "cuda")
    dy_t = to_torch(round_to(c["dy"], dtype_name), dtype_name, "cuda")
    pairs_t = torch.from_numpy(c["pairs"]).cuda()
    num_host = [int(v) for v in c["num"]]
    got = {}
    try:
        for mode in ("1", "0"):
            gpu_handle.set_kernel_choice("flat_scatter", mode == "1")
            if mode == "1":
                run_all_ops(gpu_handle, c, dtype_name, check=("fwd", "bwd_data"))
            out = mluop_hip.indice_conv_forward(gpu_handle, feats_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t, num_host,
                                                c["n_out"], c["sub_m"])
            dx = mluop_hip.indice_conv_backward_data(gpu_handle, dy_t, w_t, mluop_hip.LAYOUT_ARRAY, pairs_t,
                                                     num_host, c["sub_m"], c["ci"])
            torch.cuda.synchronize()
            as_int = torch.int16 if dtype_name != "float32" else torch.int32
            got[mode] = (out.view(as_int).cpu(), dx.view(as_int).cpu())
    finally:
        gpu_handle.set_kernel_choice("flat_scatter", None)
    assert torch.equal(got["1"][0], got["0"][0]) and torch.equal(got["1"][1], got["0"][1])
