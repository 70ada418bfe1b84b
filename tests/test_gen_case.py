"""The case dump inside the library (MLUOP_GEN_CASE, reference core/gen_case.cpp): every operator
call that passed its checks leaves a prototxt file the case-file module reads back.  The
variables are read once per process, so each case runs in a process of its own."""
import glob
import os
import subprocess
import sys
import textwrap

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

HOST_ONLY = textwrap.dedent("""
    import ctypes, sys
    sys.path.insert(0, %r)
    import mluop_hip as m
    h = m.Handle()
    lib = m.lib()
    K, L, ci, co = 27, 50, 16, 32
    conv = m.SparseConvDescriptor(1, [1, 1, 1], [1, 1, 1], [1, 1, 1], [8, 8, 8], [3, 3, 3], [8, 8, 8], True)
    d_idx = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [L, 4])
    d_pairs = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [K, 2, L])
    d_out = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [L, 4])
    d_num = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [K])
    size = ctypes.c_size_t(0)
    m.check(lib.mluOpGetIndicePairsWorkspaceSize(h.ptr, conv.ptr, d_idx.ptr, d_pairs.ptr, d_out.ptr, d_num.ptr,
                                                 ctypes.byref(size)))
    fake = 4096
    st = lib.mluOpGetIndicePairs(h.ptr, conv.ptr, d_idx.ptr, fake, fake, size.value, d_pairs.ptr, fake, d_out.ptr,
                                 fake, d_num.ptr, fake)
    assert st == m.STATUS_EXECUTION_FAILED, st      # checks passed; a handle without a device stops there
    d_f = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_HALF, [L, ci])
    d_w = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_HALF, [3, 3, 3, ci, co])
    d_y = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_HALF, [L, co])
    counts = (ctypes.c_int64 * K)(*range(K))
    m.check(lib.mluOpGetIndiceConvolutionForwardWorkspaceSize(h.ptr, d_f.ptr, d_w.ptr, d_pairs.ptr, d_y.ptr, counts,
                                                              L, 0, 1, ctypes.byref(size)))
    st = lib.mluOpIndiceConvolutionForward(h.ptr, d_f.ptr, fake, d_w.ptr, fake, d_pairs.ptr, fake, counts, L, 0, 1,
                                           fake, size.value, d_y.ptr, fake)
    assert st == m.STATUS_EXECUTION_FAILED, st
    # a call that fails its checks leaves no file
    st = lib.mluOpIndiceConvolutionForward(h.ptr, d_f.ptr, fake, d_w.ptr, fake, d_pairs.ptr, fake, counts, L + 1, 0,
                                           1, fake, size.value, d_y.ptr, fake)
    assert st == m.STATUS_BAD_PARAM, st
""")


def run(code, env):
    full = dict(os.environ)
    full.update(env)
    return subprocess.run([sys.executable, "-c", code], env=full, capture_output=True, text=True, timeout=300)


def test_parameters_and_shapes_are_dumped_without_a_device(tmp_path):
    from mluop_hip import casefile
    r = run(HOST_ONLY % os.path.join(ROOT, "mlu-ops_amd", "python"),
            {"MLUOP_GEN_CASE": "1", "MLUOP_GEN_CASE_DIR": str(tmp_path), "MLUOP_HOST_ONLY_HANDLE": "1"})
    assert r.returncode == 0, r.stderr
    files = sorted(glob.glob(str(tmp_path / "*" / "*.prototxt")))
    assert [os.path.basename(os.path.dirname(f)) for f in files] == ["get_indice_pairs",
                                                                    "indice_convolution_forward"]
    node, _ = casefile.load(files[0])
    assert node.get("op_name") == "get_indice_pairs"
    p = node.get("get_indice_pairs_param")
    assert p.get("batch") == 1 and p.get("sub_m") == 1 and p.all("filter_space") == [3, 3, 3]
    assert [t.get("id") for t in node.all("output")] == ["out_indices", "indice_pairs", "indice_num"]
    assert node.all("output")[1].get("shape").all("dims") == [27, 2, 50]
    node, _ = casefile.load(files[1])
    p = node.get("indice_convolution_forward_param")
    assert p.all("indice_num") == list(range(27)) and p.get("num_active_out") == 50
    assert [t.get("id") for t in node.all("input")] == ["features", "filters", "indice_pairs"]
    assert str(node.all("input")[0].get("dtype")) == "DTYPE_HALF"
    assert not node.all("input")[0].has("value_h")        # mode 1: no values


def test_mode_off_writes_nothing_and_mode_3_prints(tmp_path):
    code = HOST_ONLY % os.path.join(ROOT, "mlu-ops_amd", "python")
    r = run(code, {"MLUOP_GEN_CASE": "0", "MLUOP_GEN_CASE_DIR": str(tmp_path), "MLUOP_HOST_ONLY_HANDLE": "1"})
    assert r.returncode == 0, r.stderr
    assert glob.glob(str(tmp_path / "*")) == []
    r = run(code, {"MLUOP_GEN_CASE": "3", "MLUOP_GEN_CASE_DIR": str(tmp_path), "MLUOP_HOST_ONLY_HANDLE": "1"})
    assert r.returncode == 0, r.stderr
    assert "[MLUOP_GEN_CASE] get_indice_pairs: indices[50,4]" in r.stderr
    assert glob.glob(str(tmp_path / "*")) == []


WITH_DATA = textwrap.dedent("""
    import sys
    sys.path.insert(0, %r)
    import numpy as np, torch
    import mluop_hip as m
    torch.cuda.set_device(0)
    h = m.make_handle_on_current_stream()
    rng = np.random.default_rng(61)
    lin = rng.choice(2 * 6 * 9 * 9, size=300, replace=False)
    idx = np.stack([lin // 486, lin %% 486 // 81, lin %% 81 // 9, lin %% 9], axis=1).astype(np.int32)
    pairs, out_idx, num, n_out = m.get_indice_pairs(h, torch.from_numpy(idx).cuda(), 2, (6, 9, 9), (3, 3, 3), [6, 9, 9],
                                                    [1, 1, 1], [1, 1, 1], [1, 1, 1], True)
    num_host = num.cpu().tolist()
    x = torch.randn(300, 16, device="cuda").half()
    w = (torch.randn(3, 3, 3, 16, 32, device="cuda") * 0.1).half()
    dy = torch.randn(300, 32, device="cuda").half()
    m.indice_conv_forward(h, x, w, m.LAYOUT_ARRAY, pairs, num_host, n_out, True)
    m.indice_conv_backward_data(h, dy, w, m.LAYOUT_ARRAY, pairs, num_host, True, 16)
    m.indice_conv_backward_filter(h, x, dy, pairs, num_host, (3, 3, 3), True)
    pts = torch.rand(500, 4, device="cuda") * torch.tensor([4.0, 4.0, 2.0, 1.0], device="cuda")
    m.voxelization(h, pts, torch.tensor([0.5, 0.5, 0.5], device="cuda"),
                   torch.tensor([0.0, 0.0, 0.0, 4.0, 4.0, 2.0], device="cuda"), 6, 100)
    feats = torch.randn(400, 5, device="cuda")
    coors = torch.randint(0, 6, (400, 3), device="cuda", dtype=torch.int32)
    vf, vc, p2v, cnt, vn = m.dynamic_point_to_voxel_forward(h, feats, coors, "max")
    m.dynamic_point_to_voxel_backward(h, torch.randn_like(vf), feats, vf, p2v, cnt, vn, reduce_type="max")
    torch.cuda.synchronize()
""")


@pytest.mark.gpu
def test_dumped_cases_with_values_replay_through_the_library(tmp_path, gpu_handle):
    from mluop_hip import casefile
    r = run(WITH_DATA % os.path.join(ROOT, "mlu-ops_amd", "python"),
            {"MLUOP_GEN_CASE": "2", "MLUOP_GEN_CASE_DIR": str(tmp_path)})
    assert r.returncode == 0, r.stderr
    files = sorted(glob.glob(str(tmp_path / "*" / "*.prototxt")))
    ops = [os.path.basename(os.path.dirname(f)) for f in files]
    assert ops == ["dynamic_point_to_voxel_backward", "dynamic_point_to_voxel_forward", "get_indice_pairs",
                   "indice_convolution_backward_data", "indice_convolution_backward_filter",
                   "indice_convolution_forward", "voxelization"]
    for f in files:
        node, _ = casefile.load(f)
        first = node.all("input")[0]
        assert first.has("value_i") or first.has("value_h")
        res = casefile.replay(f, gpu_handle)      # inputs from the file, outputs graded against the CPU oracle
        assert res.passed, (f, res.errors)
