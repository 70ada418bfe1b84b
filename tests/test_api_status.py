"""Status-code behaviour of the C ABI, checked without a GPU.

Handles are created with MLUOP_HOST_ONLY_HANDLE=1 in the environment (for the moment of the
call only: GPU tests collected into the same process need real handles), which gives a handle
without a device on any machine; every parameter check and zero-element early return runs before any kernel
would be launched, so the reference's api_gtest expectations can be replayed here:

* tests/golden/api_status_tables.json -- the value-parameterised tables of
  test/mlu_op_gtest/api_gtest/src/gtest/<op>/<op>_general.cpp (extracted as data by
  tests/golden/extract_api_status_tables.py), replayed with the same call sequence as the
  reference fixture (workspace query first, then the operator);
* the one-NULL-argument-at-a-time cases of <op>.cpp and <op>_workspace.cpp, restated below.
Cases that pass all checks reach the launch stage and must then report EXECUTION_FAILED on a
host-only handle (the library has no CPU compute path).
"""
import ctypes
import json
import os
import re

import pytest

os.environ.setdefault("MLUOP_LOG_PRINT", "0")

import mluop_hip as m  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TABLES = json.load(open(os.path.join(ROOT, "tests", "golden", "api_status_tables.json")))

STATUS = {"MLUOP_STATUS_SUCCESS": 0, "MLUOP_STATUS_NOT_INITIALIZED": 1, "MLUOP_STATUS_ALLOC_FAILED": 2,
          "MLUOP_STATUS_BAD_PARAM": 3, "MLUOP_STATUS_INTERNAL_ERROR": 4, "MLUOP_STATUS_ARCH_MISMATCH": 5,
          "MLUOP_STATUS_EXECUTION_FAILED": 6, "MLUOP_STATUS_NOT_SUPPORTED": 7}
LAYOUT = {"MLUOP_LAYOUT_NCHW": 0, "MLUOP_LAYOUT_NHWC": 1, "MLUOP_LAYOUT_HWCN": 2, "MLUOP_LAYOUT_NDHWC": 3,
          "MLUOP_LAYOUT_ARRAY": 4, "MLUOP_LAYOUT_NCDHW": 5, "MLUOP_LAYOUT_TNC": 6, "MLUOP_LAYOUT_NTC": 7,
          "MLUOP_LAYOUT_NC": 8, "MLUOP_LAYOUT_NLC": 9, "MLUOP_LAYOUT_NCL": 10}
DTYPE = {"MLUOP_DTYPE_INVALID": 0, "MLUOP_DTYPE_HALF": 1, "MLUOP_DTYPE_FLOAT": 2, "MLUOP_DTYPE_INT8": 3,
         "MLUOP_DTYPE_INT16": 4, "MLUOP_DTYPE_INT32": 6, "MLUOP_DTYPE_INT64": 9, "MLUOP_DTYPE_DOUBLE": 14,
         "MLUOP_DTYPE_BFLOAT16": 17, "MLUOP_DTYPE_UINT8": 7, "MLUOP_DTYPE_BOOL": 8, "MLUOP_DTYPE_INT31": 5,
         "MLUOP_DTYPE_UINT32": 11, "MLUOP_DTYPE_UINT64": 12, "MLUOP_DTYPE_UINT16": 13,
         "MLUOP_DTYPE_COMPLEX_HALF": 15, "MLUOP_DTYPE_COMPLEX_FLOAT": 16}

FAKE = ctypes.c_void_p(0x1000)  # a non-NULL "device pointer"; never dereferenced on these paths


def host_only_handle():
    """A handle that never launches anything: the made-up pointers below must not reach a kernel."""
    old = os.environ.get("MLUOP_HOST_ONLY_HANDLE")
    os.environ["MLUOP_HOST_ONLY_HANDLE"] = "1"
    try:
        return m.Handle()
    finally:
        if old is None:
            del os.environ["MLUOP_HOST_ONLY_HANDLE"]
        else:
            os.environ["MLUOP_HOST_ONLY_HANDLE"] = old


@pytest.fixture(scope="module")
def handle():
    h = host_only_handle()
    yield h
    h.close()


def make_desc(p):
    d = ctypes.c_void_p()
    assert m.lib().mluOpCreateTensorDescriptor(ctypes.byref(d)) == 0
    dims = (ctypes.c_int * max(len(p["dims"]), 1))(*p["dims"])
    st = m.lib().mluOpSetTensorDescriptor(d, LAYOUT[p["layout"]], DTYPE[p["dtype"]], p["dim_nb"], dims)
    assert st == 0
    if p.get("onchip_dtype"):
        assert m.lib().mluOpSetTensorDescriptorOnchipDataType(d, DTYPE[p["onchip_dtype"]]) == 0
    return d


def free_descs(*ds):
    for d in ds:
        m.lib().mluOpDestroyTensorDescriptor(d)


def i64(vals):
    return (ctypes.c_int64 * max(len(vals), 1))(*vals)


def i32(vals):
    return (ctypes.c_int * max(len(vals), 1))(*vals)


def launch_ok(expected):
    """A table case that expects SUCCESS from a real launch ends at the launch gate here."""
    return (STATUS[expected], STATUS["MLUOP_STATUS_EXECUTION_FAILED"]) if expected == "MLUOP_STATUS_SUCCESS" \
        else (STATUS[expected],)


def cases(op):
    out = []
    for c in TABLES[op]["cases"]:
        if c["device"] != "MLUOP_UNKNOWN_DEVICE":
            continue  # bound to one MLU model in the reference; skipped there on other devices
        out.append(pytest.param(c, id=c["name"]))
    return out


@pytest.mark.parametrize("case", cases("get_indice_pairs"))
def test_get_indice_pairs_table(handle, case):
    lib = m.lib()
    sp, p_idx, p_pairs, p_out, p_num = case["params"]
    dim_nb, batch, pad, stride, dil, in_sp, f_sp, out_sp, sub_m, transpose, inverse = sp
    descs = [make_desc(p) for p in (p_idx, p_pairs, p_out, p_num)]
    sdesc = ctypes.c_void_p()
    assert lib.mluOpCreateSparseConvolutionDescriptor(ctypes.byref(sdesc)) == 0
    try:
        st = lib.mluOpSetSparseConvolutionDescriptor(sdesc, dim_nb, batch, i32(pad), i32(stride), i32(dil),
                                                     i32(in_sp), i32(f_sp), i32(out_sp), sub_m, transpose, inverse)
        if st != 0:
            assert st == STATUS[case["expected"]]
            return
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndicePairsWorkspaceSize(handle.ptr, sdesc, descs[0], descs[1], descs[2], descs[3],
                                                  ctypes.byref(size))
        if st != 0:
            assert st == STATUS[case["expected"]]
            return
        st = lib.mluOpGetIndicePairs(handle.ptr, sdesc, descs[0], FAKE, FAKE, size.value, descs[1], FAKE, descs[2],
                                     FAKE, descs[3], FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)
        lib.mluOpDestroySparseConvolutionDescriptor(sdesc)


@pytest.mark.parametrize("case", cases("indice_convolution_forward"))
def test_indice_convolution_forward_table(handle, case):
    lib = m.lib()
    p_feat, p_filt, p_pairs, p_out, extra = case["params"]
    indice_num, num_act_out, inverse, sub_m = extra
    descs = [make_desc(p) for p in (p_feat, p_filt, p_pairs, p_out)]
    try:
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndiceConvolutionForwardWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2], descs[3],
                                                               i64(indice_num), num_act_out, inverse, sub_m,
                                                               ctypes.byref(size))
        if st != 0:
            assert st == STATUS[case["expected"]]
            return
        st = lib.mluOpIndiceConvolutionForward(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE,
                                               i64(indice_num), num_act_out, inverse, sub_m, FAKE, size.value,
                                               descs[3], FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)


@pytest.mark.parametrize("case", cases("indice_convolution_backward_data"))
def test_indice_convolution_backward_data_table(handle, case):
    lib = m.lib()
    p_dy, p_filt, p_pairs, p_dx, extra = case["params"]
    indice_num, inverse, sub_m = extra
    descs = [make_desc(p) for p in (p_dy, p_filt, p_pairs, p_dx)]
    try:
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2],
                                                                    descs[3], i64(indice_num), inverse,
                                                                    ctypes.byref(size))
        if st != 0:
            assert st == STATUS[case["expected"]]
            return
        st = lib.mluOpIndiceConvolutionBackwardData(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE,
                                                    i64(indice_num), inverse, sub_m, FAKE, size.value, descs[3],
                                                    FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)


@pytest.mark.parametrize("case", cases("indice_convolution_backward_filter"))
def test_indice_convolution_backward_filter_table(handle, case):
    lib = m.lib()
    p_feat, p_dy, p_pairs, p_dw, inverse = case["params"]
    indice_num = [1, 2, 3, 4, 5, 6, 7, 8, 9]  # fixed in the reference fixture
    descs = [make_desc(p) for p in (p_feat, p_dy, p_pairs, p_dw)]
    try:
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2],
                                                                      descs[3], i64(indice_num), inverse, 0,
                                                                      ctypes.byref(size))
        if st != 0:
            assert st == STATUS[case["expected"]]
            return
        st = lib.mluOpIndiceConvolutionBackwardFilter(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE,
                                                      i64(indice_num), inverse, 0, FAKE, size.value, descs[3], FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)


# --- one NULL argument at a time (reference <op>.cpp and <op>_workspace.cpp) ----------------------

T = lambda layout, dtype, dims: {"layout": layout, "dtype": dtype, "dim_nb": len(dims), "dims": dims}


def null_sweep(call, args, nullable, expect=3):
    """Calls `call` with each argument index in `nullable` replaced by NULL in turn."""
    for i in nullable:
        a = list(args)
        a[i] = None
        assert call(*a) == expect, "argument %d NULL" % i


def test_get_indice_pairs_null_arguments(handle):
    """api_gtest/src/gtest/get_indice_pairs/get_indice_pairs.cpp:212-310 and _workspace.cpp:144-208."""
    lib = m.lib()
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", d))
             for d in ([10, 4], [27, 2, 10], [10, 4], [27])]
    sd = m.SparseConvDescriptor(1, [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], [3, 3, 3], [3, 3, 3], 1)
    size = ctypes.c_size_t(0)
    ws_args = [handle.ptr, sd.ptr, descs[0], descs[1], descs[2], descs[3], ctypes.byref(size)]
    null_sweep(lib.mluOpGetIndicePairsWorkspaceSize, ws_args, range(7))
    assert lib.mluOpGetIndicePairsWorkspaceSize(*ws_args) == 0 and size.value > 0
    args = [handle.ptr, sd.ptr, descs[0], FAKE, FAKE, size.value, descs[1], FAKE, descs[2], FAKE, descs[3], FAKE]
    null_sweep(lib.mluOpGetIndicePairs, args, [0, 1, 2, 3, 4, 6, 7, 8, 9, 10, 11])
    assert lib.mluOpGetIndicePairs(*args) == STATUS["MLUOP_STATUS_EXECUTION_FAILED"]  # host-only handle
    free_descs(*descs)


def test_indice_convolution_forward_null_arguments(handle):
    """api_gtest/src/gtest/indice_convolution_forward/indice_convolution_forward.cpp and _workspace.cpp."""
    lib = m.lib()
    descs = [make_desc(p) for p in (T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [10, 21]),
                                    T("MLUOP_LAYOUT_NDHWC", "MLUOP_DTYPE_FLOAT", [5, 3, 3, 3, 21]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", [27, 2, 10]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [10, 5]))]
    num = i64([10] * 27)
    size = ctypes.c_size_t(0)
    ws_args = [handle.ptr, descs[0], descs[1], descs[2], descs[3], num, 10, 0, 0, ctypes.byref(size)]
    null_sweep(lib.mluOpGetIndiceConvolutionForwardWorkspaceSize, ws_args, [0, 1, 2, 3, 4, 5, 9])
    assert lib.mluOpGetIndiceConvolutionForwardWorkspaceSize(*ws_args) == 0
    args = [handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE, num, 10, 0, 0, FAKE, max(size.value, 64),
            descs[3], FAKE]
    null_sweep(lib.mluOpIndiceConvolutionForward, args, [0, 1, 2, 3, 4, 5, 6, 7, 11, 13, 14])
    free_descs(*descs)


def test_indice_convolution_backward_data_null_arguments(handle):
    """api_gtest/src/gtest/indice_convolution_backward_data/indice_convolution_backward_data.cpp:197-296
    (shapes of that fixture: dY [10,10], HWCN filter [3,3,21,10], pairs [9,2,10], dX [10,21])."""
    lib = m.lib()
    descs = [make_desc(p) for p in (T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [10, 10]),
                                    T("MLUOP_LAYOUT_HWCN", "MLUOP_DTYPE_FLOAT", [3, 3, 21, 10]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", [9, 2, 10]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [10, 21]))]
    num = i64([10, 0, 0, 0, 0, 0, 0, 0, 0])
    size = ctypes.c_size_t(0)
    ws_args = [handle.ptr, descs[0], descs[1], descs[2], descs[3], num, 0, ctypes.byref(size)]
    null_sweep(lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize, ws_args, [0, 1, 2, 3, 4, 7])
    assert lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(*ws_args) == 0
    args = [handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE, num, 0, 0, FAKE, max(size.value, 64),
            descs[3], FAKE]
    null_sweep(lib.mluOpIndiceConvolutionBackwardData, args, [0, 1, 2, 3, 4, 5, 6, 10, 12, 13])
    free_descs(*descs)


def test_indice_convolution_backward_filter_null_arguments(handle):
    """api_gtest/src/gtest/indice_convolution_backward_filter/indice_convolution_backward_filter.cpp and
    _workspace.cpp."""
    lib = m.lib()
    descs = [make_desc(p) for p in (T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [10, 21]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [10, 5]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", [27, 2, 10]),
                                    T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_FLOAT", [3, 3, 3, 21, 5]))]
    num = i64([10] * 27)
    size = ctypes.c_size_t(0)
    ws_args = [handle.ptr, descs[0], descs[1], descs[2], descs[3], num, 0, 0, ctypes.byref(size)]
    null_sweep(lib.mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize, ws_args, [0, 1, 2, 3, 4, 5, 8])
    assert lib.mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(*ws_args) == 0
    args = [handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE, num, 0, 0, FAKE, max(size.value, 64),
            descs[3], FAKE]
    null_sweep(lib.mluOpIndiceConvolutionBackwardFilter, args, [0, 1, 2, 3, 4, 5, 6, 7, 10, 12, 13])
    free_descs(*descs)


# --- descriptors, handle, exports ------------------------------------------------------------------

REDUCE = {"MLUOP_REDUCE_DSUM": 0, "MLUOP_REDUCE_DMEAN": 1, "MLUOP_REDUCE_DMAX": 2}


@pytest.mark.parametrize("case", cases("voxelization"))
def test_voxelization_table(handle, case):
    """api_gtest/src/gtest/voxelization/voxelization_general.cpp: workspace query, then the operator."""
    lib = m.lib()
    p_points, p_vs, p_cr, (max_points, max_voxels, ndim, det), p_vox, p_coors, p_npv, p_num = case["params"]
    descs = [make_desc(p) for p in (p_points, p_vs, p_cr, p_vox, p_coors, p_npv, p_num)]
    det = det in ("true", 1, True)
    try:
        size = ctypes.c_size_t(0)
        st = lib.mluOpGetVoxelizationWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2], max_points,
                                                   max_voxels, ndim, det, descs[3], descs[4], descs[5], descs[6],
                                                   ctypes.byref(size))
        if st != 0:
            assert st == STATUS[case["expected"]]
            return
        st = lib.mluOpVoxelization(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE, max_points,
                                   max_voxels, ndim, det, FAKE, size.value, descs[3], FAKE, descs[4], FAKE,
                                   descs[5], FAKE, descs[6], FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)


@pytest.mark.parametrize("case", cases("dynamic_point_to_voxel_forward"))
def test_dynamic_point_to_voxel_forward_table(handle, case):
    """api_gtest/src/gtest/dynamic_point_to_voxel_forward/dynamic_point_to_voxel_forward_general.cpp."""
    lib = m.lib()
    *tensors, reduce_type = case["params"]
    descs = [make_desc(p) for p in tensors]
    try:
        st = lib.mluOpDynamicPointToVoxelForward(handle.ptr, REDUCE[reduce_type], descs[0], FAKE, descs[1], FAKE,
                                                 FAKE, 1 << 30, descs[2], FAKE, descs[3], FAKE, descs[4], FAKE,
                                                 descs[5], FAKE, descs[6], FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)


@pytest.mark.parametrize("case", cases("dynamic_point_to_voxel_backward"))
def test_dynamic_point_to_voxel_backward_table(handle, case):
    """api_gtest/src/gtest/dynamic_point_to_voxel_backward/dynamic_point_to_voxel_backward_general.cpp."""
    lib = m.lib()
    reduce_type, *tensors = case["params"]
    descs = [make_desc(p) for p in tensors]
    try:
        st = lib.mluOpDynamicPointToVoxelBackward(handle.ptr, REDUCE[reduce_type], descs[0], FAKE, descs[1], FAKE,
                                                  descs[2], FAKE, descs[3], FAKE, descs[4], FAKE, descs[5], FAKE,
                                                  FAKE, 1 << 30, descs[6], FAKE)
        assert st in launch_ok(case["expected"])
    finally:
        free_descs(*descs)


def test_dynamic_point_to_voxel_backward_null_arguments(handle):
    """api_gtest/src/gtest/dynamic_point_to_voxel_backward/dynamic_point_to_voxel_backward.cpp and
    dynamic_point_to_voxel_backward_workspace.cpp: one NULL argument at a time."""
    lib = m.lib()
    f, i = "MLUOP_DTYPE_FLOAT", "MLUOP_DTYPE_INT32"
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", dt, d)) for dt, d in
             ((f, [4, 3]), (f, [6, 3]), (f, [4, 3]), (i, [6]), (i, [4]), (i, [1]), (f, [6, 3]))]
    size = ctypes.c_size_t(0)
    mx = REDUCE["MLUOP_REDUCE_DMAX"]
    ws_args = [handle.ptr, mx, descs[0], descs[1], descs[2], descs[3], descs[4], descs[5], ctypes.byref(size)]
    null_sweep(lib.mluOpGetDynamicPointToVoxelBackwardWorkspaceSize, ws_args, [0, 2, 3, 4, 5, 6, 7, 8])
    assert lib.mluOpGetDynamicPointToVoxelBackwardWorkspaceSize(*ws_args) == 0 and size.value == 6 * 3 * 4
    args = [handle.ptr, mx, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE, descs[3], FAKE, descs[4], FAKE,
            descs[5], FAKE, FAKE, size.value, descs[6], FAKE]
    null_sweep(lib.mluOpDynamicPointToVoxelBackward, args, [0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 16, 17])
    assert lib.mluOpDynamicPointToVoxelBackward(*args) == STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    free_descs(*descs)


def test_voxelization_null_arguments(handle):
    """api_gtest/src/gtest/voxelization/voxelization.cpp:255-413 and voxelization_workspace.cpp:162-242."""
    lib = m.lib()
    f, i = "MLUOP_DTYPE_FLOAT", "MLUOP_DTYPE_INT32"
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", dt, d)) for dt, d in
             ((f, [20, 4]), (f, [3]), (f, [6]), (f, [5, 3, 4]), (i, [5, 3]), (i, [5]), (i, [1]))]
    size = ctypes.c_size_t(0)
    ws_args = [handle.ptr, descs[0], descs[1], descs[2], 3, 5, 3, True, descs[3], descs[4], descs[5], descs[6],
               ctypes.byref(size)]
    null_sweep(lib.mluOpGetVoxelizationWorkspaceSize, ws_args, [0, 1, 2, 3, 8, 9, 10, 11, 12])
    assert lib.mluOpGetVoxelizationWorkspaceSize(*ws_args) == 0 and size.value > 0
    args = [handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE, 3, 5, 3, True, FAKE, size.value, descs[3],
            FAKE, descs[4], FAKE, descs[5], FAKE, descs[6], FAKE]
    null_sweep(lib.mluOpVoxelization, args, [0, 1, 2, 3, 4, 5, 6, 11, 13, 14, 15, 16, 17, 18, 19, 20])
    assert lib.mluOpVoxelization(*args) == STATUS["MLUOP_STATUS_EXECUTION_FAILED"]  # host-only handle
    args[10] = False        # non-deterministic mode does not exist (voxelization.cpp:166-170)
    assert lib.mluOpVoxelization(*args) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    free_descs(*descs)


def test_dynamic_point_to_voxel_forward_null_arguments(handle):
    """api_gtest/src/gtest/dynamic_point_to_voxel_forward/dynamic_point_to_voxel_forward.cpp:326-500 and
    dynamic_point_to_voxel_forward_workspace.cpp:101-140."""
    lib = m.lib()
    f, i = "MLUOP_DTYPE_FLOAT", "MLUOP_DTYPE_INT32"
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", dt, d)) for dt, d in
             ((f, [20, 4]), (i, [20, 3]), (f, [20, 4]), (i, [20, 3]), (i, [20]), (i, [20]), (i, [1]))]
    size = ctypes.c_size_t(0)
    ws_args = [handle.ptr, descs[0], descs[1], ctypes.byref(size)]
    null_sweep(lib.mluOpGetDynamicPointToVoxelForwardWorkspaceSize, ws_args, range(4))
    assert lib.mluOpGetDynamicPointToVoxelForwardWorkspaceSize(*ws_args) == 0 and size.value > 0
    args = [handle.ptr, REDUCE["MLUOP_REDUCE_DMAX"], descs[0], FAKE, descs[1], FAKE, FAKE, size.value, descs[2],
            FAKE, descs[3], FAKE, descs[4], FAKE, descs[5], FAKE, descs[6], FAKE]
    null_sweep(lib.mluOpDynamicPointToVoxelForward, args, [0, 2, 3, 4, 5, 6, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17])
    assert lib.mluOpDynamicPointToVoxelForward(*args) == STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    args[1] = REDUCE["MLUOP_REDUCE_DSUM"]
    assert lib.mluOpDynamicPointToVoxelForward(*args) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    free_descs(*descs)


def test_sparse_conv_descriptor_status_codes():
    """get_indice_pairs_structs.cpp:31-134: NULL create -> NOT_INITIALIZED, NULL destroy -> EXECUTION_FAILED."""
    lib = m.lib()
    assert lib.mluOpCreateSparseConvolutionDescriptor(None) == STATUS["MLUOP_STATUS_NOT_INITIALIZED"]
    assert lib.mluOpDestroySparseConvolutionDescriptor(None) == STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    n = ctypes.c_int(7)
    assert lib.mluOpGetSparseConvolutionNumActOut(None, ctypes.byref(n)) == STATUS["MLUOP_STATUS_NOT_INITIALIZED"]
    d = ctypes.c_void_p()
    assert lib.mluOpCreateSparseConvolutionDescriptor(ctypes.byref(d)) == 0
    one, three = i32([1, 1, 1]), i32([3, 3, 3])
    ok = [d, 5, 1, one, one, one, three, three, three, 0, 0, 0]
    assert lib.mluOpSetSparseConvolutionDescriptor(*ok) == 0
    for pos, val in ((1, 4), (2, 0), (2, -1), (10, 1), (11, 1)):  # dimNb, batch, batch, transpose, inverse
        bad = list(ok)
        bad[pos] = val
        assert lib.mluOpSetSparseConvolutionDescriptor(*bad) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    for pos in range(3, 9):
        bad = list(ok)
        bad[pos] = None
        assert lib.mluOpSetSparseConvolutionDescriptor(*bad) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    bad = list(ok)
    bad[3] = i32([-1, 1, 1])
    assert lib.mluOpSetSparseConvolutionDescriptor(*bad) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    assert lib.mluOpGetSparseConvolutionNumActOut(d, ctypes.byref(n)) == 0 and n.value == 0
    assert lib.mluOpDestroySparseConvolutionDescriptor(d) == 0


def test_tensor_descriptor_roundtrip():
    lib = m.lib()
    d = ctypes.c_void_p()
    assert lib.mluOpCreateTensorDescriptor(None) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    assert lib.mluOpCreateTensorDescriptor(ctypes.byref(d)) == 0
    dims = i32([4, 3, 5])
    assert lib.mluOpSetTensorDescriptor(d, 4, 2, 3, dims) == 0
    assert lib.mluOpGetTensorElementNum(d) == 60
    layout, dtype, nb = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    out_d, out_s = i32([0] * 8), i32([0] * 8)
    assert lib.mluOpGetTensorDescriptorEx(d, ctypes.byref(layout), ctypes.byref(dtype), ctypes.byref(nb), out_d,
                                          out_s) == 0
    assert (layout.value, dtype.value, nb.value) == (4, 2, 3)
    assert list(out_d[:3]) == [4, 3, 5] and list(out_s[:3]) == [15, 5, 1]
    # explicit strides: contiguity is judged from them (core/util.cpp:42-55)
    assert lib.mluOpSetTensorDescriptorEx(d, 4, 2, 3, dims, i32([30, 10, 2])) == 0
    assert lib.mluOpGetTensorDescriptorEx(d, ctypes.byref(layout), ctypes.byref(dtype), ctypes.byref(nb), out_d,
                                          out_s) == 0
    assert list(out_s[:3]) == [30, 10, 2]
    # dim 0 is only legal for host-pointer descriptors (core/tensor.cpp:43-57)
    assert lib.mluOpSetTensorDescriptor(d, 4, 2, 0, None) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    assert lib.mluOpSetTensorDescriptorPointerMode(d, m.POINTER_MODE_HOST) == 0
    assert lib.mluOpSetTensorDescriptor(d, 4, 2, 0, None) == 0
    assert lib.mluOpResetTensorDescriptor(d) == 0
    assert lib.mluOpGetTensorElementNum(d) == 0
    assert lib.mluOpSetTensorDescriptor(d, 4, 2, 2, None) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    big = (ctypes.c_int64 * 10)(*([1] * 9 + [7]))
    assert lib.mluOpSetTensorDescriptor_v2(d, 4, 6, 10, big) == 0  # more than MLUOP_DIM_MAX dims
    assert lib.mluOpGetTensorElementNum(d) == 7
    size = ctypes.c_size_t()
    assert lib.mluOpGetSizeOfDataType(DTYPE["MLUOP_DTYPE_BFLOAT16"], ctypes.byref(size)) == 0 and size.value == 2
    assert lib.mluOpGetSizeOfDataType(0, ctypes.byref(size)) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    assert lib.mluOpDestroyTensorDescriptor(d) == 0
    assert lib.mluOpDestroyTensorDescriptor(None) == STATUS["MLUOP_STATUS_BAD_PARAM"]


def test_non_contiguous_tensor_is_not_supported(handle):
    """STRIDE_TENSOR_CHECK (core/logging.h:214-225): a strided descriptor gives NOT_SUPPORTED."""
    lib = m.lib()
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", d))
             for d in ([10, 4], [27, 2, 10], [10, 4], [27])]
    assert lib.mluOpSetTensorDescriptorEx(descs[0], 4, DTYPE["MLUOP_DTYPE_INT32"], 2, i32([10, 4]), i32([8, 1])) == 0
    sd = m.SparseConvDescriptor(1, [1, 1, 1], [1, 1, 1], [1, 1, 1], [3, 3, 3], [3, 3, 3], [3, 3, 3], 1)
    size = ctypes.c_size_t(0)
    st = lib.mluOpGetIndicePairsWorkspaceSize(handle.ptr, sd.ptr, descs[0], descs[1], descs[2], descs[3],
                                              ctypes.byref(size))
    assert st == STATUS["MLUOP_STATUS_NOT_SUPPORTED"]
    free_descs(*descs)


def test_large_inputs_are_not_supported(handle):
    """L above 1 000 000 rows (get_indice_pairs_structs.h:36) and batch*volume of 2^31 or more."""
    lib = m.lib()
    size = ctypes.c_size_t(0)
    L = 1000001
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", d)) for d in ([L, 4], [27, 2, L], [L, 4], [27])]
    sd = m.SparseConvDescriptor(1, [1, 1, 1], [1, 1, 1], [1, 1, 1], [200, 200, 200], [3, 3, 3], [200, 200, 200], 1)
    st = lib.mluOpGetIndicePairsWorkspaceSize(handle.ptr, sd.ptr, descs[0], descs[1], descs[2], descs[3],
                                              ctypes.byref(size))
    assert st == STATUS["MLUOP_STATUS_BAD_PARAM"]  # PARAM_CHECK_LE in the reference (get_indice_pairs.cpp:162)
    free_descs(*descs)
    descs = [make_desc(T("MLUOP_LAYOUT_ARRAY", "MLUOP_DTYPE_INT32", d)) for d in ([10, 4], [27, 2, 10], [10, 4], [27])]
    sd = m.SparseConvDescriptor(2, [1, 1, 1], [1, 1, 1], [1, 1, 1], [1024, 1024, 1024], [3, 3, 3],
                                [1024, 1024, 1024], 1)
    st = lib.mluOpGetIndicePairsWorkspaceSize(handle.ptr, sd.ptr, descs[0], descs[1], descs[2], descs[3],
                                              ctypes.byref(size))
    assert st == STATUS["MLUOP_STATUS_NOT_SUPPORTED"]
    free_descs(*descs)


def test_handle_queue_and_modes():
    lib = m.lib()
    assert lib.mluOpCreate(None) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    h = host_only_handle()
    q = ctypes.c_void_p(123)
    assert lib.mluOpGetQueue(h.ptr, ctypes.byref(q)) == 0 and q.value is None  # starts on the NULL stream
    assert lib.mluOpSetQueue(h.ptr, ctypes.c_void_p(0x40)) == 0
    assert lib.mluOpGetQueue(h.ptr, ctypes.byref(q)) == 0 and q.value == 0x40
    assert lib.mluOpSetQueue(h.ptr, None) == 0  # NULL queue is allowed (core/context.cpp:362-370)
    mode = ctypes.c_int()
    assert lib.mluOpGetAtomicsMode(h.ptr, ctypes.byref(mode)) == 0 and mode.value == m.ATOMICS_NOT_ALLOWED
    assert lib.mluOpSetAtomicsMode(h.ptr, m.ATOMICS_ALLOWED) == 0
    assert lib.mluOpGetAtomicsMode(h.ptr, ctypes.byref(mode)) == 0 and mode.value == m.ATOMICS_ALLOWED
    assert lib.mluOpSetQuantizeRoundMode(h.ptr, 5) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    major, minor, patch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    lib.mluOpGetLibVersion(ctypes.byref(major), ctypes.byref(minor), ctypes.byref(patch))
    assert (major.value, minor.value, patch.value) == (1, 11, 1)
    assert lib.mluOpGetErrorString(3) == b"MLUOP_STATUS_BAD_PARAM"
    assert lib.mluOpDestroy(None) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    h.close()


def test_library_exports_every_declared_symbol():
    """Every function declared in include/*.h is exported by libmluops.so and bound in the ctypes table."""
    declared = set()
    for name in ("mlu_op.h", "mlu_op_ext.h"):
        text = open(os.path.join(ROOT, "include", name)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        declared |= set(re.findall(r"\b(mluOp[A-Za-z0-9_]+)\s*\(", text))
    assert len(declared) >= 40
    lib = ctypes.CDLL(m.LIB_PATH)
    for sym in sorted(declared):
        assert hasattr(lib, sym), sym
    assert declared == set(m.SIGNATURES), declared ^ set(m.SIGNATURES)


def test_library_exports_the_c_api_and_nothing_else():
    """The dynamic symbol table of libmluops.so holds the declared mluOp* functions only: the C++
    helpers behind them are local (the reference links with a symbol map for the same reason,
    CMakeLists.txt:226, scripts/gen_symbol_visibility_map.py)."""
    import shutil
    import subprocess
    nm = shutil.which("nm")
    if nm is None:
        pytest.skip("nm is not installed")
    out = subprocess.run([nm, "-D", "--defined-only", m.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    declared = set()
    for name in ("mlu_op.h", "mlu_op_ext.h"):
        text = open(os.path.join(ROOT, "include", name)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        declared |= set(re.findall(r"\b(mluOp[A-Za-z0-9_]+)\s*\(", text))
    assert exported == declared, sorted(exported ^ declared)


# --- extended modes (mluOpExtSetSparseConvExtendedModes): inverse = 1, tagged filters_grad ------

def _d(dims, dtype="MLUOP_DTYPE_FLOAT", layout="MLUOP_LAYOUT_ARRAY"):
    return make_desc({"layout": layout, "dtype": dtype, "dim_nb": len(dims), "dims": list(dims)})


def _forward_status(handle, feat, filt, pairs, out, num, n_out, inverse):
    lib = m.lib()
    descs = [_d(feat), _d(filt), _d(pairs, "MLUOP_DTYPE_INT32"), _d(out)]
    try:
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndiceConvolutionForwardWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2], descs[3],
                                                               i64(num), n_out, inverse, 0, ctypes.byref(size))
        if st != 0:
            return st
        return lib.mluOpIndiceConvolutionForward(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE,
                                                 i64(num), n_out, inverse, 0, FAKE, size.value, descs[3], FAKE)
    finally:
        free_descs(*descs)


def _backward_data_status(handle, dy, filt, pairs, dx, num, inverse):
    lib = m.lib()
    descs = [_d(dy), _d(filt), _d(pairs, "MLUOP_DTYPE_INT32"), _d(dx)]
    try:
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2],
                                                                    descs[3], i64(num), inverse, ctypes.byref(size))
        if st != 0:
            return st
        return lib.mluOpIndiceConvolutionBackwardData(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE,
                                                      i64(num), inverse, 0, FAKE, size.value, descs[3], FAKE)
    finally:
        free_descs(*descs)


def _backward_filter_status(handle, feat, dy, pairs, dw, num, inverse, dw_layout="MLUOP_LAYOUT_ARRAY"):
    lib = m.lib()
    descs = [_d(feat), _d(dy), _d(pairs, "MLUOP_DTYPE_INT32"), _d(dw, layout=dw_layout)]
    try:
        size = ctypes.c_size_t(64)
        st = lib.mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(handle.ptr, descs[0], descs[1], descs[2],
                                                                      descs[3], i64(num), inverse, 0,
                                                                      ctypes.byref(size))
        if st != 0:
            return st
        return lib.mluOpIndiceConvolutionBackwardFilter(handle.ptr, descs[0], FAKE, descs[1], FAKE, descs[2], FAKE,
                                                        i64(num), inverse, 0, FAKE, size.value, descs[3], FAKE)
    finally:
        free_descs(*descs)


@pytest.fixture()
def extended(handle):
    handle.set_extended_modes(True)
    yield handle
    handle.set_extended_modes(False)


def test_inverse_keeps_the_reference_status_until_switched_on(handle):
    K, L, n_in, ci, co = 8, 10, 6, 4, 5     # partner: 10 input rows, 6 output rows, 2x2x2 kernel
    num = [3] * K
    fwd = ([n_in, ci], [2, 2, 2, ci, co], [K, 2, L], [L, co], num, L, 1)
    bwd = ([L, co], [2, 2, 2, ci, co], [K, 2, L], [n_in, ci], num, 1)
    flt = ([n_in, ci], [L, co], [K, 2, L], [2, 2, 2, ci, co], num, 1)
    assert _forward_status(handle, *fwd) == STATUS["MLUOP_STATUS_NOT_SUPPORTED"]
    assert _backward_data_status(handle, *bwd) == STATUS["MLUOP_STATUS_NOT_SUPPORTED"]
    assert _backward_filter_status(handle, *flt) == STATUS["MLUOP_STATUS_BAD_PARAM"]
    handle.set_extended_modes(True)
    try:
        launched = STATUS["MLUOP_STATUS_EXECUTION_FAILED"]   # every check passed; a host-only handle stops here
        assert _forward_status(handle, *fwd) == launched
        assert _backward_data_status(handle, *bwd) == launched
        assert _backward_filter_status(handle, *flt) == launched
    finally:
        handle.set_extended_modes(False)
    assert _forward_status(handle, *fwd) == STATUS["MLUOP_STATUS_NOT_SUPPORTED"]
    assert m.lib().mluOpExtSetSparseConvExtendedModes(None, 1) == STATUS["MLUOP_STATUS_BAD_PARAM"]


def test_inverse_shape_checks(extended):
    K, L, n_in, ci, co = 8, 10, 6, 4, 5
    num = [3] * K
    bad = STATUS["MLUOP_STATUS_BAD_PARAM"]
    filt = [2, 2, 2, ci, co]
    # indice_pairs.dim[2] is the row count of the output side under inverse = 1
    assert _forward_status(extended, [n_in, ci], filt, [K, 2, L], [L + 1, co], num, L + 1, 1) == bad
    assert _forward_status(extended, [n_in, ci], filt, [K, 2, L], [L, co], num, L - 1, 1) == bad
    assert _forward_status(extended, [n_in, ci + 1], filt, [K, 2, L], [L, co], num, L, 1) == bad
    assert _forward_status(extended, [n_in, ci], filt, [K, 2, L], [L, co], [L + 1] * K, L, 1) == bad
    # more pairs than input rows is what repeated coordinates in the partner layer give
    assert _forward_status(extended, [n_in, ci], filt, [K, 2, L], [L, co], [n_in + 1] * K, L, 1) == \
        STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    assert _forward_status(extended, [n_in, ci], filt, [K, 2, L], [L, co], num, L, 2) == bad
    assert _backward_data_status(extended, [L + 1, co], filt, [K, 2, L], [n_in, ci], num, 1) == bad
    assert _backward_data_status(extended, [L, co], filt, [K, 2, L], [2, ci], num, 1) == \
        STATUS["MLUOP_STATUS_EXECUTION_FAILED"]   # fewer input rows than pairs: repeated coordinates
    assert _backward_data_status(extended, [L, co], filt, [K, 2, L], [n_in, ci + 1], num, 1) == bad
    assert _backward_filter_status(extended, [n_in, ci], [L + 1, co], [K, 2, L], filt, num, 1) == bad
    assert _backward_filter_status(extended, [n_in, ci], [L, co], [K, 2, L], filt, num, 2) == bad
    # the regular direction keeps its own rule with the switch on
    assert _forward_status(extended, [L, ci], filt, [K, 2, L], [n_in, co], num, n_in, 0) == \
        STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    assert _forward_status(extended, [L + 1, ci], filt, [K, 2, L], [n_in, co], num, n_in, 0) == bad


def test_tagged_filters_grad_layouts(handle):
    K, L, n_out, ci, co = 8, 10, 6, 4, 5
    num = [3] * K
    ndhwc, ncdhw = [co, 2, 2, 2, ci], [co, ci, 2, 2, 2]
    args = ([L, ci], [n_out, co], [K, 2, L])
    # positional reading, as in the reference: the tagged shapes do not fit
    assert _backward_filter_status(handle, *args, ndhwc, num, 0, "MLUOP_LAYOUT_NDHWC") == STATUS["MLUOP_STATUS_BAD_PARAM"]
    assert _backward_filter_status(handle, *args, ncdhw, num, 0, "MLUOP_LAYOUT_NCDHW") == STATUS["MLUOP_STATUS_BAD_PARAM"]
    assert _backward_filter_status(handle, *args, [2, 2, 2, ci, co], num, 0, "MLUOP_LAYOUT_NDHWC") == \
        STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    handle.set_extended_modes(True)
    try:
        launched = STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
        assert _backward_filter_status(handle, *args, ndhwc, num, 0, "MLUOP_LAYOUT_NDHWC") == launched
        assert _backward_filter_status(handle, *args, ncdhw, num, 0, "MLUOP_LAYOUT_NCDHW") == launched
        assert _backward_filter_status(handle, *args, [co, 2, 2, ci], [3] * 4, 0, "MLUOP_LAYOUT_NHWC") == \
            STATUS["MLUOP_STATUS_BAD_PARAM"]          # K = 4 against 8 offsets in indice_pairs
        assert _backward_filter_status(handle, ([L, ci]), [n_out, co], [4, 2, L], [co, 2, 2, ci], [3] * 4, 0,
                                       "MLUOP_LAYOUT_NHWC") == launched
        assert _backward_filter_status(handle, *args, [2, 2, 2, ci, co], num, 0, "MLUOP_LAYOUT_NDHWC") == \
            STATUS["MLUOP_STATUS_BAD_PARAM"]          # now read as [Co, kd, kh, kw, Ci]
        assert _backward_filter_status(handle, *args, [2, 2, 2, ci, co], num, 0, "MLUOP_LAYOUT_ARRAY") == launched
    finally:
        handle.set_extended_modes(False)


def test_missing_library_fails_loudly(monkeypatch):
    """No fallback path: without the built library the binding raises instead of computing elsewhere."""
    monkeypatch.setattr(m, "_lib", None)
    monkeypatch.setattr(m, "LIB_PATH", os.path.join(ROOT, "mlu-ops_amd", "lib", "no_such_library.so"))
    with pytest.raises(RuntimeError, match="there is no fallback path"):
        m.lib()


def test_descriptors_from_many_threads():
    """The descriptor pool is the one shared structure (locked, as core/tensor.cpp:205-241 locks
    the reference's): eight threads create, set, read back and destroy descriptors at once."""
    import threading
    lib = m.lib()
    errors = []

    def worker(seed):
        try:
            for i in range(300):
                dims = [seed + 1, (i % 7) + 1, 3]
                d = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_FLOAT, dims)
                n = lib.mluOpGetTensorElementNum(d.ptr)
                if n != dims[0] * dims[1] * dims[2]:
                    errors.append((seed, i, n))
                d.close()
        except Exception as e:
            errors.append((seed, repr(e)))

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=60)
    assert not errors, errors[:3]


def test_row_map_entry_points(handle):
    """Checks of mluOpExtGetRowMapSize / BuildRowMap / UseRowMap / ForgetRowMap; with every check
    passed a handle without a device stops where the build would launch."""
    lib = m.lib()
    bad, failed = STATUS["MLUOP_STATUS_BAD_PARAM"], STATUS["MLUOP_STATUS_EXECUTION_FAILED"]
    K, L, n_out = 27, 100, 40
    def desc(dtype, dims):
        return make_desc({"layout": "MLUOP_LAYOUT_ARRAY", "dtype": dtype, "dim_nb": len(dims), "dims": dims})

    pairs = desc("MLUOP_DTYPE_INT32", [K, 2, L])
    floats = desc("MLUOP_DTYPE_FLOAT", [K, 2, L])
    flat = desc("MLUOP_DTYPE_INT32", [K, L])
    try:
        size = ctypes.c_size_t(0)
        assert lib.mluOpExtGetRowMapSize(pairs, n_out, ctypes.byref(size)) == 0
        assert size.value >= K * n_out * 4
        assert lib.mluOpExtGetRowMapSize(None, n_out, ctypes.byref(size)) == bad
        assert lib.mluOpExtGetRowMapSize(pairs, n_out, None) == bad
        assert lib.mluOpExtGetRowMapSize(pairs, -1, ctypes.byref(size)) == bad
        assert lib.mluOpExtGetRowMapSize(flat, n_out, ctypes.byref(size)) == bad
        small = size.value
        assert lib.mluOpExtGetRowMapSize(pairs, L, ctypes.byref(size)) == 0 and size.value > small
        num, lost = i64([3] * K), ctypes.c_int64(0)

        def build(desc=pairs, data=FAKE, counts=num, rows=n_out, source=L, column=1, out=FAKE, nbytes=None,
                  lost_ref=ctypes.byref(lost), h=handle.ptr):
            return lib.mluOpExtBuildRowMap(h, desc, data, counts, rows, source, column, out,
                                           size.value if nbytes is None else nbytes, lost_ref)

        assert build() == failed                       # all checks passed
        assert build(rows=L, source=n_out, column=0) == failed
        assert build(h=None) == bad
        assert build(desc=None) == bad
        assert build(desc=floats) == bad
        assert build(data=None) == bad
        assert build(counts=None) == bad
        assert build(out=None) == bad
        assert build(lost_ref=None) == bad             # no place for the verdict and no promise
        handle.promise_distinct_pairs(True)
        try:
            assert build(lost_ref=None) == failed      # the promise stands in for it
        finally:
            handle.promise_distinct_pairs(False)
        assert build(column=2) == bad
        assert build(rows=0) == bad
        assert build(source=L + 1) == bad              # column 0 indexes indice_pairs.dim[2] rows
        assert build(rows=L + 1, source=n_out, column=0) == bad
        assert build(nbytes=small - 1) == bad
        assert build(counts=i64([L + 1] + [0] * (K - 1))) == bad
        assert build(counts=i64([-1] + [0] * (K - 1))) == bad

        assert lib.mluOpExtUseRowMap(None, FAKE) == bad
        assert lib.mluOpExtUseRowMap(handle.ptr, FAKE) == bad      # nothing was built into it
        assert lib.mluOpExtUseRowMap(handle.ptr, None) == 0        # withdraws an announcement
        assert lib.mluOpExtForgetRowMap(handle.ptr, FAKE) == 0
        assert lib.mluOpExtForgetRowMap(handle.ptr, None) == 0
        assert lib.mluOpExtForgetRowMap(None, None) == bad
    finally:
        free_descs(pairs, floats, flat)


def test_kernel_choice_setter_checks_its_arguments(handle):
    ok, bad = STATUS["MLUOP_STATUS_SUCCESS"], STATUS["MLUOP_STATUS_BAD_PARAM"]
    f = m.lib().mluOpExtSetKernelChoice
    for which in range(8):
        for value in (-1, 0, 1, -1):
            assert f(handle.ptr, which, value) == ok
    assert f(None, 0, 1) == bad
    assert f(handle.ptr, 8, 1) == bad and f(handle.ptr, -1, 1) == bad
    assert f(handle.ptr, 0, 2) == bad and f(handle.ptr, 0, -2) == bad


def test_gather_workspaces_do_not_grow_with_offsets_times_rows(handle):
    """The row map of forward and backward data covers a chunk of result rows at a time (64 MiB at
    most), so the workspace of a 5x5x5 filter over 400 000 or 1 000 000 rows stays far below the
    K x rows x 4 bytes (200 MB, 500 MB) a whole map would take."""
    lib = m.lib()
    for rows, bound in ((400000, 128 << 20), (1000000, 160 << 20)):
        K, c = 125, 128
        descs = [_d([rows, c]), _d([5, 5, 5, c, c]), _d([K, 2, rows], "MLUOP_DTYPE_INT32"), _d([rows, c])]
        try:
            size = ctypes.c_size_t(0)
            num = [rows] * K
            assert lib.mluOpGetIndiceConvolutionForwardWorkspaceSize(
                handle.ptr, descs[0], descs[1], descs[2], descs[3], i64(num), rows, 0, 1, ctypes.byref(size)) == 0
            assert 0 < size.value < bound < K * rows * 4, size.value
            assert lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(
                handle.ptr, descs[0], descs[1], descs[2], descs[3], i64(num), 0, ctypes.byref(size)) == 0
            assert 0 < size.value < bound, size.value
        finally:
            free_descs(*descs)
