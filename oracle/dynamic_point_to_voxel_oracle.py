"""numpy front end of the CPU oracle for dynamic point-to-voxel scatter (TEST INFRASTRUCTURE, not
product code).  Loads ``libdynamic_point_to_voxel_oracle.so``; only tests import this module."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdynamic_point_to_voxel_oracle.so")
_lib = None
_i32p = ctypes.POINTER(ctypes.c_int32)
_f32p = ctypes.POINTER(ctypes.c_float)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            subprocess.check_call(["make", "-C", _HERE, "-s"])
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_dynamic_point_to_voxel_forward.restype = ctypes.c_int32
        _lib.oracle_dynamic_point_to_voxel_backward.restype = ctypes.c_int32
    return _lib


def forward(reduce_type, feats, coors, rows=None):
    """reduce_type "max" or "mean".  Returns (voxel_feats [rows, C], voxel_coors [rows, 3],
    point2voxel_map [N], voxel_points_count [rows], voxel_num, coors as the operator leaves it);
    rows defaults to N."""
    feats = np.ascontiguousarray(feats, dtype=np.float32)
    coors = np.array(coors, dtype=np.int32, order="C", copy=True)
    n, c = feats.shape
    m = n if rows is None else rows
    vf = np.empty((m, c), np.float32)
    vc = np.empty((m, 3), np.int32)
    p2v = np.full((n,), -1, np.int32)
    cnt = np.empty((m,), np.int32)
    num = np.zeros((1,), np.int32)
    rc = lib().oracle_dynamic_point_to_voxel_forward(
        ctypes.c_int32(1 if reduce_type == "max" else 0), feats.ctypes.data_as(_f32p),
        coors.ctypes.data_as(_i32p), ctypes.c_int32(n), ctypes.c_int32(c), ctypes.c_int32(m),
        vf.ctypes.data_as(_f32p), vc.ctypes.data_as(_i32p), p2v.ctypes.data_as(_i32p),
        cnt.ctypes.data_as(_i32p), num.ctypes.data_as(_i32p))
    if rc != 0:
        raise MemoryError("oracle_dynamic_point_to_voxel_forward")
    return vf, vc, p2v, cnt, int(num[0]), coors


def backward(grad_voxel_feats, feats, voxel_feats, point2voxel_map, voxel_num):
    """Gradient of the max reduction with respect to feats: [N, C]."""
    g = np.ascontiguousarray(grad_voxel_feats, dtype=np.float32)
    feats = np.ascontiguousarray(feats, dtype=np.float32)
    vf = np.ascontiguousarray(voxel_feats, dtype=np.float32)
    p2v = np.ascontiguousarray(point2voxel_map, dtype=np.int32)
    n, c = feats.shape
    out = np.empty((n, c), np.float32)
    rc = lib().oracle_dynamic_point_to_voxel_backward(
        g.ctypes.data_as(_f32p), feats.ctypes.data_as(_f32p), vf.ctypes.data_as(_f32p),
        p2v.ctypes.data_as(_i32p), ctypes.c_int32(int(voxel_num)), ctypes.c_int32(n), ctypes.c_int32(c),
        ctypes.c_int32(g.shape[0]), out.ctypes.data_as(_f32p))
    if rc != 0:
        raise MemoryError("oracle_dynamic_point_to_voxel_backward")
    return out
