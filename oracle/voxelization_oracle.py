"""numpy front end of the CPU oracle for hard voxelization (TEST INFRASTRUCTURE, not product
code).  Loads ``libvoxelization_oracle.so`` built from ``voxelization_oracle.c``; only tests and
the smoke check import this module."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvoxelization_oracle.so")
_lib = None
_i32p = ctypes.POINTER(ctypes.c_int32)
_f32p = ctypes.POINTER(ctypes.c_float)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            subprocess.check_call(["make", "-C", _HERE, "-s"])
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_voxelization.restype = ctypes.c_int32
    return _lib


def voxelization(points, voxel_size, coors_range, max_points, max_voxels):
    """Returns (voxels [max_voxels, max_points, F] float32, coors [max_voxels, 3] int32 as
    (z, y, x), num_points_per_voxel [max_voxels] int32, voxel_num int)."""
    points = np.ascontiguousarray(points, dtype=np.float32)
    vs = np.ascontiguousarray(voxel_size, dtype=np.float32)
    cr = np.ascontiguousarray(coors_range, dtype=np.float32)
    n, f = points.shape
    voxels = np.empty((max_voxels, max_points, f), dtype=np.float32)
    coors = np.empty((max_voxels, 3), dtype=np.int32)
    npv = np.empty((max_voxels,), dtype=np.int32)
    num = np.zeros((1,), dtype=np.int32)
    rc = lib().oracle_voxelization(
        points.ctypes.data_as(_f32p), vs.ctypes.data_as(_f32p), cr.ctypes.data_as(_f32p),
        ctypes.c_int64(n), ctypes.c_int64(f), ctypes.c_int32(max_points), ctypes.c_int32(max_voxels),
        voxels.ctypes.data_as(_f32p), coors.ctypes.data_as(_i32p), npv.ctypes.data_as(_i32p),
        num.ctypes.data_as(_i32p))
    if rc != 0:
        raise MemoryError("oracle_voxelization")
    return voxels, coors, npv, int(num[0])
