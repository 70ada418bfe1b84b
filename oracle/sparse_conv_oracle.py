"""numpy front end of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Loads ``libsparse_conv_oracle.so`` built from ``sparse_conv_oracle.c`` (a plain-C
restatement of the reference gtest executors' ``cpuCompute``) and exposes it on
numpy arrays.  Only tests, the smoke check and the benchmark's cpu_baseline leg
import this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsparse_conv_oracle.so")
_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_get_indice_pairs.restype = ctypes.c_int32
        for name in ("oracle_diff1", "oracle_diff2", "oracle_diff3"):
            getattr(_lib, name).restype = ctypes.c_double
    return _lib


def _p(a, t):
    return a.ctypes.data_as(t)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def get_indice_pairs(indices, batch, pad, stride, dilation, filter_space, out_space, sub_m,
                     out_rows=None, exact_count=False):
    """Returns (indice_pairs [K,2,L], out_indices [out_rows,4], indice_num [K], num_act_out)."""
    indices = _i32(indices).reshape(-1, 4)
    L = indices.shape[0]
    K = int(np.prod(filter_space))
    if out_rows is None:
        out_rows = L if sub_m else int(batch * np.prod(out_space))
    pairs = np.empty((K, 2, L), dtype=np.int32)
    out_indices = np.empty((out_rows, 4), dtype=np.int32)
    num = np.empty((K,), dtype=np.int32)
    arr = lambda v: _i32(np.asarray(v))
    pad_a, st_a, di_a, fs_a, os_a = arr(pad), arr(stride), arr(dilation), arr(filter_space), arr(out_space)
    n = lib().oracle_get_indice_pairs(
        _p(indices, _i32p), ctypes.c_int32(L), ctypes.c_int32(batch), _p(pad_a, _i32p),
        _p(st_a, _i32p), _p(di_a, _i32p), _p(fs_a, _i32p), _p(os_a, _i32p),
        ctypes.c_int32(1 if sub_m else 0), ctypes.c_int32(out_rows),
        ctypes.c_int32(1 if exact_count else 0), _p(pairs, _i32p), _p(out_indices, _i32p),
        _p(num, _i32p))
    if n < 0:
        raise MemoryError("oracle_get_indice_pairs")
    return pairs, out_indices, num, int(n)


def filters_to_kcico(filters, layout, K, ci, co):
    f = _f32(filters).reshape(-1)
    out = np.empty((K, ci, co), dtype=np.float32)
    lib().oracle_filters_to_kcico(_p(f, _f32p), ctypes.c_int32(layout), ctypes.c_int64(K),
                                  ctypes.c_int64(ci), ctypes.c_int64(co), _p(out, _f32p))
    return out


def _swapped(indice_pairs):
    """The rulebook with its two pair columns exchanged."""
    return np.ascontiguousarray(_i32(indice_pairs)[:, ::-1, :])


def _num64(indice_num):
    return np.ascontiguousarray(indice_num, dtype=np.int64)


def forward(features, filters_kcico, indice_pairs, indice_num, num_act_out, inverse=False):
    """inverse=True is the sparse inverse convolution, which the reference does not
    implement (indice_convolution_forward.cpp:74-78 rejects it): the operator of the PyTorch
    sparse-convolution stacks the reference serves (spconv 1.x indice_conv / mmcv
    SparseInverseConv3d, neither vendored here) runs the partner layer's rulebook backwards,
    out[pairs[k,0,p]] += features[pairs[k,1,p]] . W[k]; that is this function on the rulebook
    with its columns exchanged.  Pinned in tests against dense conv_transpose3d."""
    features = _f32(features)
    w = _f32(filters_kcico)
    pairs = _swapped(indice_pairs) if inverse else _i32(indice_pairs)
    num = _num64(indice_num)
    K, _, L = pairs.shape
    ci, co = w.shape[1], w.shape[2]
    out = np.empty((num_act_out, co), dtype=np.float32)
    lib().oracle_indice_conv_forward(_p(features, _f32p), _p(w, _f32p), _p(pairs, _i32p),
                                     _p(num, _i64p), ctypes.c_int64(L), ctypes.c_int64(K),
                                     ctypes.c_int64(ci), ctypes.c_int64(co),
                                     ctypes.c_int64(num_act_out), _p(out, _f32p))
    return out


def backward_data(output_grad, filters_kcico, indice_pairs, indice_num, inverse=False, rows=None):
    """inverse=True: dX[pairs[k,1,p]] += dY[pairs[k,0,p]] . W[k]^T over `rows` input rows, which
    is the forward loop over the unchanged rulebook with dY as features and W[k]^T as filter."""
    if inverse:
        wt = np.ascontiguousarray(np.transpose(_f32(filters_kcico), (0, 2, 1)))
        return forward(output_grad, wt, indice_pairs, indice_num, int(rows))
    dy = _f32(output_grad)
    w = _f32(filters_kcico)
    pairs = _i32(indice_pairs)
    num = _num64(indice_num)
    K, _, L = pairs.shape
    ci, co = w.shape[1], w.shape[2]
    dx = np.empty((L, ci), dtype=np.float32)
    lib().oracle_indice_conv_backward_data(_p(dy, _f32p), _p(w, _f32p), _p(pairs, _i32p),
                                           _p(num, _i64p), ctypes.c_int64(L), ctypes.c_int64(K),
                                           ctypes.c_int64(ci), ctypes.c_int64(co), _p(dx, _f32p))
    return dx


def backward_filter(features, output_grad, indice_pairs, indice_num, fast=False, inverse=False):
    """inverse=True: dW[k] = sum_p features[pairs[k,1,p]]^T . dY[pairs[k,0,p]], the same loop on
    the rulebook with its columns exchanged."""
    x = _f32(features)
    dy = _f32(output_grad)
    pairs = _swapped(indice_pairs) if inverse else _i32(indice_pairs)
    num = _num64(indice_num)
    K, _, L = pairs.shape
    ci, co = x.shape[1], dy.shape[1]
    dw = np.empty((K, ci, co), dtype=np.float32)
    fn = lib().oracle_indice_conv_backward_filter_fast if fast else \
        lib().oracle_indice_conv_backward_filter
    fn(_p(x, _f32p), _p(dy, _f32p), _p(pairs, _i32p), _p(num, _i64p), ctypes.c_int64(L),
       ctypes.c_int64(K), ctypes.c_int64(ci), ctypes.c_int64(co), _p(dw, _f32p))
    return dw


def round_through_half(a):
    a = _f32(a)
    out = np.empty_like(a)
    lib().oracle_round_through_half(_p(a, _f32p), _p(out, _f32p), ctypes.c_int64(a.size))
    return out


def float_to_half_bits(a):
    a = _f32(a)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().oracle_float_to_half_bits(_p(a, _f32p), _p(out, _u16p), ctypes.c_int64(a.size))
    return out


def round_through_bf16(a):
    a = _f32(a)
    out = np.empty_like(a)
    lib().oracle_round_through_bf16(_p(a, _f32p), _p(out, _f32p), ctypes.c_int64(a.size))
    return out


def float_to_bf16_bits(a):
    a = _f32(a)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().oracle_float_to_bf16_bits(_p(a, _f32p), _p(out, _u16p), ctypes.c_int64(a.size))
    return out


def diff1(a, b):
    a, b = _f32(a).reshape(-1), _f32(b).reshape(-1)
    return lib().oracle_diff1(_p(a, _f32p), _p(b, _f32p), ctypes.c_int64(a.size))


def diff2(a, b):
    a, b = _f32(a).reshape(-1), _f32(b).reshape(-1)
    return lib().oracle_diff2(_p(a, _f32p), _p(b, _f32p), ctypes.c_int64(a.size))


def diff3(a, b, half=False):
    a, b = _f32(a).reshape(-1), _f32(b).reshape(-1)
    return lib().oracle_diff3(_p(a, _f32p), _p(b, _f32p), ctypes.c_int64(a.size),
                              ctypes.c_double(1e-4 if half else 1e-6))
