"""ctypes binding of libmluops.so, the MI355X sparse-convolution library.

The module mirrors the C API of ``include/mlu_op.h`` one to one (``lib()`` returns
the loaded library with argument types set) and adds a thin convenience layer
(`Handle`, `TensorDescriptor`, `SparseConvDescriptor`, `get_indice_pairs`,
`indice_conv_forward`, ...) that follows the call sequence a framework uses:
create descriptor -> query workspace -> run op -> read num_act_out -> copy
indice_num to the host -> convolution ops.

Device buffers are torch tensors; torch supplies memory and the stream, every
computation runs in the library's own HIP kernels.  There is no CPU fallback: a
missing library raises at import of the first symbol.
"""
import ctypes
import threading
import os

from . import datagen  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
# MLUOP_LIBRARY names another build of the library (the sanitizer build of `make asan`).
LIB_PATH = os.environ.get("MLUOP_LIBRARY") or os.path.normpath(
    os.path.join(_HERE, "..", "..", "lib", "libmluops.so"))

# mluOpStatus_t
STATUS_SUCCESS = 0
STATUS_NOT_INITIALIZED = 1
STATUS_ALLOC_FAILED = 2
STATUS_BAD_PARAM = 3
STATUS_INTERNAL_ERROR = 4
STATUS_ARCH_MISMATCH = 5
STATUS_EXECUTION_FAILED = 6
STATUS_NOT_SUPPORTED = 7
STATUS_NUMERICAL_OVERFLOW = 8

# mluOpTensorLayout_t
LAYOUT_NCHW, LAYOUT_NHWC, LAYOUT_HWCN, LAYOUT_NDHWC, LAYOUT_ARRAY, LAYOUT_NCDHW = 0, 1, 2, 3, 4, 5
LAYOUT_TNC, LAYOUT_NTC, LAYOUT_NC, LAYOUT_NLC, LAYOUT_NCL = 6, 7, 8, 9, 10

# mluOpDataType_t
DTYPE_INVALID, DTYPE_HALF, DTYPE_FLOAT, DTYPE_INT8, DTYPE_INT16, DTYPE_INT31 = 0, 1, 2, 3, 4, 5
DTYPE_INT32, DTYPE_UINT8, DTYPE_BOOL, DTYPE_INT64 = 6, 7, 8, 9
DTYPE_UINT32, DTYPE_UINT64, DTYPE_UINT16, DTYPE_DOUBLE = 11, 12, 13, 14
DTYPE_COMPLEX_HALF, DTYPE_COMPLEX_FLOAT, DTYPE_BFLOAT16 = 15, 16, 17

ATOMICS_NOT_ALLOWED, ATOMICS_ALLOWED = 1, 2
REDUCE_DSUM, REDUCE_DMEAN, REDUCE_DMAX = 0, 1, 2
POINTER_MODE_HOST, POINTER_MODE_DEVICE = 0, 1

_vp = ctypes.c_void_p
_ip = ctypes.POINTER(ctypes.c_int)
_i64p = ctypes.POINTER(ctypes.c_int64)
_szp = ctypes.POINTER(ctypes.c_size_t)

# name -> (restype, argtypes); every symbol declared in include/mlu_op.h.
SIGNATURES = {
    "mluOpCreate": (ctypes.c_int, [ctypes.POINTER(_vp)]),
    "mluOpDestroy": (ctypes.c_int, [_vp]),
    "mluOpSetQueue": (ctypes.c_int, [_vp, _vp]),
    "mluOpGetQueue": (ctypes.c_int, [_vp, ctypes.POINTER(_vp)]),
    "mluOpGetErrorString": (ctypes.c_char_p, [ctypes.c_int]),
    "mluOpGetSizeOfDataType": (ctypes.c_int, [ctypes.c_int, _szp]),
    "mluOpGetLibVersion": (None, [_ip, _ip, _ip]),
    "mluOpSetQuantizeRoundMode": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpGetQuantizeRoundMode": (ctypes.c_int, [_vp, _ip]),
    "mluOpSetAtomicsMode": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpGetAtomicsMode": (ctypes.c_int, [_vp, _ip]),
    "mluOpCreateTensorDescriptor": (ctypes.c_int, [ctypes.POINTER(_vp)]),
    "mluOpSetTensorDescriptor": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _ip]),
    "mluOpSetTensorDescriptor_v2": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i64p]),
    "mluOpSetTensorDescriptorEx": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _ip, _ip]),
    "mluOpSetTensorDescriptorEx_v2": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i64p, _i64p]),
    "mluOpSetTensorDescriptorPointerMode": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpGetTensorDescriptorPointerMode": (ctypes.c_int, [_vp, _ip]),
    "mluOpSetTensorDescriptorOnchipDataType": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpGetTensorDescriptorOnchipDataType": (ctypes.c_int, [_vp, _ip]),
    "mluOpGetTensorDescriptor": (ctypes.c_int, [_vp, _ip, _ip, _ip, _ip]),
    "mluOpGetTensorDescriptor_v2": (ctypes.c_int, [_vp, _ip, _ip, _ip, _i64p]),
    "mluOpGetTensorDescriptorEx": (ctypes.c_int, [_vp, _ip, _ip, _ip, _ip, _ip]),
    "mluOpGetTensorDescriptorEx_v2": (ctypes.c_int, [_vp, _ip, _ip, _ip, _i64p, _i64p]),
    "mluOpGetTensorElementNum": (ctypes.c_size_t, [_vp]),
    "mluOpResetTensorDescriptor": (ctypes.c_int, [_vp]),
    "mluOpDestroyTensorDescriptor": (ctypes.c_int, [_vp]),
    "mluOpCreateSparseConvolutionDescriptor": (ctypes.c_int, [ctypes.POINTER(_vp)]),
    "mluOpDestroySparseConvolutionDescriptor": (ctypes.c_int, [_vp]),
    "mluOpSetSparseConvolutionDescriptor": (
        ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int, _ip, _ip, _ip, _ip, _ip, _ip,
                       ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mluOpGetSparseConvolutionNumActOut": (ctypes.c_int, [_vp, _ip]),
    "mluOpGetIndicePairs": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, ctypes.c_size_t, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mluOpGetIndicePairsWorkspaceSize": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _szp]),
    "mluOpGetIndiceConvolutionForwardWorkspaceSize": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, ctypes.c_int64,
                       ctypes.c_int64, _szp]),
    "mluOpIndiceConvolutionForward": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, ctypes.c_int64,
                       ctypes.c_int64, _vp, ctypes.c_size_t, _vp, _vp]),
    "mluOpGetIndiceConvolutionBackwardDataWorkspaceSize": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, _szp]),
    "mluOpIndiceConvolutionBackwardData": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, ctypes.c_int64,
                       _vp, ctypes.c_size_t, _vp, _vp]),
    "mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, ctypes.c_int64, _szp]),
    "mluOpIndiceConvolutionBackwardFilter": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, ctypes.c_int64,
                       _vp, ctypes.c_size_t, _vp, _vp]),
    "mluOpGetVoxelizationWorkspaceSize": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_bool,
                       _vp, _vp, _vp, _vp, _szp]),
    "mluOpVoxelization": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                       ctypes.c_bool, _vp, ctypes.c_size_t, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mluOpGetDynamicPointToVoxelForwardWorkspaceSize": (ctypes.c_int, [_vp, _vp, _vp, _szp]),
    "mluOpDynamicPointToVoxelForward": (
        ctypes.c_int, [_vp, ctypes.c_int, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t, _vp, _vp, _vp, _vp,
                       _vp, _vp, _vp, _vp, _vp, _vp]),
    "mluOpGetDynamicPointToVoxelBackwardWorkspaceSize": (
        ctypes.c_int, [_vp, ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _szp]),
    "mluOpDynamicPointToVoxelBackward": (
        ctypes.c_int, [_vp, ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                       ctypes.c_size_t, _vp, _vp]),
    # mlu_op_ext.h
    "mluOpExtSetKernelTiming": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpExtSetKernelChoice": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int]),
    "mluOpExtSetSparseConvExtendedModes": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpExtSetDistinctPairsPromise": (ctypes.c_int, [_vp, ctypes.c_int]),
    "mluOpExtGetRowMapSize": (ctypes.c_int, [_vp, ctypes.c_int64, ctypes.POINTER(ctypes.c_size_t)]),
    "mluOpExtBuildRowMap": (ctypes.c_int, [_vp, _vp, _vp, ctypes.POINTER(ctypes.c_int64), ctypes.c_int64,
                                           ctypes.c_int64, ctypes.c_int, _vp, ctypes.c_size_t,
                                           ctypes.POINTER(ctypes.c_int64)]),
    "mluOpExtUseRowMap": (ctypes.c_int, [_vp, _vp]),
    "mluOpExtForgetRowMap": (ctypes.c_int, [_vp, _vp]),
    "mluOpExtIndiceConvolutionBackwardFilterNoAlloc": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64p, ctypes.c_int64, ctypes.c_int64, _vp, _vp]),
    "mluOpExtGetKernelTimingCount": (ctypes.c_int, [_vp, _ip]),
    "mluOpExtGetKernelTiming": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p),
                                               ctypes.POINTER(ctypes.c_float)]),
}

_lib = None


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmluops.so is missing (%s): build it with `make -C mlu-ops_amd` or "
                "__graft_entry__.build(); there is no fallback path." % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


class MluOpError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        name = lib().mluOpGetErrorString(status).decode()
        super().__init__("%s returned %s" % (what, name))


def check(status, what="mluOp call"):
    if status != STATUS_SUCCESS:
        raise MluOpError(status, what)


def _int_array(values, ctype=ctypes.c_int):
    values = [int(v) for v in values]
    return (ctype * max(len(values), 1))(*values)


class Handle:
    """mluOpHandle_t bound to the current device; `queue` is a raw hipStream_t."""

    def __init__(self, queue=None):
        self.ptr = _vp()
        check(lib().mluOpCreate(ctypes.byref(self.ptr)), "mluOpCreate")
        if queue is not None:
            self.set_queue(queue)

    def set_queue(self, queue):
        check(lib().mluOpSetQueue(self.ptr, _vp(queue)), "mluOpSetQueue")

    def set_kernel_timing(self, enable):
        check(lib().mluOpExtSetKernelTiming(self.ptr, 1 if enable else 0))

    KERNEL_CHOICES = {"gather_simt": 0, "dense_tiles": 1, "wave_per_tile": 2, "flat_slice_sum": 3,
                      "flat_scatter": 4, "small_map_chunks": 5, "filter_stores": 6,
                      "lists_on_trust": 7}   # mluOpExtKernelChoice_t

    def set_kernel_choice(self, which, value):
        """mluOpExtSetKernelChoice: value None (the shape decides), False or True."""
        v = -1 if value is None else (1 if value else 0)
        check(lib().mluOpExtSetKernelChoice(self.ptr, self.KERNEL_CHOICES[which], v), "mluOpExtSetKernelChoice")

    def set_extended_modes(self, enable):
        """Accept inverse = 1 and tagged filters_grad layouts, which the reference rejects."""
        check(lib().mluOpExtSetSparseConvExtendedModes(self.ptr, 1 if enable else 0))

    def promise_distinct_pairs(self, promised):
        """No offset of the rulebooks names a result row twice: skip the check for lost pairs."""
        check(lib().mluOpExtSetDistinctPairsPromise(self.ptr, 1 if promised else 0))

    def kernel_timings(self):
        """[(kernel name, milliseconds)] per launch since timing was enabled (waits for the queue)."""
        n = ctypes.c_int(0)
        check(lib().mluOpExtGetKernelTimingCount(self.ptr, ctypes.byref(n)))
        out = []
        name = ctypes.c_char_p()
        ms = ctypes.c_float(0)
        for i in range(n.value):
            check(lib().mluOpExtGetKernelTiming(self.ptr, i, ctypes.byref(name), ctypes.byref(ms)))
            out.append((name.value.decode(), ms.value))
        return out

    def close(self):
        if self.ptr:
            lib().mluOpDestroy(self.ptr)
            self.ptr = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class TensorDescriptor:
    def __init__(self, layout, dtype, dims, onchip_dtype=None):
        self.ptr = _vp()
        check(lib().mluOpCreateTensorDescriptor(ctypes.byref(self.ptr)))
        dims = list(dims)
        check(lib().mluOpSetTensorDescriptor(self.ptr, layout, dtype, len(dims), _int_array(dims)),
              "mluOpSetTensorDescriptor")
        if onchip_dtype is not None:
            check(lib().mluOpSetTensorDescriptorOnchipDataType(self.ptr, onchip_dtype))
        self.dims = dims
        self.dtype = dtype
        self.layout = layout

    def close(self):
        if self.ptr:
            lib().mluOpDestroyTensorDescriptor(self.ptr)
            self.ptr = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_descriptors = {}


def _descriptor(layout, dtype, dims, onchip_dtype=None):
    """A tensor descriptor for the operator wrappers below, shared by every call of the same
    (layout, dtype, dims): a layer's calls repeat their shapes, and creating and setting a
    descriptor through ctypes costs more host time than the operator's own launch code."""
    key = (layout, dtype, tuple(int(d) for d in dims), onchip_dtype)
    d = _descriptors.get(key)
    if d is None:
        if len(_descriptors) >= 1024:
            _descriptors.clear()   # (descriptors in use are kept alive by their callers)
        d = _descriptors[key] = TensorDescriptor(layout, dtype, list(key[2]), onchip_dtype)
    return d


class SparseConvDescriptor:
    def __init__(self, batch, pad, stride, dilation, input_space, filter_space, output_space,
                 sub_m, transpose=0, inverse=0, dim_nb=5):
        self.ptr = _vp()
        check(lib().mluOpCreateSparseConvolutionDescriptor(ctypes.byref(self.ptr)))
        check(lib().mluOpSetSparseConvolutionDescriptor(
            self.ptr, dim_nb, batch, _int_array(pad), _int_array(stride), _int_array(dilation),
            _int_array(input_space), _int_array(filter_space), _int_array(output_space),
            int(sub_m), int(transpose), int(inverse)), "mluOpSetSparseConvolutionDescriptor")

    def num_act_out(self):
        n = ctypes.c_int(0)
        check(lib().mluOpGetSparseConvolutionNumActOut(self.ptr, ctypes.byref(n)))
        return n.value

    def close(self):
        if self.ptr:
            lib().mluOpDestroySparseConvolutionDescriptor(self.ptr)
            self.ptr = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def regular_output_space(input_space, filter_space, pad, stride, dilation):
    """Output extent of a regular convolution per axis (the caller supplies it to the API)."""
    return [(i + 2 * p - d * (k - 1) - 1) // s + 1
            for i, k, p, s, d in zip(input_space, filter_space, pad, stride, dilation)]


# ---------------------------------------------------------------------------
# torch-facing convenience layer (device memory and stream only)
# ---------------------------------------------------------------------------

def _torch():
    import torch
    return torch


def torch_dtype_code(dtype):
    torch = _torch()
    return {torch.float16: DTYPE_HALF, torch.float32: DTYPE_FLOAT, torch.bfloat16: DTYPE_BFLOAT16,
            torch.int32: DTYPE_INT32}[dtype]


def make_handle_on_current_stream():
    torch = _torch()
    return Handle(queue=torch.cuda.current_stream().cuda_stream)


# Guard bands for tests (the reference's test runner does the same around every device buffer,
# pb_gtest/src/runtime.cpp:99-145): with GUARD_BYTES > 0 every output tensor and workspace these
# wrappers allocate sits between two bands of GUARD_BYTES bytes holding GUARD_PATTERN, and after
# every operator call the wrappers wait for the queue and raise if a band has changed.
GUARD_BYTES = 0
GUARD_PATTERN = 0xA5
_guard_state = threading.local()   # .bands: (whole buffer, payload bytes, what) of this thread's next call


def _bands():
    if not hasattr(_guard_state, "bands"):
        _guard_state.bands = []
    return _guard_state.bands


def _capturing():
    """Inside a stream capture nothing runs, so bands could be neither filled nor checked."""
    torch = _torch()
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def _guarded_bytes(nbytes, device, what):
    torch = _torch()
    nbytes = int(nbytes)
    if GUARD_BYTES <= 0 or _capturing():
        return torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=device)
    whole = torch.empty((nbytes + 2 * GUARD_BYTES,), dtype=torch.uint8, device=device)
    whole[:GUARD_BYTES] = GUARD_PATTERN
    whole[GUARD_BYTES + nbytes:] = GUARD_PATTERN
    _bands().append((whole, nbytes, what))
    return whole[GUARD_BYTES:GUARD_BYTES + max(nbytes, 1)]


# Tests of workspaces the caller did not align: every workspace starts this many bytes behind
# an aligned address.
WORKSPACE_SKEW = 0


def _workspace(nbytes, device):
    if WORKSPACE_SKEW:
        return _guarded_bytes(int(nbytes) + WORKSPACE_SKEW, device, "workspace")[WORKSPACE_SKEW:]
    return _guarded_bytes(nbytes, device, "workspace")


def _output(shape, dtype, device, what, fill=None):
    """An output tensor of the operator `what` is about to write (between guard bands in guard mode)."""
    torch = _torch()
    shape = tuple(int(v) for v in shape)
    if GUARD_BYTES <= 0 or _capturing():
        if fill is None:
            return torch.empty(shape, dtype=dtype, device=device)
        return torch.full(shape, fill, dtype=dtype, device=device)
    n = 1
    for v in shape:
        n *= v
    item = torch.empty((), dtype=dtype).element_size()
    raw = _guarded_bytes(n * item, device, what)
    t = raw[:n * item].view(dtype).view(shape)
    if fill is not None:
        t.fill_(fill)
    return t


def _guards_intact(call):
    """After operator `call`: in guard mode, waits for the GPU and checks every band allocated for it."""
    bands = _bands()
    if not bands:
        return
    torch = _torch()
    if torch.cuda.is_available():
        torch.cuda.synchronize()
    bad = []
    for whole, nbytes, what in bands:
        front = whole[:GUARD_BYTES]
        back = whole[GUARD_BYTES + nbytes:]
        if not bool((front == GUARD_PATTERN).all()):
            bad.append("%s: bytes in front of it were written" % what)
        if not bool((back == GUARD_PATTERN).all()):
            bad.append("%s: bytes behind it were written" % what)
    del bands[:]
    if bad:
        raise AssertionError("%s wrote outside its buffers: %s" % (call, "; ".join(bad)))


def get_indice_pairs(handle, indices, batch, input_space, filter_space, output_space, pad, stride,
                     dilation, sub_m, out_rows=None, out_indices=None):
    """Builds the rulebook for `indices` (int32 [L, 4] device tensor).

    Returns (indice_pairs [K,2,L], out_indices [out_rows,4], indice_num [K] device int32,
    num_act_out).  In submanifold mode num_act_out is L.  Rows of out_indices from
    num_act_out on are -1: this wrapper allocates the tensor that way, the operator leaves
    them alone (the reference decodes num_act_out rows, normal_get_indice_pairs.cpp:1143-1150)."""
    torch = _torch()
    L = indices.shape[0]
    K = 1
    for k in filter_space:
        K *= int(k)
    if out_rows is None:
        if sub_m:
            out_rows = L
        else:
            vol = batch
            for o in output_space:
                vol *= int(o)
            out_rows = min(vol, K * L)
    dev = indices.device
    pairs = _output((K, 2, L), torch.int32, dev, "indice_pairs")
    # the operator writes the first num_act_out rows only; the rest keep this initial -1
    if out_indices is None:
        out_indices = _output((out_rows, 4), torch.int32, dev, "out_indices", fill=-1)
    else:
        out_rows = out_indices.shape[0]
    indice_num = _output((K,), torch.int32, dev, "indice_num")
    desc = SparseConvDescriptor(batch, pad, stride, dilation, input_space, filter_space,
                                output_space, sub_m)
    d_in = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [L, 4])
    d_pairs = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K, 2, L])
    d_out = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [out_rows, 4])
    d_num = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K])
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetIndicePairsWorkspaceSize(handle.ptr, desc.ptr, d_in.ptr, d_pairs.ptr,
                                                 d_out.ptr, d_num.ptr, ctypes.byref(size)),
          "mluOpGetIndicePairsWorkspaceSize")
    ws = _workspace(size.value, dev)
    check(lib().mluOpGetIndicePairs(handle.ptr, desc.ptr, d_in.ptr, indices.data_ptr(),
                                    ws.data_ptr(), size.value, d_pairs.ptr, pairs.data_ptr(),
                                    d_out.ptr, out_indices.data_ptr(), d_num.ptr,
                                    indice_num.data_ptr()), "mluOpGetIndicePairs")
    _guards_intact("mluOpGetIndicePairs")
    num_act_out = L if sub_m else desc.num_act_out()
    return pairs, out_indices, indice_num, num_act_out


def _host_counts(indice_num):
    vals = [int(v) for v in indice_num]
    return (ctypes.c_int64 * max(len(vals), 1))(*vals)


class RowMap:
    """A [K, rows] row map built once for a rulebook and one direction (mluOpExtBuildRowMap):
    `buffer` is the device memory, `lost_pairs` how many pairs found no slot of their own (a map
    with lost pairs is not recorded by the library and `usable` is False)."""

    def __init__(self, handle, indice_pairs, indice_num_host, rows, source_rows, row_column, verify=True):
        """verify=False (needs the handle's distinct-pairs promise) skips the count of lost pairs and
        the wait for the queue that reads it."""
        torch = _torch()
        K, _, L = indice_pairs.shape
        d_pairs = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K, 2, L])
        size = ctypes.c_size_t(0)
        check(lib().mluOpExtGetRowMapSize(d_pairs.ptr, int(rows), ctypes.byref(size)), "mluOpExtGetRowMapSize")
        self.handle = handle
        self.pairs = indice_pairs          # the map is valid for this tensor only: keep it alive
        self.buffer = _guarded_bytes(size.value, indice_pairs.device, "row map")
        lost = ctypes.c_int64(0)
        check(lib().mluOpExtBuildRowMap(handle.ptr, d_pairs.ptr, indice_pairs.data_ptr(),
                                        _host_counts(indice_num_host), int(rows), int(source_rows),
                                        int(row_column), self.buffer.data_ptr(), size.value,
                                        ctypes.byref(lost) if verify else None),
              "mluOpExtBuildRowMap")
        _guards_intact("mluOpExtBuildRowMap")
        self.lost_pairs = int(lost.value) if verify else None
        self.usable = not verify or self.lost_pairs == 0

    def announce(self):
        """The next forward / backward-data call on the handle uses this map."""
        check(lib().mluOpExtUseRowMap(self.handle.ptr, self.buffer.data_ptr()), "mluOpExtUseRowMap")

    def close(self):
        if self.buffer is not None and self.handle.ptr:
            lib().mluOpExtForgetRowMap(self.handle.ptr, self.buffer.data_ptr())
        self.buffer = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def indice_conv_forward(handle, features, filters, filters_layout, indice_pairs, indice_num_host,
                        num_act_out, sub_m, inverse=0, row_map=None):
    """features [L,Ci], filters 5-D in `filters_layout`, indice_num_host: K python ints.
    `row_map`: a usable RowMap built for this pair tensor and direction."""
    torch = _torch()
    code = torch_dtype_code(features.dtype)
    K, _, L = indice_pairs.shape
    if filters_layout == LAYOUT_ARRAY:
        co = filters.shape[4]
    else:
        co = filters.shape[0]
    out = _output((num_act_out, co), features.dtype, features.device, "features_out")
    d_feat = _descriptor(LAYOUT_ARRAY, code, list(features.shape))
    d_filt = _descriptor(filters_layout, code, list(filters.shape))
    d_pairs = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K, 2, L])
    d_out = _descriptor(LAYOUT_ARRAY, code, [num_act_out, co])
    counts = _host_counts(indice_num_host)
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetIndiceConvolutionForwardWorkspaceSize(
        handle.ptr, d_feat.ptr, d_filt.ptr, d_pairs.ptr, d_out.ptr, counts, num_act_out, inverse,
        int(sub_m), ctypes.byref(size)), "mluOpGetIndiceConvolutionForwardWorkspaceSize")
    ws = _workspace(size.value, features.device)
    if row_map is not None:
        row_map.announce()
    check(lib().mluOpIndiceConvolutionForward(
        handle.ptr, d_feat.ptr, features.data_ptr(), d_filt.ptr, filters.data_ptr(), d_pairs.ptr,
        indice_pairs.data_ptr(), counts, num_act_out, inverse, int(sub_m), ws.data_ptr(),
        size.value, d_out.ptr, out.data_ptr()), "mluOpIndiceConvolutionForward")
    _guards_intact("mluOpIndiceConvolutionForward")
    return out


def indice_conv_backward_data(handle, output_grad, filters, filters_layout, indice_pairs,
                              indice_num_host, sub_m, ci, inverse=0, rows=None, row_map=None):
    """input_grad [rows, ci]; rows = indice_pairs.shape[2] unless the convolution is an inverse one."""
    torch = _torch()
    code = torch_dtype_code(output_grad.dtype)
    K, _, L = indice_pairs.shape
    rows = L if rows is None else int(rows)
    dx = _output((rows, ci), output_grad.dtype, output_grad.device, "input_grad")
    d_dy = _descriptor(LAYOUT_ARRAY, code, list(output_grad.shape))
    d_filt = _descriptor(filters_layout, code, list(filters.shape))
    d_pairs = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K, 2, L])
    d_dx = _descriptor(LAYOUT_ARRAY, code, [rows, ci])
    counts = _host_counts(indice_num_host)
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(
        handle.ptr, d_dy.ptr, d_filt.ptr, d_pairs.ptr, d_dx.ptr, counts, inverse,
        ctypes.byref(size)), "mluOpGetIndiceConvolutionBackwardDataWorkspaceSize")
    ws = _workspace(size.value, output_grad.device)
    if row_map is not None:
        row_map.announce()
    check(lib().mluOpIndiceConvolutionBackwardData(
        handle.ptr, d_dy.ptr, output_grad.data_ptr(), d_filt.ptr, filters.data_ptr(), d_pairs.ptr,
        indice_pairs.data_ptr(), counts, inverse, int(sub_m), ws.data_ptr(), size.value, d_dx.ptr,
        dx.data_ptr()), "mluOpIndiceConvolutionBackwardData")
    _guards_intact("mluOpIndiceConvolutionBackwardData")
    return dx


def indice_conv_backward_filter(handle, features, output_grad, indice_pairs, indice_num_host,
                                filter_space, sub_m, inverse=0, onchip_float=True,
                                grad_layout=LAYOUT_ARRAY):
    """Returns filters_grad laid out [kd, kh, kw, Ci, Co]; with the handle's extended modes on,
    grad_layout NDHWC gives [Co, kd, kh, kw, Ci] and NCDHW [Co, Ci, kd, kh, kw]."""
    torch = _torch()
    code = torch_dtype_code(features.dtype)
    K, _, L = indice_pairs.shape
    ci, co = features.shape[1], output_grad.shape[1]
    if grad_layout in (LAYOUT_NDHWC, LAYOUT_NHWC):
        shape = (co,) + tuple(filter_space) + (ci,)
    elif grad_layout in (LAYOUT_NCDHW, LAYOUT_NCHW):
        shape = (co, ci) + tuple(filter_space)
    else:
        shape = tuple(filter_space) + (ci, co)
    dw = _output(shape, features.dtype, features.device, "filters_grad")
    d_x = _descriptor(LAYOUT_ARRAY, code, list(features.shape))
    d_dy = _descriptor(LAYOUT_ARRAY, code, list(output_grad.shape))
    d_pairs = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K, 2, L])
    d_dw = _descriptor(grad_layout, code, list(dw.shape),
                            onchip_dtype=DTYPE_FLOAT if onchip_float else None)
    counts = _host_counts(indice_num_host)
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(
        handle.ptr, d_x.ptr, d_dy.ptr, d_pairs.ptr, d_dw.ptr, counts, inverse, int(sub_m),
        ctypes.byref(size)), "mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize")
    ws = _workspace(size.value, features.device)
    check(lib().mluOpIndiceConvolutionBackwardFilter(
        handle.ptr, d_x.ptr, features.data_ptr(), d_dy.ptr, output_grad.data_ptr(), d_pairs.ptr,
        indice_pairs.data_ptr(), counts, inverse, int(sub_m), ws.data_ptr(), size.value, d_dw.ptr,
        dw.data_ptr()), "mluOpIndiceConvolutionBackwardFilter")
    _guards_intact("mluOpIndiceConvolutionBackwardFilter")
    return dw


NO_ALLOC_SCRATCH_BYTES = 16 * 1024 * 1024  # MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES


def indice_conv_backward_filter_no_alloc(handle, features, output_grad, indice_pairs, indice_num_host,
                                         filter_space, sub_m, filters_grad, inverse=0,
                                         onchip_float=True):
    """mluOpExtIndiceConvolutionBackwardFilterNoAlloc into the caller's `filters_grad`
    ([kd, kh, kw, Ci, Co]): no workspace, the library's own scratch array instead."""
    code = torch_dtype_code(features.dtype)
    K, _, L = indice_pairs.shape
    d_x = _descriptor(LAYOUT_ARRAY, code, list(features.shape))
    d_dy = _descriptor(LAYOUT_ARRAY, code, list(output_grad.shape))
    d_pairs = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [K, 2, L])
    d_dw = _descriptor(LAYOUT_ARRAY, code, list(filters_grad.shape),
                            onchip_dtype=DTYPE_FLOAT if onchip_float else None)
    check(lib().mluOpExtIndiceConvolutionBackwardFilterNoAlloc(
        handle.ptr, d_x.ptr, features.data_ptr(), d_dy.ptr, output_grad.data_ptr(), d_pairs.ptr,
        indice_pairs.data_ptr(), _host_counts(indice_num_host), inverse, int(sub_m), d_dw.ptr,
        filters_grad.data_ptr()), "mluOpExtIndiceConvolutionBackwardFilterNoAlloc")
    _guards_intact("mluOpExtIndiceConvolutionBackwardFilterNoAlloc")
    return filters_grad


def voxelization(handle, points, voxel_size, coors_range, max_points, max_voxels, deterministic=True):
    """Hard voxelization of `points` [N, F] (float32 device tensor; x, y, z first).

    voxel_size [3] and coors_range [6] are float32 device tensors.  Returns (voxels
    [max_voxels, max_points, F], coors [max_voxels, 3] int32 (z, y, x), num_points_per_voxel
    [max_voxels] int32, voxel_num [1] int32), all on the device."""
    torch = _torch()
    n, f = points.shape
    dev = points.device
    voxels = _output((max_voxels, max_points, f), torch.float32, dev, "voxels")
    coors = _output((max_voxels, 3), torch.int32, dev, "coors")
    npv = _output((max_voxels,), torch.int32, dev, "num_points_per_voxel")
    voxel_num = torch.zeros((1,), dtype=torch.int32, device=dev)
    d_points = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [n, f])
    d_vs = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [3])
    d_cr = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [6])
    d_voxels = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [max_voxels, max_points, f])
    d_coors = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [max_voxels, 3])
    d_npv = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [max_voxels])
    d_num = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [1])
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetVoxelizationWorkspaceSize(
        handle.ptr, d_points.ptr, d_vs.ptr, d_cr.ptr, max_points, max_voxels, 3, bool(deterministic),
        d_voxels.ptr, d_coors.ptr, d_npv.ptr, d_num.ptr, ctypes.byref(size)),
        "mluOpGetVoxelizationWorkspaceSize")
    ws = _workspace(size.value, dev)
    check(lib().mluOpVoxelization(
        handle.ptr, d_points.ptr, points.data_ptr(), d_vs.ptr, voxel_size.data_ptr(), d_cr.ptr,
        coors_range.data_ptr(), max_points, max_voxels, 3, bool(deterministic), ws.data_ptr(), size.value,
        d_voxels.ptr, voxels.data_ptr(), d_coors.ptr, coors.data_ptr(), d_npv.ptr, npv.data_ptr(), d_num.ptr,
        voxel_num.data_ptr()), "mluOpVoxelization")
    _guards_intact("mluOpVoxelization")
    return voxels, coors, npv, voxel_num


def dynamic_point_to_voxel_forward(handle, feats, coors, reduce_type="max", rows=None):
    """Groups points by coordinate triple and reduces their features ("max" or "mean").

    feats [N, C] float32 and coors [N, 3] int32 are device tensors; coors is modified in place
    (rows with a negative coordinate become -1,-1,-1).  Returns (voxel_feats [rows, C], voxel_coors
    [rows, 3], point2voxel_map [N], voxel_points_count [rows], voxel_num [1]); rows defaults to N."""
    torch = _torch()
    n, c = feats.shape
    m = n if rows is None else int(rows)
    dev = feats.device
    voxel_feats = _output((m, c), torch.float32, dev, "voxel_feats")
    voxel_coors = _output((m, 3), torch.int32, dev, "voxel_coors")
    p2v = _output((n,), torch.int32, dev, "point2voxel_map")
    count = _output((m,), torch.int32, dev, "voxel_points_count")
    voxel_num = torch.zeros((1,), dtype=torch.int32, device=dev)
    mode = {"max": REDUCE_DMAX, "mean": REDUCE_DMEAN, "sum": REDUCE_DSUM}[reduce_type]
    d_feats = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [n, c])
    d_coors = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [n, 3])
    d_vf = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [m, c])
    d_vc = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [m, 3])
    d_p2v = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [n])
    d_cnt = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [m])
    d_num = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [1])
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetDynamicPointToVoxelForwardWorkspaceSize(handle.ptr, d_feats.ptr, d_coors.ptr,
                                                                ctypes.byref(size)),
          "mluOpGetDynamicPointToVoxelForwardWorkspaceSize")
    ws = _workspace(size.value, dev)
    check(lib().mluOpDynamicPointToVoxelForward(
        handle.ptr, mode, d_feats.ptr, feats.data_ptr(), d_coors.ptr, coors.data_ptr(), ws.data_ptr(),
        size.value, d_vf.ptr, voxel_feats.data_ptr(), d_vc.ptr, voxel_coors.data_ptr(), d_p2v.ptr,
        p2v.data_ptr(), d_cnt.ptr, count.data_ptr(), d_num.ptr, voxel_num.data_ptr()),
        "mluOpDynamicPointToVoxelForward")
    _guards_intact("mluOpDynamicPointToVoxelForward")
    return voxel_feats, voxel_coors, p2v, count, voxel_num


def dynamic_point_to_voxel_backward(handle, grad_voxel_feats, feats, voxel_feats, point2voxel_map,
                                    voxel_points_count, voxel_num, reduce_type="max"):
    """Gradient of `dynamic_point_to_voxel_forward(..., "max")` with respect to feats: [N, C]."""
    torch = _torch()
    n, c = feats.shape
    m = grad_voxel_feats.shape[0]
    grad_feats = _output((n, c), torch.float32, feats.device, "grad_feats")
    mode = {"max": REDUCE_DMAX, "mean": REDUCE_DMEAN, "sum": REDUCE_DSUM}[reduce_type]
    d_g = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [m, c])
    d_feats = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [n, c])
    d_vf = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [m, c])
    d_p2v = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [n])
    d_cnt = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [m])
    d_num = _descriptor(LAYOUT_ARRAY, DTYPE_INT32, [1])
    d_out = _descriptor(LAYOUT_ARRAY, DTYPE_FLOAT, [n, c])
    size = ctypes.c_size_t(0)
    check(lib().mluOpGetDynamicPointToVoxelBackwardWorkspaceSize(
        handle.ptr, mode, d_g.ptr, d_feats.ptr, d_vf.ptr, d_p2v.ptr, d_cnt.ptr, d_num.ptr, ctypes.byref(size)),
        "mluOpGetDynamicPointToVoxelBackwardWorkspaceSize")
    ws = _workspace(size.value, feats.device)
    check(lib().mluOpDynamicPointToVoxelBackward(
        handle.ptr, mode, d_g.ptr, grad_voxel_feats.data_ptr(), d_feats.ptr, feats.data_ptr(), d_vf.ptr,
        voxel_feats.data_ptr(), d_p2v.ptr, point2voxel_map.data_ptr(), d_cnt.ptr,
        voxel_points_count.data_ptr(), d_num.ptr, voxel_num.data_ptr(), ws.data_ptr(), size.value, d_out.ptr,
        grad_feats.data_ptr()), "mluOpDynamicPointToVoxelBackward")
    _guards_intact("mluOpDynamicPointToVoxelBackward")
    return grad_feats
