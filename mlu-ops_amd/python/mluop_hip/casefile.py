"""Test-case files in the reference's prototxt form, for the four sparse-convolution operators
and the three operators upstream of them (voxelization, dynamic point-to-voxel forward/backward).

The reference's gtest replays one operator call per case file: a protobuf `Node` in text format
with `op_name`, `input {}` / `output {}` tensors (id, shape.dims, layout, dtype, and the values as
`value_i` / `value_l` / `value_f` / `value_h` lists, a `random_data {}` recipe or a binary `path`),
one `<op>_param {}` message and `test_param { error_func, error_threshold, baseline_device }`
(sample: test/mlu_op_gtest/pb_gtest/tests/parser_test.prototxt; the readers:
test/mlu_op_gtest/pb_gtest/src/parser.cpp:100-162 for test_param, :373-397 for the value kinds,
:727-745 for the hex strings of value_h).  The schema itself (mlu_op_test.proto) lives in a git
submodule the reference tree does not vendor, so this module reads and writes the text format
without a schema and takes the field names from the executors that consume them:

  get_indice_pairs_param { dimnb batch pad[] stride[] dilation[] input_space[] filter_space[]
      output_space[] sub_m transpose inverse }   (pb_gtest/src/zoo/get_indice_pairs/get_indice_pairs.cpp:59-80)
      tensors: input indices; outputs out_indices, indice_pairs, indice_num           (:55-58)
  indice_convolution_forward_param { indice_num[] num_active_out sub_m inverse }
      (zoo/indice_convolution_forward/indice_convolution_forward.cpp:33-39)
      tensors: inputs features, filters, indice_pairs; output features_out            (:29-32)
  indice_convolution_backward_data_param { indice_num[] sub_m inverse }
      (zoo/indice_convolution_backward_data/indice_convolution_backward_data.cpp:76-121)
      tensors: inputs output_grad, filters, indice_pairs; output input_grad           (:111-114)
  indice_convolution_backward_param { indice_num[] sub_m inverse }
      (zoo/indice_convolution_backward_filter/indice_convolution_backward_filter.cpp:37-42)
      tensors: inputs features, output_grad, indice_pairs; output filters_grad
  voxelization_param { max_points max_voxels ndim deterministic }   (zoo/voxelization/voxelization.cpp:47-54)
      tensors: inputs points, voxel_size, coors_range; outputs voxels, coors,
      num_points_per_voxel, voxel_num                                                 (:62-90)
  dynamic_point_to_voxel_forward_param { reduce_type: REDUCE_MODE_MAX | REDUCE_MODE_MEAN }
      (zoo/dynamic_point_to_voxel_forward/dynamic_point_to_voxel_forward.cpp:60-70)
      tensors: inputs feats, coors; outputs voxel_feats, voxel_coors, point2voxel_map,
      voxel_points_count, voxel_num                                                   (:71-85)
  dynamic_point_to_voxel_backward_param { reduce_type }
      (zoo/dynamic_point_to_voxel_backward/dynamic_point_to_voxel_backward.cpp:44-47)
      tensors: inputs grad_voxel_feats, feats, voxel_feats, point2voxel_map, voxel_points_count,
      voxel_num; output grad_feats

A tensor may list fewer values than its shape has elements (the reference's own backward case
does): the parser takes the element count from the value list and warns (parser.cpp:371-383), the
rest of the buffer stays zero, and so it does here.

`random_data` tensors are filled by numpy's generator from the recipe's seed and bounds: the
distribution is the recipe's, the bit stream is not the reference generator's, so a case whose
inputs are random carries no baseline values and is replayed for its status and shapes only.

`replay(path_or_text, handle)` runs a case through the C API on the GPU and returns the outputs
(and, where the case file holds baseline values for them, the error measures test_param names)."""
import os
import re

import numpy as np

from . import (DTYPE_BFLOAT16, DTYPE_FLOAT, DTYPE_HALF, DTYPE_INT32, LAYOUT_ARRAY, LAYOUT_NCDHW,
               LAYOUT_NDHWC, LAYOUT_HWCN, LAYOUT_NCHW, LAYOUT_NHWC)

# ---------------------------------------------------------------------------
# protobuf text format, schema-less: a message is a list of (name, value) in file order, a value is
# a python int / float / str (quoted string), an `Enum` (bare identifier) or a nested message
# ---------------------------------------------------------------------------


class Enum(str):
    """A bare identifier in the text format (enum value or true/false)."""


class Message(list):
    """Ordered (name, value) fields; repeated fields simply occur more than once."""

    def get(self, name, default=None):
        for n, v in self:
            if n == name:
                return v
        return default

    def all(self, name):
        return [v for n, v in self if n == name]

    def has(self, name):
        return any(n == name for n, _ in self)

    def add(self, name, value):
        self.append((name, value))
        return self


_TOKEN = re.compile(r"""
    \s+ | \#[^\n]* |
    (?P<str>"(?:[^"\\]|\\.)*"|'(?:[^'\\]|\\.)*') |
    (?P<punct>[{}:<>\[\],;]) |
    (?P<word>[^\s{}:<>\[\],;"'#]+)
""", re.VERBOSE)


def _tokens(text):
    pos = 0
    while pos < len(text):
        m = _TOKEN.match(text, pos)
        if m is None:
            raise ValueError("prototxt: cannot read at offset %d: %r" % (pos, text[pos:pos + 20]))
        pos = m.end()
        if m.lastgroup:
            yield m.lastgroup, m.group(m.lastgroup)
    yield "end", ""


_UNESCAPE = {"n": "\n", "t": "\t", "r": "\r", "\\": "\\", '"': '"', "'": "'"}


def _scalar(kind, tok):
    if kind == "str":
        body = tok[1:-1]
        return re.sub(r"\\(.)", lambda m: _UNESCAPE.get(m.group(1), m.group(1)), body)
    try:
        return int(tok, 0)
    except ValueError:
        pass
    for cand in (tok, tok[:-1] if tok[-1:] in "fF" else tok):
        try:
            return float(cand)
        except ValueError:
            pass
    return Enum(tok)


def parse(text):
    """Text format -> Message."""
    toks = list(_tokens(text))
    pos = [0]

    def peek():
        return toks[pos[0]]

    def take():
        t = toks[pos[0]]
        pos[0] += 1
        return t

    def message(closer):
        msg = Message()
        while True:
            kind, tok = take()
            if kind == "end" or (kind == "punct" and tok in "}>"):
                if (tok or None) != closer:
                    raise ValueError("prototxt: unbalanced braces")
                return msg
            if kind == "punct" and tok in ",;":
                continue
            if kind != "word":
                raise ValueError("prototxt: field name expected, got %r" % tok)
            name = tok
            kind, tok = peek()
            if kind == "punct" and tok == ":":
                take()
                kind, tok = peek()
            if kind == "punct" and tok in "{<":
                take()
                msg.append((name, message("}" if tok == "{" else ">")))
            elif kind == "punct" and tok == "[":
                take()
                while True:
                    kind, tok = take()
                    if kind == "punct" and tok == "]":
                        break
                    if kind == "punct" and tok == ",":
                        continue
                    msg.append((name, _scalar(kind, tok)))
            elif kind in ("word", "str"):
                take()
                msg.append((name, _scalar(kind, tok)))
            else:
                raise ValueError("prototxt: value expected after %s" % name)

    return message(None)


def dump(msg, indent=0):
    """Message -> text format (two-space indent, one field per line, as the reference writes it)."""
    pad = "  " * indent
    lines = []
    for name, v in msg:
        if isinstance(v, Message):
            lines.append("%s%s {" % (pad, name))
            lines.append(dump(v, indent + 1))
            lines.append("%s}" % pad)
        elif isinstance(v, Enum):
            lines.append("%s%s: %s" % (pad, name, v))
        elif isinstance(v, str):
            lines.append('%s%s: "%s"' % (pad, name, v.replace("\\", "\\\\").replace('"', '\\"')))
        elif isinstance(v, bool):
            lines.append("%s%s: %s" % (pad, name, "true" if v else "false"))
        elif isinstance(v, float):
            lines.append("%s%s: %s" % (pad, name, repr(v)))
        else:
            lines.append("%s%s: %d" % (pad, name, v))
    return "\n".join(l for l in lines if l != "")


# ---------------------------------------------------------------------------
# tensors
# ---------------------------------------------------------------------------

_DTYPES = {"DTYPE_HALF": ("float16", DTYPE_HALF), "DTYPE_FLOAT": ("float32", DTYPE_FLOAT),
           "DTYPE_INT32": ("int32", DTYPE_INT32), "DTYPE_BFLOAT16": ("bfloat16", DTYPE_BFLOAT16)}
_LAYOUTS = {"LAYOUT_ARRAY": LAYOUT_ARRAY, "LAYOUT_NDHWC": LAYOUT_NDHWC, "LAYOUT_NCDHW": LAYOUT_NCDHW,
            "LAYOUT_NCHW": LAYOUT_NCHW, "LAYOUT_NHWC": LAYOUT_NHWC, "LAYOUT_HWCN": LAYOUT_HWCN}


def _truthy(v):
    return v in (1, True) or (isinstance(v, str) and v.lower() == "true")


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    """Round to nearest even, as the device conversion does."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


class CaseTensor:
    """One `input` / `output` entry: shape, dtype name, layout code and, when the file holds them,
    values as a float32 / int32 array (bfloat16 values are kept as float32)."""

    def __init__(self, msg, base_dir=None):
        self.id = msg.get("id", "")
        shape = msg.get("shape", Message())
        self.shape = [int(d) for d in shape.all("dims")]
        self.dtype_name, self.dtype_code = _DTYPES[str(msg.get("dtype"))]
        self.layout = _LAYOUTS[str(msg.get("layout", "LAYOUT_ARRAY"))]
        onchip = msg.get("onchip_dtype")
        self.onchip_dtype = _DTYPES[str(onchip)][1] if onchip is not None else None
        self.values = self._values(msg, base_dir)

    def count(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def _values(self, msg, base_dir):
        n = self.count()
        int_like = self.dtype_name == "int32"
        for field in ("value_i", "value_l"):
            if msg.has(field):
                vals = np.array(msg.all(field), dtype=np.int64)
                assert vals.size <= n, "%s: %d values for %d elements" % (self.id, vals.size, n)
                if vals.size < n:
                    vals = np.concatenate([vals, np.zeros(n - vals.size, np.int64)])
                if int_like:
                    return vals.astype(np.int32).reshape(self.shape)
                # value_i of a floating tensor holds the elements' bit patterns (parser.cpp:568-578)
                if self.dtype_name == "float32":
                    out = vals.astype(np.int32).view(np.float32)
                elif self.dtype_name == "float16":
                    out = vals.astype(np.int16).view(np.float16).astype(np.float32)
                else:
                    out = bf16_bits_to_f32(vals.astype(np.int16).view(np.uint16))
                return out.reshape(self.shape)
        if msg.has("value_f"):
            vals = np.array(msg.all("value_f"), dtype=np.float32)
            assert vals.size == n
            return vals.reshape(self.shape)
        if msg.has("value_h"):
            # lower-case hex digits of the element's bits, no prefix (parser.cpp:727-745)
            raw = [int(str(h), 16) for h in msg.all("value_h")]
            assert len(raw) == n
            if self.dtype_name == "float16":
                vals = np.array(raw, dtype=np.uint16).view(np.float16).astype(np.float32)
            elif self.dtype_name == "bfloat16":
                vals = bf16_bits_to_f32(np.array(raw, dtype=np.uint16))
            else:
                vals = np.array(raw, dtype=np.uint32).view(np.float32)
            return vals.reshape(self.shape)
        if msg.has("path"):
            path = msg.get("path")
            if base_dir is not None:
                path = os.path.join(base_dir, path)
            np_dtype = {"float16": np.float16, "float32": np.float32, "int32": np.int32,
                        "bfloat16": np.uint16}[self.dtype_name]
            raw = np.fromfile(path, dtype=np_dtype, count=n)
            assert raw.size == n, "%s: %s holds %d of %d elements" % (self.id, path, raw.size, n)
            if self.dtype_name == "bfloat16":
                raw = bf16_bits_to_f32(raw)
            return (raw.astype(np.int32) if int_like else raw.astype(np.float32)).reshape(self.shape)
        if msg.has("random_data"):
            r = msg.get("random_data")
            rng = np.random.default_rng(int(r.get("seed", 0)))
            if str(r.get("distribution", "UNIFORM")) == "GAUSSIAN":
                vals = rng.normal(float(r.get("mu", r.get("mu_double", 0.0))),
                                  float(r.get("sigma", r.get("sigma_double", 1.0))), size=n)
            else:
                lo = float(r.get("lower_bound", r.get("lower_bound_double", 0.0)))
                hi = float(r.get("upper_bound", r.get("upper_bound_double", 1.0)))
                vals = rng.uniform(lo, hi, size=n)
            # integer tensors take the truncated value, as the executors convert the float draw
            # (zoo/get_indice_pairs/get_indice_pairs.cpp:126-131)
            return (np.trunc(vals).astype(np.int32) if int_like else vals.astype(np.float32)).reshape(self.shape)
        return None


def tensor_message(tid, array, dtype_name, layout="LAYOUT_ARRAY", with_values=True, onchip_dtype=None):
    """Builds an `input`/`output` message; float values go out as value_h, integers as value_i."""
    msg = Message()
    msg.add("id", tid)
    shape = Message()
    for d in array.shape:
        shape.add("dims", int(d))
    msg.add("shape", shape)
    msg.add("layout", Enum(layout))
    proto_dtype = {"float16": "DTYPE_HALF", "float32": "DTYPE_FLOAT", "int32": "DTYPE_INT32",
                   "bfloat16": "DTYPE_BFLOAT16"}[dtype_name]
    msg.add("dtype", Enum(proto_dtype))
    if onchip_dtype is not None:
        msg.add("onchip_dtype", Enum(onchip_dtype))
    if with_values:
        flat = np.ascontiguousarray(array).reshape(-1)
        if dtype_name == "int32":
            for v in flat.astype(np.int64):
                msg.add("value_i", int(v))
        elif dtype_name == "float16":
            for v in flat.astype(np.float16).view(np.uint16):
                msg.add("value_h", "%04x" % int(v))
        elif dtype_name == "bfloat16":
            for v in f32_to_bf16_bits(flat):
                msg.add("value_h", "%04x" % int(v))
        else:
            for v in flat.astype(np.float32).view(np.uint32):
                msg.add("value_h", "%08x" % int(v))
    return msg


def _test_param(thresholds):
    tp = Message()
    for name, _ in thresholds:
        tp.add("error_func", Enum(name))
    for _, thr in thresholds:
        tp.add("error_threshold", float(thr))
    tp.add("baseline_device", Enum("CPU"))
    return tp


# ---------------------------------------------------------------------------
# writers: one function per operator
# ---------------------------------------------------------------------------

def get_indice_pairs_case(indices, batch, pad, stride, dilation, input_space, filter_space, output_space,
                          sub_m, baseline=None):
    """`baseline` = (out_indices, indice_pairs, indice_num) arrays to store as expected values."""
    L = indices.shape[0]
    K = int(np.prod(filter_space))
    node = Message()
    node.add("op_name", "get_indice_pairs")
    node.add("input", tensor_message("indices", indices, "int32"))
    outs = baseline if baseline is not None else (np.zeros((L if sub_m else 0, 4), np.int32),
                                                  np.zeros((K, 2, L), np.int32), np.zeros((K,), np.int32))
    for tid, arr in zip(("out_indices", "indice_pairs", "indice_num"), outs):
        node.add("output", tensor_message(tid, arr, "int32", with_values=baseline is not None))
    p = Message()
    p.add("dimnb", 5)
    p.add("batch", int(batch))
    for name, vals in (("pad", pad), ("stride", stride), ("dilation", dilation), ("input_space", input_space),
                       ("filter_space", filter_space), ("output_space", output_space)):
        for v in vals:
            p.add(name, int(v))
    p.add("sub_m", int(bool(sub_m)))
    p.add("transpose", 0)
    p.add("inverse", 0)
    node.add("get_indice_pairs_param", p)
    node.add("test_param", _test_param([("DIFF1", 0.0), ("DIFF2", 0.0)]))
    return node


def _conv_case(op_name, param_name, inputs, output, indice_num, sub_m, threshold, num_active_out=None):
    node = Message()
    node.add("op_name", op_name)
    for m in inputs:
        node.add("input", m)
    node.add("output", output)
    p = Message()
    for v in indice_num:
        p.add("indice_num", int(v))
    if num_active_out is not None:
        p.add("num_active_out", int(num_active_out))
    p.add("sub_m", int(bool(sub_m)))
    p.add("inverse", 0)
    node.add(param_name, p)
    node.add("test_param", _test_param([("DIFF1", threshold), ("DIFF2", threshold)]))
    return node


def indice_convolution_forward_case(features, filters, indice_pairs, indice_num, num_active_out, sub_m,
                                    dtype_name, filters_layout="LAYOUT_ARRAY", baseline=None, threshold=3e-3):
    co = filters.shape[4] if filters_layout == "LAYOUT_ARRAY" else (
        filters.shape[0] if filters_layout in ("LAYOUT_NDHWC", "LAYOUT_NCDHW") else filters.shape[-1])
    out = baseline if baseline is not None else np.zeros((num_active_out, co), np.float32)
    return _conv_case(
        "indice_convolution_forward", "indice_convolution_forward_param",
        [tensor_message("features", features, dtype_name),
         tensor_message("filters", filters, dtype_name, layout=filters_layout),
         tensor_message("indice_pairs", indice_pairs, "int32")],
        tensor_message("features_out", out, dtype_name, with_values=baseline is not None),
        indice_num, sub_m, threshold, num_active_out=num_active_out)


def indice_convolution_backward_data_case(output_grad, filters, indice_pairs, indice_num, n_in, sub_m,
                                          dtype_name, filters_layout="LAYOUT_ARRAY", baseline=None,
                                          threshold=3e-3):
    ci = filters.shape[3] if filters_layout == "LAYOUT_ARRAY" else (
        filters.shape[4] if filters_layout == "LAYOUT_NDHWC" else filters.shape[1])
    out = baseline if baseline is not None else np.zeros((n_in, ci), np.float32)
    return _conv_case(
        "indice_convolution_backward_data", "indice_convolution_backward_data_param",
        [tensor_message("output_grad", output_grad, dtype_name),
         tensor_message("filters", filters, dtype_name, layout=filters_layout),
         tensor_message("indice_pairs", indice_pairs, "int32")],
        tensor_message("input_grad", out, dtype_name, with_values=baseline is not None),
        indice_num, sub_m, threshold)


def indice_convolution_backward_filter_case(features, output_grad, indice_pairs, indice_num, filter_space,
                                            sub_m, dtype_name, baseline=None, threshold=3e-3):
    shape = tuple(filter_space) + (features.shape[1], output_grad.shape[1])
    out = baseline if baseline is not None else np.zeros(shape, np.float32)
    return _conv_case(
        "indice_convolution_backward_filter", "indice_convolution_backward_param",
        [tensor_message("features", features, dtype_name),
         tensor_message("output_grad", output_grad, dtype_name),
         tensor_message("indice_pairs", indice_pairs, "int32")],
        tensor_message("filters_grad", out, dtype_name, with_values=baseline is not None,
                       onchip_dtype="DTYPE_FLOAT"),
        indice_num, sub_m, threshold)


def _upstream_case(op_name, inputs, outputs, param_name, param, baseline, thresholds):
    node = Message()
    node.add("op_name", op_name)
    for tid, arr, dtype_name in inputs:
        node.add("input", tensor_message(tid, arr, dtype_name))
    for tid, arr, dtype_name in outputs:
        node.add("output", tensor_message(tid, arr, dtype_name, with_values=baseline))
    node.add(param_name, param)
    node.add("test_param", _test_param(thresholds))
    return node


def voxelization_case(points, voxel_size, coors_range, max_points, max_voxels, deterministic=True,
                      baseline=None):
    """`baseline` = (voxels, coors, num_points_per_voxel, voxel_num) to store as expected values."""
    f = points.shape[1]
    outs = baseline if baseline is not None else (
        np.zeros((max_voxels, max_points, f), np.float32), np.zeros((max_voxels, 3), np.int32),
        np.zeros((max_voxels,), np.int32), np.zeros((1,), np.int32))
    p = Message()
    p.add("max_points", int(max_points))
    p.add("max_voxels", int(max_voxels))
    p.add("ndim", 3)
    p.add("deterministic", Enum("true" if deterministic else "false"))
    return _upstream_case(
        "voxelization",
        [("points", points, "float32"), ("voxel_size", np.asarray(voxel_size, np.float32), "float32"),
         ("coors_range", np.asarray(coors_range, np.float32), "float32")],
        [("voxels", outs[0], "float32"), ("coors", outs[1], "int32"),
         ("num_points_per_voxel", outs[2], "int32"),
         ("voxel_num", np.asarray(outs[3], np.int32).reshape(1), "int32")],
        "voxelization_param", p, baseline is not None, [("DIFF1", 0.0), ("DIFF2", 0.0)])


def _reduce_param(reduce_type):
    p = Message()
    p.add("reduce_type", Enum({"max": "REDUCE_MODE_MAX", "mean": "REDUCE_MODE_MEAN"}[reduce_type]))
    return p


def dynamic_point_to_voxel_forward_case(feats, coors, reduce_type, baseline=None):
    """`baseline` = (voxel_feats, voxel_coors, point2voxel_map, voxel_points_count, voxel_num)."""
    n, c = feats.shape
    outs = baseline if baseline is not None else (
        np.zeros((n, c), np.float32), np.zeros((n, 3), np.int32), np.zeros((n,), np.int32),
        np.zeros((n,), np.int32), np.zeros((1,), np.int32))
    return _upstream_case(
        "dynamic_point_to_voxel_forward", [("feats", feats, "float32"), ("coors", coors, "int32")],
        [("voxel_feats", outs[0], "float32"), ("voxel_coors", outs[1], "int32"),
         ("point2voxel_map", outs[2], "int32"), ("voxel_points_count", outs[3], "int32"),
         ("voxel_num", np.asarray(outs[4], np.int32).reshape(1), "int32")],
        "dynamic_point_to_voxel_forward_param", _reduce_param(reduce_type), baseline is not None,
        [("DIFF1", 0.0), ("DIFF2", 0.0)])


def dynamic_point_to_voxel_backward_case(grad_voxel_feats, feats, voxel_feats, point2voxel_map,
                                         voxel_points_count, voxel_num, reduce_type="max", baseline=None):
    """`baseline` = grad_feats to store as the expected values."""
    out = baseline if baseline is not None else np.zeros(feats.shape, np.float32)
    return _upstream_case(
        "dynamic_point_to_voxel_backward",
        [("grad_voxel_feats", grad_voxel_feats, "float32"), ("feats", feats, "float32"),
         ("voxel_feats", voxel_feats, "float32"), ("point2voxel_map", point2voxel_map, "int32"),
         ("voxel_points_count", voxel_points_count, "int32"),
         ("voxel_num", np.asarray(voxel_num, np.int32).reshape(1), "int32")],
        [("grad_feats", out, "float32")],
        "dynamic_point_to_voxel_backward_param", _reduce_param(reduce_type), baseline is not None,
        [("DIFF1", 0.0), ("DIFF2", 0.0)])


# ---------------------------------------------------------------------------
# replay
# ---------------------------------------------------------------------------

def diff1(got, want):
    """sum|got - want| / sum|want| (evaluator.cpp: DIFF1)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    den = np.abs(want).sum()
    num = np.abs(got - want).sum()
    return num / den if den > 0 else num


def diff2(got, want):
    """sqrt(sum (got - want)^2 / sum want^2) (evaluator.cpp: DIFF2)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    den = (want ** 2).sum()
    num = ((got - want) ** 2).sum()
    return float(np.sqrt(num / den)) if den > 0 else float(np.sqrt(num))


def diff3(got, want, dtype_name="float32"):
    """Largest relative error; the absolute error where |want| is below 1e-4 (half) or 1e-6
    (float) (evaluator.h: computeDiff3)."""
    got, want = np.asarray(got, np.float64).reshape(-1), np.asarray(want, np.float64).reshape(-1)
    if got.size == 0:
        return 0.0
    eps = {"float16": 1e-4, "float32": 1e-6}.get(dtype_name, 0.0)
    num, den = np.abs(got - want), np.abs(want)
    return float(np.where(den < eps, num, num / (den + 1e-9)).max())


_ERROR_FUNCS = {"DIFF1": diff1, "DIFF2": diff2, "DIFF3": diff3}


def criteria(node):
    """(error function names, thresholds): `test_param`, or the older node-level
    `evaluation_criterion` / `evaluation_threshold` fields (parser.cpp:129-196)."""
    tp = node.get("test_param")
    if tp is not None and tp.has("error_func"):
        return [str(f) for f in tp.all("error_func")], [float(t) for t in tp.all("error_threshold")]
    return ([str(f) for f in node.all("evaluation_criterion")],
            [float(t) for t in node.all("evaluation_threshold")])


class Replay:
    """Outputs of one replayed case: `outputs` (name -> numpy array), `errors` (list of
    (output name, error_func, value, threshold)) and `passed`."""

    def __init__(self):
        self.outputs = {}
        self.errors = []
        self.passed = True


def _reduce_name(param):
    return {"REDUCE_MODE_MAX": "max", "REDUCE_MODE_MEAN": "mean", "REDUCE_MODE_SUM": "sum"}[
        str(param.get("reduce_type", "REDUCE_MODE_MAX"))]


def load(path_or_text):
    """Returns (Message, base_dir) from a file path or from the text itself."""
    if "\n" not in path_or_text and os.path.exists(path_or_text):
        with open(path_or_text) as f:
            return parse(f.read()), os.path.dirname(os.path.abspath(path_or_text))
    return parse(path_or_text), None


def replay(path_or_text, handle):
    """Runs the case's operator through the C API on the current GPU."""
    import torch
    import mluop_hip as m
    node, base_dir = load(path_or_text)
    op = node.get("op_name")
    ins = [CaseTensor(t, base_dir) for t in node.all("input")]
    outs = [CaseTensor(t, base_dir) for t in node.all("output")]

    def dev(t):
        assert t.values is not None, "case tensor %s carries no values" % t.id
        if t.dtype_name == "int32":
            return torch.from_numpy(np.ascontiguousarray(t.values, dtype=np.int32)).cuda()
        tt = torch.from_numpy(np.ascontiguousarray(t.values, dtype=np.float32)).cuda()
        return tt.to({"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}[t.dtype_name])

    def host(t):
        return t.float().cpu().numpy() if t.dtype != torch.int32 else t.cpu().numpy()

    res = Replay()
    if op == "get_indice_pairs":
        p = node.get("get_indice_pairs_param")
        assert len(ins) == 1 and len(outs) == 3, "get_indice_pairs: 1 input and 3 outputs"
        sub_m = _truthy(p.get("sub_m", 0))
        pairs, out_idx, num, n_out = m.get_indice_pairs(
            handle, dev(ins[0]), int(p.get("batch")), p.all("input_space"), p.all("filter_space"),
            p.all("output_space"), p.all("pad"), p.all("stride"), p.all("dilation"), sub_m,
            out_rows=outs[0].shape[0] if outs[0].shape else None)
        torch.cuda.synchronize()
        # rows of out_indices past num_act_out are not defined by the operator
        oi = host(out_idx)
        oi[n_out:] = 0
        res.outputs = {outs[0].id or "out_indices": oi, outs[1].id or "indice_pairs": host(pairs),
                       outs[2].id or "indice_num": host(num)}
        res.num_act_out = n_out
    elif op in ("indice_convolution_forward", "indice_convolution_backward_data",
                "indice_convolution_backward_filter"):
        pname = {"indice_convolution_forward": "indice_convolution_forward_param",
                 "indice_convolution_backward_data": "indice_convolution_backward_data_param",
                 "indice_convolution_backward_filter": "indice_convolution_backward_param"}[op]
        p = node.get(pname)
        assert p is not None, "%s missing" % pname
        assert len(ins) == 3 and len(outs) == 1, "%s: 3 inputs and 1 output" % op
        num = [int(v) for v in p.all("indice_num")]
        sub_m = _truthy(p.get("sub_m", 0))
        inverse = int(p.get("inverse", 0))
        pairs = dev(ins[2])
        if op == "indice_convolution_forward":
            out = m.indice_conv_forward(handle, dev(ins[0]), dev(ins[1]), ins[1].layout, pairs, num,
                                        int(p.get("num_active_out")), sub_m, inverse)
        elif op == "indice_convolution_backward_data":
            out = m.indice_conv_backward_data(handle, dev(ins[0]), dev(ins[1]), ins[1].layout, pairs, num, sub_m,
                                              outs[0].shape[1], inverse)
        else:
            out = m.indice_conv_backward_filter(handle, dev(ins[0]), dev(ins[1]), pairs, num, outs[0].shape[:-2],
                                                sub_m, inverse, onchip_float=outs[0].onchip_dtype == DTYPE_FLOAT)
        torch.cuda.synchronize()
        res.outputs = {outs[0].id or "output": host(out)}
    elif op == "voxelization":
        p = node.get("voxelization_param")
        assert p is not None, "voxelization_param missing"
        assert len(ins) == 3 and len(outs) == 4, "voxelization: 3 inputs and 4 outputs"
        assert int(p.get("ndim", 3)) == 3, "voxelization: ndim must be 3"
        got = m.voxelization(handle, dev(ins[0]), dev(ins[1]).reshape(-1), dev(ins[2]).reshape(-1),
                             int(p.get("max_points")), int(p.get("max_voxels")),
                             _truthy(p.get("deterministic", 1)))
        torch.cuda.synchronize()
        res.outputs = {t.id or name: host(g) for t, name, g in
                       zip(outs, ("voxels", "coors", "num_points_per_voxel", "voxel_num"), got)}
    elif op == "dynamic_point_to_voxel_forward":
        p = node.get("dynamic_point_to_voxel_forward_param")
        assert p is not None, "dynamic_point_to_voxel_forward_param missing"
        assert len(ins) == 2 and len(outs) == 5, "dynamic_point_to_voxel_forward: 2 inputs and 5 outputs"
        got = m.dynamic_point_to_voxel_forward(handle, dev(ins[0]), dev(ins[1]), _reduce_name(p),
                                               rows=outs[0].shape[0] if outs[0].shape else None)
        torch.cuda.synchronize()
        names = ("voxel_feats", "voxel_coors", "point2voxel_map", "voxel_points_count", "voxel_num")
        arrays = [host(g) for g in got]
        # rows past voxel_num of the per-voxel outputs are not defined by the operator
        res.voxel_num = int(arrays[4][0])
        for a in (arrays[0], arrays[1], arrays[3]):
            a[res.voxel_num:] = 0
        res.outputs = {t.id or name: a for t, name, a in zip(outs, names, arrays)}
    elif op == "dynamic_point_to_voxel_backward":
        p = node.get("dynamic_point_to_voxel_backward_param")
        assert p is not None, "dynamic_point_to_voxel_backward_param missing"
        assert len(ins) == 6 and len(outs) == 1, "dynamic_point_to_voxel_backward: 6 inputs and 1 output"
        got = m.dynamic_point_to_voxel_backward(handle, *[dev(t) for t in ins], reduce_type=_reduce_name(p))
        torch.cuda.synchronize()
        res.outputs = {outs[0].id or "grad_feats": host(got)}
    else:
        raise ValueError("case file names operator %r, which is not built" % op)

    funcs, thresholds = criteria(node)
    for i, t in enumerate(outs):
        if t.values is None:
            continue
        got = res.outputs[t.id] if t.id in res.outputs else list(res.outputs.values())[i]
        want = t.values
        if op == "get_indice_pairs" and t is outs[0]:
            want = want.copy()
            want[res.num_act_out:] = 0
        if op == "dynamic_point_to_voxel_forward" and i in (0, 1, 3):
            want = want.copy()
            want[res.voxel_num:] = 0
        for f, thr in zip(funcs, thresholds):
            if f not in _ERROR_FUNCS:
                continue
            e = diff3(got, want, t.dtype_name) if f == "DIFF3" else _ERROR_FUNCS[f](got, want)
            res.errors.append((t.id, f, float(e), thr))
            if not e <= thr:
                res.passed = False
    return res
