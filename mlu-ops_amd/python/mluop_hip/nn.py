"""PyTorch caller layer over the C API: the call sequence mmcv's sparse-conv ops run against
mlu-ops (descriptor -> workspace size -> mluOpGetIndicePairs -> num_act_out -> device-to-host
copy of indice_num -> the three indice-convolution operators), wrapped in an autograd function and
the modules `SubMConv3d`, `SparseConv3d` and `SparseInverseConv3d` (the last one through the
library's extended modes, which the reference does not have).

A `SparseTensor` carries features [L, C], int32 indices [L, 4] = (n, d, h, w), the spatial shape
and the batch size, plus a cache of rulebooks keyed by `indice_key`, so that stacked submanifold
layers with the same key build the rulebook once (the reference design's layer chain,
docs/design_docs/indice_convolution_forward/indice_convolution_forward.md:229-234).

torch is used for device memory, the stream and the autograd graph only; every number is computed
by libmluops.so.  Weights are stored [kd, kh, kw, Ci, Co] (LAYOUT_ARRAY), the one layout all three
operators accept (indice_convolution_backward_filter.cpp:227-242 in the reference)."""
import math

import torch

from . import (LAYOUT_ARRAY, RowMap, get_indice_pairs, indice_conv_backward_data, indice_conv_backward_filter,
               indice_conv_forward, make_handle_on_current_stream, regular_output_space, voxelization)

_handles = {}


def _handle():
    """One library handle per (device, stream): a handle is used from one stream at a time."""
    key = (torch.cuda.current_device(), torch.cuda.current_stream().cuda_stream)
    if key not in _handles:
        _handles[key] = make_handle_on_current_stream()
        _handles[key].set_extended_modes(True)  # SparseInverseConv3d runs the operators with inverse = 1
    return _handles[key]


_share_row_maps = False


def share_row_maps(enable):
    """Layers and passes that use one rulebook share its row maps (built once per rulebook and
    direction, without the verifying count since the coordinates are known to be distinct)
    instead of rebuilding them in every operator call.  Pays when a rulebook serves many calls
    (a fixed scene, deep stages: the config-4 forward takes 0.036 ms instead of 0.047 ms); with a
    new rulebook per step and two layers per stage it saves one map build in four (measured on
    the 11-layer encoder: 6.29-6.35 ms a step against 6.32-6.38 ms) and holds K x rows x 8 bytes
    per rulebook, hence off by default."""
    global _share_row_maps
    _share_row_maps = bool(enable)


class Rulebook:
    """indice_pairs [K,2,L] (device), indice_num as host ints, out_indices, num_act_out."""

    def __init__(self, pairs, out_indices, indice_num_host, num_act_out, filter_space, sub_m, out_space,
                 in_indices=None, in_space=None, distinct=False):
        # the input coordinates were distinct: no offset names a result row twice, and the
        # operators may skip their check for such pairs (mluOpExtSetDistinctPairsPromise)
        self.distinct = distinct
        self.in_indices = in_indices  # what an inverse convolution over this rulebook gives back
        self.in_space = None if in_space is None else tuple(in_space)
        self.pairs = pairs
        self.out_indices = out_indices
        self.indice_num = indice_num_host
        self.num_act_out = num_act_out
        self.filter_space = tuple(filter_space)
        self.sub_m = sub_m
        self.out_space = tuple(out_space)
        self._row_maps = {}

    def row_map(self, handle, row_column):
        """The [K, rows] row map of this rulebook for one direction (row_column 1: rows are the
        layer's outputs; 0: its inputs), built on first use and shared by every layer and pass that
        uses the rulebook.  None when the coordinates are not known to be distinct, or when the
        build found pairs that share a slot: the operators then build their own map per call."""
        if not (self.distinct and _share_row_maps):
            return None
        key = (handle.ptr.value, row_column)   # the library records a map with the handle that built it
        if key not in self._row_maps:
            L = self.pairs.shape[2]
            rows, source_rows = (self.num_act_out, L) if row_column == 1 else (L, self.num_act_out)
            # the coordinates are known to be distinct and the handle carries that promise: the
            # build need not count lost pairs, which would make the host wait for the stream
            m = RowMap(handle, self.pairs, self.indice_num, rows, source_rows, row_column, verify=False)
            self._row_maps[key] = m if m.usable else None
        return self._row_maps[key]


class SparseTensor:
    """`distinct=True` is the caller's word that no coordinate occurs twice (the output of a
    voxelizer, or of a strided layer, never repeats one); the convolution operators then skip
    their check for pairs of one offset that share a result row."""

    def __init__(self, features, indices, spatial_shape, batch_size, rulebooks=None, distinct=False):
        assert indices.dtype == torch.int32 and indices.dim() == 2 and indices.shape[1] == 4
        assert features.shape[0] == indices.shape[0]
        self.features = features
        self.indices = indices.contiguous()
        self.spatial_shape = tuple(int(s) for s in spatial_shape)
        self.batch_size = int(batch_size)
        self.rulebooks = {} if rulebooks is None else rulebooks
        self.distinct = bool(distinct)

    def replace_features(self, features):
        return SparseTensor(features, self.indices, self.spatial_shape, self.batch_size, self.rulebooks,
                            self.distinct)

    def dense(self):
        """[N, C, D, H, W] dense tensor (for inspection and tests)."""
        d, h, w = self.spatial_shape
        out = torch.zeros((self.batch_size, d, h, w, self.features.shape[1]), dtype=self.features.dtype,
                          device=self.features.device)
        i = self.indices.long()
        out[i[:, 0], i[:, 1], i[:, 2], i[:, 3]] = self.features
        return out.permute(0, 4, 1, 2, 3).contiguous()


class _IndiceConv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, features, weight, rulebook, inverse=False):
        handle = _handle()
        features = features.contiguous()
        weight = weight.contiguous()
        handle.promise_distinct_pairs(rulebook.distinct)
        if inverse:
            # the partner layer's rulebook backwards: one output row per input row of the partner
            out = indice_conv_forward(handle, features, weight, LAYOUT_ARRAY, rulebook.pairs, rulebook.indice_num,
                                      rulebook.pairs.shape[2], False, inverse=1,
                                      row_map=rulebook.row_map(handle, 0))
        else:
            out = indice_conv_forward(handle, features, weight, LAYOUT_ARRAY, rulebook.pairs,
                                      rulebook.indice_num, rulebook.num_act_out, rulebook.sub_m,
                                      row_map=rulebook.row_map(handle, 1))
        ctx.save_for_backward(features, weight)
        ctx.rulebook = rulebook
        ctx.inverse = inverse
        return out

    @staticmethod
    def backward(ctx, grad_out):
        features, weight = ctx.saved_tensors
        rb = ctx.rulebook
        handle = _handle()
        handle.promise_distinct_pairs(rb.distinct)
        grad_out = grad_out.contiguous()
        grad_features = grad_weight = None
        inverse, sub_m = (1, False) if ctx.inverse else (0, rb.sub_m)
        if ctx.needs_input_grad[0]:
            grad_features = indice_conv_backward_data(handle, grad_out, weight, LAYOUT_ARRAY, rb.pairs,
                                                      rb.indice_num, sub_m, features.shape[1], inverse=inverse,
                                                      rows=features.shape[0],
                                                      row_map=rb.row_map(handle, 1 if ctx.inverse else 0))
        if ctx.needs_input_grad[1]:
            grad_weight = indice_conv_backward_filter(handle, features, grad_out, rb.pairs, rb.indice_num,
                                                      rb.filter_space, sub_m, inverse=inverse)
        return grad_features, grad_weight, None, None


def _mfma_channels(c):
    """The next channel count the matrix-core kernels take, or c itself beyond 128."""
    for size in (16, 32, 64, 128):
        if c <= size:
            return size
    return c


def _triple(v):
    return [int(v)] * 3 if isinstance(v, int) else [int(x) for x in v]


class _ConvBase(torch.nn.Module):
    inverse = False

    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation, sub_m, bias,
                 indice_key):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size = _triple(kernel_size)
        self.stride, self.padding, self.dilation = _triple(stride), _triple(padding), _triple(dilation)
        self.sub_m = sub_m
        self.indice_key = indice_key
        k = self.kernel_size[0] * self.kernel_size[1] * self.kernel_size[2]
        bound = 1.0 / math.sqrt(k * in_channels)
        self.weight = torch.nn.Parameter(
            torch.empty(*self.kernel_size, in_channels, out_channels).uniform_(-bound, bound))
        self.bias = torch.nn.Parameter(torch.zeros(out_channels)) if bias else None

    def _rulebook(self, x):
        if self.indice_key is not None and self.indice_key in x.rulebooks:
            rb = x.rulebooks[self.indice_key]
            assert rb.filter_space == tuple(self.kernel_size) and rb.sub_m == self.sub_m
            return rb
        # a rulebook planned for this layer and these very coordinates (SparseSequential)
        planned = x.rulebooks.get(("planned", id(self)))
        if planned is not None and planned.in_indices is x.indices and planned.in_space == x.spatial_shape:
            return planned
        if self.sub_m:
            out_space = list(x.spatial_shape)
        else:
            out_space = regular_output_space(x.spatial_shape, self.kernel_size, self.padding, self.stride,
                                             self.dilation)
        pairs, out_indices, num, n_out = get_indice_pairs(
            _handle(), x.indices, x.batch_size, x.spatial_shape, self.kernel_size, out_space, self.padding,
            self.stride, self.dilation, self.sub_m)
        # the operators take indice_num as host int64: one device-to-host copy per rulebook
        rb = Rulebook(pairs, out_indices[:n_out], num.cpu().tolist(), n_out, self.kernel_size, self.sub_m,
                      out_space, in_indices=x.indices, in_space=x.spatial_shape, distinct=x.distinct)
        if self.indice_key is not None:
            x.rulebooks[self.indice_key] = rb
        else:
            x.rulebooks[("planned", id(self))] = rb
        return rb

    def _cells_after(self, x, rb):
        """(indices, spatial shape, distinct) of this layer's result on `x`, from the rulebook alone."""
        if self.sub_m:
            return x.indices, x.spatial_shape, x.distinct
        if self.inverse:
            return rb.in_indices, rb.in_space, rb.distinct
        return rb.out_indices.contiguous(), rb.out_space, True

    def _result(self, x, rb, feats):
        if self.sub_m:
            return x.replace_features(feats)
        # the cache travels on, so that an inverse layer downstream finds this rulebook by its key;
        # the active output cells of a regular convolution are distinct by construction
        return SparseTensor(feats, rb.out_indices.contiguous(), rb.out_space, x.batch_size, x.rulebooks,
                            distinct=True)

    def forward(self, x):
        rb = self._rulebook(x)
        feats, weight = x.features, self.weight.to(x.features.dtype)
        # Channel counts the matrix-core kernels take are 16, 32, 64 and 128; a smaller count (the
        # 4 or 5 point features of a first layer) is padded with zero channels, which costs a few
        # megabytes of traffic and saves the several times slower generic kernels.  autograd slices
        # the gradients back.
        ci, co = _mfma_channels(self.in_channels), _mfma_channels(self.out_channels)
        if ci != self.in_channels or co != self.out_channels:
            feats = torch.nn.functional.pad(feats, (0, ci - self.in_channels))
            weight = torch.nn.functional.pad(weight, (0, co - self.out_channels, 0, ci - self.in_channels))
        feats = _IndiceConv.apply(feats, weight, rb, self.inverse)
        if co != self.out_channels:
            feats = feats[:, :self.out_channels]
        if self.bias is not None:
            feats = feats + self.bias.to(feats.dtype)
        return self._result(x, rb, feats)


class SubMConv3d(_ConvBase):
    """Submanifold 3-D sparse convolution: outputs live on the input's active cells."""

    def __init__(self, in_channels, out_channels, kernel_size, dilation=1, bias=False, indice_key=None):
        ks = _triple(kernel_size)
        dil = _triple(dilation)
        pad = [d * (k // 2) for k, d in zip(ks, dil)]
        super().__init__(in_channels, out_channels, ks, 1, pad, dil, True, bias, indice_key)


class SparseConv3d(_ConvBase):
    """Regular (strided / dilated) 3-D sparse convolution: every cell an active input reaches is active."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, bias=False,
                 indice_key=None):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, False, bias,
                         indice_key)


class SparseInverseConv3d(_ConvBase):
    """Inverse of the `SparseConv3d` that cached its rulebook under `indice_key`: takes a tensor on that
    layer's output cells back to its input cells (spconv / mmcv SparseInverseConv3d).  The rulebook
    is read backwards; the filter is this layer's own [kd, kh, kw, Ci, Co]."""

    inverse = True

    def __init__(self, in_channels, out_channels, kernel_size, indice_key, bias=False):
        super().__init__(in_channels, out_channels, kernel_size, 1, 0, 1, False, bias, indice_key)

    def _rulebook(self, x):
        rb = x.rulebooks.get(self.indice_key)
        assert rb is not None, "no layer has cached a rulebook under indice_key %r" % (self.indice_key,)
        assert rb.filter_space == tuple(self.kernel_size) and not rb.sub_m
        assert rb.num_act_out == x.features.shape[0], "the input does not live on the partner layer's output"
        return rb

    def _result(self, x, rb, feats):
        return SparseTensor(feats, rb.in_indices, rb.in_space, x.batch_size, x.rulebooks, distinct=rb.distinct)


class SparseSequential(torch.nn.Sequential):
    """Layers applied in order to a SparseTensor (spconv's SparseSequential): sparse convolutions
    take and return the tensor, any other module is applied to its features.

    Before the first layer runs, the rulebooks of all its convolutions are built, one after the
    other: a rulebook needs coordinates only, and each ends in a wait for its pair counts (the
    operators take `indice_num` on the host).  Built layer by layer inside the network, every such
    wait drains the queue in front of the convolutions that follow; built up front, the host
    runs ahead through all convolutions and the device stays busy."""

    def plan(self, x):
        cells = x
        for m in self:
            if isinstance(m, SparseSequential):
                cells = m.plan(cells)
            elif isinstance(m, _ConvBase):
                rb = m._rulebook(cells)
                indices, space, distinct = m._cells_after(cells, rb)
                if indices is not cells.indices:
                    # (features are not looked at while planning: a view of the right height)
                    cells = SparseTensor(indices.new_empty((indices.shape[0], 0)), indices, space,
                                         cells.batch_size, cells.rulebooks, distinct)
        return cells

    def forward(self, x):
        self.plan(x)
        for m in self:
            if isinstance(m, (_ConvBase, SparseSequential)):
                x = m(x)
            else:
                x = x.replace_features(m(x.features))
        return x


class Voxelization(torch.nn.Module):
    """Hard voxelization of one point cloud [N, F] (x, y, z first), the module mmcv puts in front of
    its sparse encoder: returns (voxels [V, max_num_points, F], coors [V, 3] as (z, y, x),
    num_points_per_voxel [V]) cut to the V voxels found.  Reading V costs one device-to-host copy."""

    def __init__(self, voxel_size, point_cloud_range, max_num_points, max_voxels):
        super().__init__()
        self.register_buffer("voxel_size", torch.tensor(voxel_size, dtype=torch.float32))
        self.register_buffer("point_cloud_range", torch.tensor(point_cloud_range, dtype=torch.float32))
        self.max_num_points = int(max_num_points)
        self.max_voxels = int(max_voxels)

    def grid_shape(self):
        """(D, H, W) = cells along (z, y, x), the spatial shape of the sparse tensor."""
        r, s = self.point_cloud_range.tolist(), self.voxel_size.tolist()
        return tuple(int(math.floor((r[3 + a] - r[a]) / s[a] + 0.5)) for a in (2, 1, 0))

    @torch.no_grad()
    def forward(self, points):
        voxels, coors, npv, num = voxelization(_handle(), points.contiguous().float(), self.voxel_size,
                                               self.point_cloud_range, self.max_num_points, self.max_voxels)
        v = int(num.item())
        return voxels[:v], coors[:v], npv[:v]


def mean_voxel_features(voxels, num_points_per_voxel):
    """Mean of the points of every voxel (mmcv's HardSimpleVFE): [V, max_points, F] -> [V, F]."""
    return voxels.sum(dim=1) / num_points_per_voxel.clamp(min=1).to(voxels.dtype).unsqueeze(1)


def sparse_tensor_from_voxels(features, coors, spatial_shape, batch_index=0, batch_size=1, order_by_cell=True):
    """SparseTensor of one cloud's voxels: indices (n, z, y, x) with n = batch_index.

    A voxelizer numbers its voxels by their first point, not by their place in the grid.  With
    `order_by_cell` (the default) the voxels are put in ascending order of their linear cell
    index here, once: every rulebook built from them, and from the outputs of the layers that
    follow, then sees rows in cell order, which mluOpGetIndicePairs resolves without its hash
    table and the convolutions read as pair lists without a row map.  The rows of the returned
    tensor are a permutation of the voxelizer's; `order_by_cell=False` keeps its order."""
    coors = coors.to(torch.int32)
    if order_by_cell and coors.shape[0] > 1:
        d, h, w = (int(v) for v in spatial_shape)
        key = (coors[:, 0].to(torch.int64) * h + coors[:, 1].to(torch.int64)) * w + coors[:, 2].to(torch.int64)
        order = torch.argsort(key)
        coors = coors[order]
        features = features[order]
    n = torch.full((coors.shape[0], 1), int(batch_index), dtype=torch.int32, device=coors.device)
    # a voxelizer emits every voxel once
    return SparseTensor(features, torch.cat([n, coors], dim=1).contiguous(), spatial_shape, batch_size,
                        distinct=True)
