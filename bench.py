#!/usr/bin/env python3
"""Benchmark of the sparse-convolution hot path on one MI355X.

A step is one pass of the path over one synthetic voxel set already resident in HBM, in the call
sequence the API prescribes: mluOpGetIndicePairs (rulebook), the copy of indice_num to the host
(the convolutions take the counts as a host array), mluOpIndiceConvolutionForward; all through the
library's C ABI with descriptors and workspaces prepared once.  The default workload is BASELINE
configuration 4 (submanifold 3x3x3, 120 000 clustered voxels in 1x41x1600x1408, Ci=Co=64 fp16);
--workload names the other BASELINE layers (regular ones included: their rulebook call waits for
num_act_out inside, as the reference's does) and four layers of a detection network.

Prints one JSON line: `value` is the forward operator's algorithmic TFLOP/s (2*P*Ci*Co per call
over its device time), `rulebook_mvoxels_per_s` the second half of the metric, `roofline`
describes the kernel that takes the most time in a step, `cpu_baseline` times the CPU oracle on
the same workload on one host core.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "mlu-ops_amd", "python"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "indice_conv fwd TFLOP/s + get_indice_pairs Mvoxels/s, 120k voxels Ci=Co=64"
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_F32_PEAK_TFLOPS = 157.3

WORKLOADS = {
    # name: grid N,D,H,W, rows, generator, seed, channels, dtype, kernel / stride / padding, mode
    "config4": dict(grid=(1, 41, 1600, 1408), per_batch=120000, gen="clustered", seed=4, ci=64, co=64,
                    dtype="float16", ks=(3, 3, 3),
                    text="BASELINE config 4: subm 3x3x3, 120000 clustered voxels in 1x41x1600x1408, "
                         "Ci=Co=64 fp16, rows sorted by linear cell index"),
    "config2": dict(grid=(2, 41, 1600, 1408), per_batch=60000, gen="clustered", seed=2, ci=32, co=32,
                    dtype="float16", ks=(3, 3, 3),
                    text="BASELINE config 2: subm 3x3x3, 2x60000 clustered voxels in 2x41x1600x1408, "
                         "Ci=Co=32 fp16"),
    "config1": dict(grid=(1, 40, 400, 352), per_batch=20000, gen="uniform", seed=1, ci=16, co=16,
                    dtype="float32", ks=(3, 3, 3),
                    text="BASELINE config 1: subm 3x3x3, 20000 uniform voxels in 1x40x400x352, Ci=Co=16 fp32"),
    "config3": dict(grid=(4, 41, 1600, 1408), per_batch=30000, gen="clustered", seed=3, ci=64, co=64,
                    dtype="bfloat16", ks=(3, 3, 3), sub_m=False, stride=(2, 2, 2), pad=(1, 1, 1),
                    text="BASELINE config 3: regular 3x3x3 stride 2 pad 1, 4x30000 clustered voxels in "
                         "4x41x1600x1408 -> 4x21x800x704, Ci=Co=64 bf16"),
    "config5a": dict(grid=(1, 64, 1024, 1024), per_batch=400000, gen="surface", seed=5, ci=128, co=128,
                     dtype="float16", ks=(5, 5, 5),
                     text="BASELINE config 5, first layer: subm 5x5x5, 400000 voxels on 50 planes and spheres "
                          "(5 % uniform noise) in 1x64x1024x1024, Ci=Co=128 fp16"),
    "config5a_fp32": dict(grid=(1, 64, 1024, 1024), per_batch=400000, gen="surface", seed=5, ci=128, co=128,
                          dtype="float32", ks=(5, 5, 5),
                          text="BASELINE config 5, first layer in fp32: subm 5x5x5, 400000 voxels on 50 planes "
                               "and spheres in 1x64x1024x1024, Ci=Co=128"),
    "config5b": dict(grid=(1, 64, 1024, 1024), per_batch=400000, gen="surface", seed=5, ci=128, co=128,
                     dtype="float16", ks=(2, 2, 2), sub_m=False, stride=(2, 2, 2), pad=(0, 0, 0),
                     text="BASELINE config 5, second layer: regular 2x2x2 stride 2 pad 0 on the first layer's "
                          "400000 output voxels, 1x64x1024x1024 -> 1x32x512x512, Ci=Co=128 fp16"),
    "config5b_fp32": dict(grid=(1, 64, 1024, 1024), per_batch=400000, gen="surface", seed=5, ci=128, co=128,
                          dtype="float32", ks=(2, 2, 2), sub_m=False, stride=(2, 2, 2), pad=(0, 0, 0),
                          text="BASELINE config 5, second layer in fp32: regular 2x2x2 stride 2 pad 0, "
                               "1x64x1024x1024 -> 1x32x512x512, Ci=Co=128"),
    # the shapes the reference's design documents quote from a detection network
    # (docs/design_docs/get_indice_pairs/get_indice_pairs.md:331-368,
    # docs/design_docs/indice_convolution_forward/indice_convolution_forward.md:229-234)
    "network_subm16": dict(grid=(4, 41, 1440, 1440), rows=248636, gen="scene", seed=11, ci=16, co=16,
                           dtype="float16", ks=(3, 3, 3),
                           text="network layer: subm 3x3x3, 248636 scene voxels (11 pairs a voxel) in "
                                "4x41x1440x1440, Ci=Co=16 fp16"),
    "network_subm64": dict(grid=(4, 41, 1440, 1440), rows=248636, gen="scene", seed=11, ci=64, co=64,
                           dtype="float16", ks=(3, 3, 3),
                           text="network layer: subm 3x3x3, 248636 scene voxels (11 pairs a voxel) in "
                                "4x41x1440x1440, Ci=Co=64 fp16"),
    "network_subm128": dict(grid=(4, 41, 1440, 1440), rows=248636, gen="scene", seed=11, ci=128, co=128,
                            dtype="float16", ks=(3, 3, 3),
                            text="network layer: subm 3x3x3, 248636 scene voxels (11 pairs a voxel) in "
                                 "4x41x1440x1440, Ci=Co=128 fp16"),
    "network_strided": dict(grid=(4, 11, 360, 360), rows=149100, gen="scene", seed=12, ci=64, co=128,
                            dtype="float16", ks=(3, 3, 3), sub_m=False, stride=(2, 2, 2), pad=(0, 1, 1),
                            scene=dict(sheet_frac=0.68, wall_frac=0.30),
                            text="network layer: regular 3x3x3 stride 2 pad (0,1,1), 149100 scene voxels in "
                                 "4x11x360x360 -> 4x5x180x180 (about 59000 outputs), 64 -> 128 channels fp16"),
}


def library_fingerprint():
    """sha256 over the library's sources: what a committed counter summary was measured on."""
    import hashlib
    h = hashlib.sha256()
    base = os.path.join(ROOT, "mlu-ops_amd")
    files = [os.path.join(base, "Makefile")]
    for d, _, names in sorted(os.walk(os.path.join(base, "csrc"))):
        files += [os.path.join(d, n) for n in sorted(names)]
    for f in files:
        with open(f, "rb") as fh:
            h.update(os.path.relpath(f, base).encode())
            h.update(fh.read())
    return h.hexdigest()[:16]


class Step:
    """Descriptors, buffers and workspaces of one sparse-convolution layer, built once."""

    def __init__(self, handle, wl):
        import numpy as np
        import torch
        import mluop_hip as m
        self.m, self.torch, self.handle, self.wl = m, torch, handle, wl
        grid = wl["grid"]
        if wl["gen"] == "clustered":
            idx = m.datagen.clustered_voxels(grid, wl["per_batch"], wl["seed"])
        elif wl["gen"] == "surface":
            idx = m.datagen.surface_voxels(grid, wl["per_batch"], wl["seed"])
        elif wl["gen"] == "scene":
            idx = m.datagen.scene_voxels(grid, wl["rows"], wl["seed"], **wl.get("scene", {}))
        else:
            idx = m.datagen.uniform_voxels(grid, wl["per_batch"] * grid[0], wl["seed"])
        if wl.get("shuffle"):
            idx = np.ascontiguousarray(idx[np.random.default_rng(wl["seed"]).permutation(idx.shape[0])])
        self.idx_np = idx
        L = idx.shape[0]
        ks = wl["ks"]
        K = ks[0] * ks[1] * ks[2]
        ci, co = wl["ci"], wl["co"]
        self.L, self.K, self.ci, self.co = L, K, ci, co
        self.sub_m = wl.get("sub_m", True)
        self.space = list(grid[1:])
        self.stride = list(wl.get("stride", (1, 1, 1)))
        self.pad = list(wl.get("pad", tuple(k // 2 for k in ks)))
        self.out_space = self.space if self.sub_m else m.regular_output_space(
            self.space, list(ks), self.pad, self.stride, [1, 1, 1])
        tdt = getattr(torch, wl["dtype"])
        self.tdt = tdt
        self.elem = 4 if wl["dtype"] == "float32" else 2
        rng = np.random.default_rng(wl["seed"])
        self.feats_np = rng.standard_normal((L, ci)).astype(np.float32)
        self.w_np = m.datagen.kaiming_uniform_filters(ks, ci, co, wl["seed"])
        dev = "cuda"
        self.indices = torch.from_numpy(idx).to(dev)
        self.features = torch.from_numpy(self.feats_np).to(dev, tdt)
        self.filters = torch.from_numpy(self.w_np).to(dev, tdt)
        self.pairs = torch.empty((K, 2, L), dtype=torch.int32, device=dev)
        out_cells = grid[0] * self.out_space[0] * self.out_space[1] * self.out_space[2]
        self.out_rows = L if self.sub_m else min(out_cells, K * L)
        self.out_indices = torch.empty((self.out_rows, 4), dtype=torch.int32, device=dev)
        self.indice_num = torch.empty((K,), dtype=torch.int32, device=dev)
        self.num_pinned = torch.empty((K,), dtype=torch.int32).pin_memory()
        code = m.torch_dtype_code(tdt)
        self.code = code
        self.sdesc = m.SparseConvDescriptor(grid[0], self.pad, self.stride, [1, 1, 1], self.space, list(ks),
                                            self.out_space, 1 if self.sub_m else 0)
        self.d_idx = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [L, 4])
        self.d_pairs = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [K, 2, L])
        self.d_oidx = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [self.out_rows, 4])
        self.d_num = m.TensorDescriptor(m.LAYOUT_ARRAY, m.DTYPE_INT32, [K])
        self.d_feat = m.TensorDescriptor(m.LAYOUT_ARRAY, code, [L, ci])
        self.d_filt = m.TensorDescriptor(m.LAYOUT_ARRAY, code, list(ks) + [ci, co])
        self.d_dw = m.TensorDescriptor(m.LAYOUT_ARRAY, code, list(ks) + [ci, co], onchip_dtype=m.DTYPE_FLOAT)
        lib = m.lib()
        size = ctypes.c_size_t(0)
        m.check(lib.mluOpGetIndicePairsWorkspaceSize(handle.ptr, self.sdesc.ptr, self.d_idx.ptr, self.d_pairs.ptr,
                                                     self.d_oidx.ptr, self.d_num.ptr, ctypes.byref(size)))
        self.ws_rb_size = size.value
        self.ws_rb = torch.empty(max(size.value, 1), dtype=torch.uint8, device=dev)
        # one rulebook build to learn the shapes that depend on it
        self.rulebook()
        self.read_counts()
        self.n_out = L if self.sub_m else self.sdesc.num_act_out()
        self.P = int(sum(self.counts))
        n_out = self.n_out
        self.dy_np = (rng.standard_normal((n_out, co)) * 0.1).astype(np.float32)
        self.dy = torch.from_numpy(self.dy_np).to(dev, tdt)
        self.out = torch.empty((n_out, co), dtype=tdt, device=dev)
        self.dx = torch.empty((L, ci), dtype=tdt, device=dev)
        self.dw = torch.empty(tuple(ks) + (ci, co), dtype=tdt, device=dev)
        self.d_out = m.TensorDescriptor(m.LAYOUT_ARRAY, code, [n_out, co])
        self.d_dy = m.TensorDescriptor(m.LAYOUT_ARRAY, code, [n_out, co])
        self.d_dx = m.TensorDescriptor(m.LAYOUT_ARRAY, code, [L, ci])
        sm = 1 if self.sub_m else 0
        m.check(lib.mluOpGetIndiceConvolutionForwardWorkspaceSize(
            handle.ptr, self.d_feat.ptr, self.d_filt.ptr, self.d_pairs.ptr, self.d_out.ptr, self.counts, n_out, 0, sm,
            ctypes.byref(size)))
        self.ws_fwd_size = size.value
        self.ws_fwd = torch.empty(max(size.value, 1), dtype=torch.uint8, device=dev)
        m.check(lib.mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(
            handle.ptr, self.d_dy.ptr, self.d_filt.ptr, self.d_pairs.ptr, self.d_dx.ptr, self.counts, 0,
            ctypes.byref(size)))
        self.ws_bd_size = size.value
        self.ws_bd = torch.empty(max(size.value, 1), dtype=torch.uint8, device=dev)
        m.check(lib.mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(
            handle.ptr, self.d_feat.ptr, self.d_dy.ptr, self.d_pairs.ptr, self.d_dw.ptr, self.counts, 0, sm,
            ctypes.byref(size)))
        self.ws_bf_size = size.value
        self.ws_bf = torch.empty(max(size.value, 1), dtype=torch.uint8, device=dev)

    def rulebook(self):
        m = self.m
        m.check(m.lib().mluOpGetIndicePairs(
            self.handle.ptr, self.sdesc.ptr, self.d_idx.ptr, self.indices.data_ptr(), self.ws_rb.data_ptr(),
            self.ws_rb_size, self.d_pairs.ptr, self.pairs.data_ptr(), self.d_oidx.ptr, self.out_indices.data_ptr(),
            self.d_num.ptr, self.indice_num.data_ptr()), "mluOpGetIndicePairs")

    def read_counts(self):
        """The hand-off the API prescribes between the rulebook and the convolutions: indice_num
        leaves the device and becomes the host array of 64-bit counts the operators take."""
        self.num_pinned.copy_(self.indice_num, non_blocking=True)
        self.torch.cuda.current_stream().synchronize()
        self.counts = (ctypes.c_int64 * self.K)(*self.num_pinned.tolist())

    def forward(self):
        m = self.m
        m.check(m.lib().mluOpIndiceConvolutionForward(
            self.handle.ptr, self.d_feat.ptr, self.features.data_ptr(), self.d_filt.ptr, self.filters.data_ptr(),
            self.d_pairs.ptr, self.pairs.data_ptr(), self.counts, self.n_out, 0, 1 if self.sub_m else 0,
            self.ws_fwd.data_ptr(), self.ws_fwd_size, self.d_out.ptr, self.out.data_ptr()),
            "mluOpIndiceConvolutionForward")

    def backward_data(self):
        m = self.m
        m.check(m.lib().mluOpIndiceConvolutionBackwardData(
            self.handle.ptr, self.d_dy.ptr, self.dy.data_ptr(), self.d_filt.ptr, self.filters.data_ptr(),
            self.d_pairs.ptr, self.pairs.data_ptr(), self.counts, 0, 1 if self.sub_m else 0, self.ws_bd.data_ptr(),
            self.ws_bd_size, self.d_dx.ptr, self.dx.data_ptr()), "mluOpIndiceConvolutionBackwardData")

    def backward_filter(self):
        m = self.m
        m.check(m.lib().mluOpIndiceConvolutionBackwardFilter(
            self.handle.ptr, self.d_feat.ptr, self.features.data_ptr(), self.d_dy.ptr, self.dy.data_ptr(),
            self.d_pairs.ptr, self.pairs.data_ptr(), self.counts, 0, 1 if self.sub_m else 0, self.ws_bf.data_ptr(),
            self.ws_bf_size, self.d_dw.ptr, self.dw.data_ptr()), "mluOpIndiceConvolutionBackwardFilter")

    # algorithmic work (per call)
    def conv_flops(self):
        return 2.0 * self.P * self.ci * self.co

    def rulebook_bytes(self):
        return 16.0 * self.L + 8.0 * self.K * self.L + 4.0 * self.K + 16.0 * self.n_out

    def forward_bytes(self):
        s = self.elem
        return self.L * self.ci * s + self.n_out * self.co * s + self.K * self.ci * self.co * s + 8.0 * self.P

    def backward_filter_bytes(self):
        s = self.elem
        return self.L * self.ci * s + self.n_out * self.co * s + self.K * self.ci * self.co * 4.0 + 8.0 * self.P


def median(v):
    v = sorted(v)
    return v[len(v) // 2]


def time_ops(torch, ops, steps):
    """Runs every op of `ops` once per step, with events between them on the current stream.
    Returns (wall seconds, {name: [ms per step]})."""
    names = [n for n, _ in ops]
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(ops) + 1)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        ev[s][0].record()
        for i, (_, fn) in enumerate(ops):
            fn()
            ev[s][i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = {n: [ev[s][i].elapsed_time(ev[s][i + 1]) for s in range(steps)] for i, n in enumerate(names)}
    return wall, per


def cpu_baseline(step):
    """The CPU oracle (plain-C restatement of the reference's cpuCompute) on the same workload,
    one thread: rulebook, then forward on the device-rounded inputs.  Workloads whose forward is
    more than a few seconds of CPU work are timed once, and on a prefix of the pairs of every offset
    (the oracle's cost is linear in the pairs)."""
    import numpy as np
    import sparse_conv_oracle as oracle
    wl = step.wl
    ks = list(wl["ks"])
    if wl["dtype"] == "float16":
        rnd = oracle.round_through_half
    elif wl["dtype"] == "bfloat16":
        rnd = oracle.round_through_bf16
    else:
        rnd = lambda a: a
    feats, w = rnd(step.feats_np), rnd(step.w_np).reshape(step.K, step.ci, step.co)
    macs = float(step.P) * step.ci * step.co
    reps = 3 if macs < 3e9 else 1
    keep = 1.0 if macs < 6e10 else 6e10 / macs   # at most about 15 s of forward
    t_rb, t_fw = [], []
    for _ in range(reps):
        t0 = time.perf_counter()
        pairs, oidx, num, n_out = oracle.get_indice_pairs(step.idx_np, wl["grid"][0], step.pad, step.stride,
                                                          [1, 1, 1], ks, step.out_space, step.sub_m)
        t1 = time.perf_counter()
        num_s = np.maximum((np.asarray(num) * keep).astype(np.asarray(num).dtype), np.minimum(num, 1))
        t1b = time.perf_counter()
        oracle.forward(feats, w, pairs, num_s, n_out)
        t2 = time.perf_counter()
        t_rb.append(t1 - t0)
        t_fw.append(t2 - t1b)
    P_timed = int(np.sum(num_s))
    fw, rb = median(t_fw), median(t_rb)
    sample = "full workload" if keep == 1.0 else "rulebook in full, forward on the first %.0f %% of every offset's pairs" % (keep * 100)
    return {"value": 2.0 * P_timed * step.ci * step.co / fw / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": "%s (%d voxels, %d pairs timed), median of %d, gcc -O2 single thread, host has %d logical "
                      "cores" % (sample, step.L, P_timed, reps, os.cpu_count()),
            "forward_ms": fw * 1e3, "rulebook_ms": rb * 1e3,
            "rulebook_mvoxels_per_s": step.L / rb / 1e6}


def graph_replay_step(torch, m, handle, step, step_ops, steps):
    """The same step captured once into a HIP graph and replayed `steps` times: what a caller that
    captures its layers pays (the operators enqueue kernels only).  Reported beside the headline
    figures, which stay those of plain calls."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    try:
        with torch.cuda.stream(side):
            handle.set_queue(side.cuda_stream)
            for _, fn in step_ops:
                fn()
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _, fn in step_ops:
                    fn()
            graph.replay()
            side.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            for _ in range(steps):
                graph.replay()
            e1.record(side)
            side.synchronize()
            ms = e0.elapsed_time(e1) / steps
        return {"ms_per_step": ms, "note": "get_indice_pairs + forward captured in one HIP graph"}
    except Exception as exc:  # capture is a convenience of the caller, never the headline number
        return {"ms_per_step": None, "note": "capture failed: %s" % exc}
    finally:
        handle.set_queue(torch.cuda.current_stream().cuda_stream)
        torch.cuda.current_stream().wait_stream(side)


def measured_traffic(workload, kernel):
    """(HBM bytes per launch of `kernel`, note) from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE
    summary of this workload (counters cannot be read from inside the process).  The summary names
    the library sources it was measured on; for other sources the figure is withheld."""
    path = os.path.join(ROOT, "profiles", "pmc_traffic_%s.json" % workload)
    try:
        with open(path) as f:
            doc = json.load(f)
        if doc.get("library_fingerprint") != library_fingerprint():
            return None, "profiles/pmc_traffic_%s.json was measured on other library sources" % workload
        return doc["kernels"][kernel]["total_bytes"], None
    except (OSError, KeyError, ValueError):
        return None, "no counter summary for this kernel and workload"


def operator_roofline(workload, kernels, names, op_ms, alg_bytes, bytes_model, flops=None, mfma_peak=None):
    """Roofline object of one operator: its algorithmic bytes over its device time `op_ms` (HIP
    events around back-to-back calls, launch gaps between its kernels included), the counter
    traffic summed over its kernels `names` (those of them that ran).  `kernel_sum_us` adds up
    the library's per-kernel event timing of the same kernels, which reads about 2 us a launch
    above the kernel trace."""
    ran = [n for n in names if n in kernels]
    if not ran:
        return None
    kernel_sum = sum(kernels[n]["avg_us"] * kernels[n].get("launches_per_step", kernels[n].get("launches", 1.0))
                     for n in ran)
    us = op_ms * 1e3
    traffic, note = 0.0, None
    for n in ran:
        t, why = measured_traffic(workload, n)
        if t is None:
            traffic, note = None, why
            break
        traffic += t
    achieved = alg_bytes / (us * 1e-6) / 1e9
    out = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "kernels": ran, "operator_us": us,
           "kernel_sum_us": kernel_sum, "algorithmic_bytes": alg_bytes, "bytes_model": bytes_model}
    if note:
        out["traffic_note"] = note
    if flops is not None:
        out["mfma_frac"] = flops / (us * 1e-6) / 1e12 / mfma_peak
    return out


UPSTREAM = {
    # the operators in front of the sparse convolutions: 1.2 M points on a 1408 x 1600 x 40 grid
    "voxelization": "hard voxelization, 1 200 000 points (4 features), voxel 0.05 x 0.05 x 0.1 in "
                    "[0,70.4]x[-40,40]x[-3,1], max_points 5, max_voxels 150000",
    "dynamic_point_to_voxel": "dynamic point-to-voxel scatter (mean), 1 000 000 points (4 features), "
                              "coordinates in 40 x 1600 x 1408, 5 % invalid",
}


def run_backbone(args, torch, m):
    """Forward + backward of a sparse encoder in the shape of SECOND / CenterPoint's (submanifold
    pairs at four resolutions, strided convolutions between them) over the caller layer
    (mluop_hip.nn): what a training step of the sparse part costs end to end, Python included."""
    import numpy as np
    from mluop_hip import nn as spnn
    grid = (1, 41, 1600, 1408)
    idx = m.datagen.clustered_voxels(grid, 120000, 4)
    rng = np.random.default_rng(4)
    feats = torch.from_numpy(rng.standard_normal((idx.shape[0], 5)).astype(np.float32)).cuda().half()
    indices = torch.from_numpy(idx).cuda()
    torch.manual_seed(0)
    layers = [spnn.SubMConv3d(5, 16, 3, indice_key="s1"), spnn.SubMConv3d(16, 16, 3, indice_key="s1")]
    c = 16
    for stage, co in enumerate((32, 64, 128), start=2):
        layers.append(spnn.SparseConv3d(c, co, 3, stride=2, padding=1))
        layers += [spnn.SubMConv3d(co, co, 3, indice_key="s%d" % stage) for _ in range(2)]
        c = co
    # (a ReLU behind every layer; the container builds all rulebooks before the first layer runs)
    net = spnn.SparseSequential(*[m for layer in layers for m in (layer, torch.nn.ReLU())]).cuda().half()
    # MLUOP_BENCH_SHARE_ROW_MAPS=1: layers of a stage share their rulebook's row maps
    spnn.share_row_maps(os.environ.get("MLUOP_BENCH_SHARE_ROW_MAPS", "0") == "1")

    def step():
        # the voxels are distinct, as a voxelizer's output is: the layers skip the collision check
        x = net(spnn.SparseTensor(feats.clone().requires_grad_(True), indices, grid[1:], grid[0], distinct=True))
        x.features.float().square().mean().backward()
        return x

    for _ in range(max(args.warmup, 2)):
        out = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    rows = [int(idx.shape[0])]
    x = spnn.SparseTensor(feats, indices, grid[1:], grid[0], distinct=True)
    with torch.no_grad():
        for layer in layers:
            x = layer(x)
            if not layer.sub_m:
                rows.append(int(x.features.shape[0]))
    print(json.dumps({"metric": "sparse encoder forward+backward ms", "value": ms, "unit": "ms", "n_gpus": 1,
                      "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": False,
                      "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
                      "config": {"workload": "11 sparse layers (5-16-16 | 32x3 | 64x3 | 128x3 channels, 3 strided), "
                                             "120000 clustered voxels in 1x41x1600x1408, fp16, wall clock with "
                                             "the Python caller layer", "rows_per_stage": rows},
                      "output_rows": int(out.features.shape[0])}))


def run_upstream(args, torch, m, handle):
    """Times one of the upstream operators (not the headline metric): prints its own JSON line."""
    import numpy as np
    rng = np.random.default_rng(10)
    if args.workload == "voxelization":
        n = 1200000
        pts = np.empty((n, 4), np.float32)
        pts[:, 0] = rng.uniform(0.0, 70.4, n)
        pts[:, 1] = rng.uniform(-40.0, 40.0, n)
        pts[:, 2] = rng.uniform(-3.0, 1.0, n)
        pts[:, 3] = rng.uniform(0.0, 1.0, n)
        far = rng.choice(n, n // 20, replace=False)
        pts[far, :3] += 200.0
        points = torch.from_numpy(pts).cuda()
        vs = torch.tensor([0.05, 0.05, 0.1], device="cuda")
        cr = torch.tensor([0.0, -40.0, -3.0, 70.4, 40.0, 1.0], device="cuda")
        op = lambda: m.voxelization(handle, points, vs, cr, 5, 150000)
        # points read, voxels/coors/counts zero-filled and written
        algorithmic = n * 16 + 150000 * (5 * 16 + 12 + 4) * 2
    else:
        n = 1000000
        feats = torch.from_numpy(rng.uniform(-100, 100, (n, 4)).astype(np.float32)).cuda()
        c = np.stack([rng.integers(0, 40, n), rng.integers(0, 1600, n), rng.integers(0, 1408, n)], axis=1)
        c[rng.choice(n, n // 20, replace=False), 0] = -1
        coors = torch.from_numpy(c.astype(np.int32)).cuda()
        op = lambda: m.dynamic_point_to_voxel_forward(handle, feats, coors, "mean")
        # feats + coors read; per-point map and (at most N) voxel rows written
        algorithmic = n * (16 + 12 + 4) + n * (16 + 12 + 4)
    for _ in range(args.warmup):
        op()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        op()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    result = {"metric": args.workload + " Mpoints/s", "value": n / (ms * 1e-3) / 1e6, "unit": "Mpoints/s",
              "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32/int32",
              "data": "synthetic", "config": {"workload": UPSTREAM[args.workload], "points": n}}
    if not args.only_step:
        handle.set_kernel_timing(True)
        op()
        torch.cuda.synchronize()
        agg = {}
        for name, t in handle.kernel_timings():
            agg[name] = agg.get(name, 0.0) + t * 1e3
        handle.set_kernel_timing(False)
        result["kernels_us_per_call"] = agg
        result["roofline"] = {"bound": "hbm", "achieved": algorithmic / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                              "unit": "GB/s", "frac": algorithmic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                              "traffic": None, "kernel": "whole operator", "algorithmic_bytes": algorithmic}
    print(json.dumps(result))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="config4", choices=sorted(WORKLOADS) + sorted(UPSTREAM) + ["backbone"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only-step", action="store_true",
                    help="run just warmup + timed steps (for profiler runs)")
    ap.add_argument("--with-backward", action="store_true",
                    help="with --only-step: every step also runs backward data and backward filter "
                         "(profiler runs of the backward kernels; the printed figures stay those of "
                         "rulebook + forward)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="with --only-step: also run one 64 MiB device-to-device copy, the known-size "
                         "kernel that scales the profiler's FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the rulebook and the "
              "convolutions shard by batch index without communication); run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import mluop_hip as m
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.workload == "backbone":
        run_backbone(args, torch, m)
        return
    handle = m.make_handle_on_current_stream()
    if args.workload in UPSTREAM:
        run_upstream(args, torch, m, handle)
        return
    wl = WORKLOADS[args.workload]
    step = Step(handle, wl)
    # The step as the API prescribes it: the rulebook, the copy of indice_num to the host (the
    # convolutions take it as a host array), the forward convolution.
    step_ops = [("get_indice_pairs", step.rulebook), ("read_counts", step.read_counts), ("forward", step.forward)]

    for _ in range(args.warmup):
        for _, fn in step_ops:
            fn()
    torch.cuda.synchronize()

    # timed region: exactly --steps steps
    wall, _ = time_ops(torch, step_ops, args.steps)
    ms_per_step = wall * 1e3 / args.steps
    # Device time of the two operators: the same number of calls of each, back to back, events on
    # the handle's stream between them.  (Inside a step the forward call follows a wait for the
    # queue, so an event pair around it there would also count the host's way to the first launch.)
    _, per_rb = time_ops(torch, [("get_indice_pairs", step.rulebook)], args.steps)
    step.read_counts()
    _, per_fw = time_ops(torch, [("forward", step.forward)], args.steps)
    per = {"forward": per_fw["forward"], "get_indice_pairs": per_rb["get_indice_pairs"]}
    fwd_ms = sum(per["forward"]) / args.steps
    rb_ms = sum(per["get_indice_pairs"]) / args.steps
    result = {
        "metric": METRIC, "value": step.conv_flops() / (fwd_ms * 1e-3) / 1e12, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}[wl["dtype"]], "data": "synthetic",
        "config": {"workload": wl["text"] + "; step = get_indice_pairs + copy of indice_num to the host + "
                               "indice_convolution_forward",
                   "voxels": step.L, "outputs": step.n_out, "pairs": step.P, "Ci": step.ci, "Co": step.co,
                   "kernel_volume": step.K},
        "rulebook_mvoxels_per_s": step.L / (rb_ms * 1e-3) / 1e6,
        "forward_ms": fwd_ms, "forward_ms_min": min(per["forward"]),
        "rulebook_ms": rb_ms, "rulebook_ms_min": min(per["get_indice_pairs"]),
    }
    if args.only_step:
        if args.with_backward:
            for _ in range(args.steps):
                step.backward_data()
                step.backward_filter()
            torch.cuda.synchronize()
        if args.calibration_copy:
            src = torch.ones(16 * 1024 * 1024, dtype=torch.float32, device="cuda")
            dst = torch.empty_like(src)
            torch.cuda.synchronize()
            dst.copy_(src)
            torch.cuda.synchronize()
        print(json.dumps(result))
        return

    # the same steps again with the library's per-kernel event timing switched on
    handle.set_kernel_timing(True)
    for _ in range(args.steps):
        for _, fn in step_ops:
            fn()
    records = handle.kernel_timings()
    handle.set_kernel_timing(False)
    agg = {}
    for name, ms in records:
        tot, cnt = agg.get(name, (0.0, 0))
        agg[name] = (tot + ms, cnt + 1)
    kernels = {n: {"avg_us": t / c * 1e3, "launches_per_step": c / args.steps} for n, (t, c) in agg.items()}
    result["kernels"] = kernels
    dominant = max(agg, key=lambda n: agg[n][0])
    dom_ms = agg[dominant][0] / agg[dominant][1]
    if dominant.startswith("rb"):
        alg_bytes, what = step.rulebook_bytes(), "rulebook bytes 16L + 8KL + 4K + 16N_out"
    else:
        alg_bytes, what = step.forward_bytes(), "forward bytes L*Ci*s + N*Co*s + K*Ci*Co*s + 8P"
    # The bound that binds: a kernel that moves more than 312 FLOP per algorithmic byte (2.5 PFLOP/s
    # over 8 TB/s) is priced against the matrix cores, any other against HBM.
    mfma_peak = MFMA_F32_PEAK_TFLOPS if wl["dtype"] == "float32" else MFMA_F16_PEAK_TFLOPS
    traffic, traffic_note = measured_traffic(args.workload, dominant)
    if not dominant.startswith("rb") and step.conv_flops() / alg_bytes > mfma_peak * 1e12 / (HBM_PEAK_GBS * 1e9):
        achieved = step.conv_flops() / (dom_ms * 1e-3) / 1e12
        result["roofline"] = {"bound": "mfma", "achieved": achieved, "peak": mfma_peak, "unit": "TFLOP/s",
                              "frac": achieved / mfma_peak, "traffic": traffic, "kernel": dominant,
                              "kernel_avg_us": dom_ms * 1e3, "algorithmic_flops": step.conv_flops(),
                              "algorithmic_bytes": alg_bytes}
    else:
        achieved = alg_bytes / (dom_ms * 1e-3) / 1e9
        result["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "kernel": dominant,
                              "kernel_avg_us": dom_ms * 1e3, "algorithmic_bytes": alg_bytes, "bytes_model": what}
    if traffic_note:
        result["roofline"]["traffic_note"] = traffic_note
    # the other half of the metric: the rulebook's kernels against its algorithmic bytes
    result["rulebook_roofline"] = operator_roofline(
        args.workload, kernels, [n for n in kernels if n.startswith("rb")], rb_ms, step.rulebook_bytes(),
        "rulebook bytes 16L + 8KL + 4K + 16N_out")
    gather = [n for n in agg if n.startswith("gatherConv")]
    if gather:
        g = max(gather, key=lambda n: agg[n][0])
        g_ms = agg[g][0] / agg[g][1]
        result["forward_kernel"] = {
            "kernel": g, "avg_us": g_ms * 1e3,
            "hbm_frac": step.forward_bytes() / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "mfma_frac": step.conv_flops() / (g_ms * 1e-3) / 1e12 / mfma_peak}

    # the two backward operators of the same layer, reported beside the metric
    _, per_b = time_ops(torch, [("backward_data", step.backward_data), ("backward_filter", step.backward_filter)],
                        max(args.steps // 4, 5))
    handle.set_kernel_timing(True)
    for _ in range(5):
        step.backward_data()
        step.backward_filter()
    agg_b = {}
    for name, ms in handle.kernel_timings():
        tot, cnt = agg_b.get(name, (0.0, 0))
        agg_b[name] = (tot + ms, cnt + 1)
    handle.set_kernel_timing(False)
    result["backward_kernels"] = {n: {"avg_us": t / c * 1e3, "launches": c / 5} for n, (t, c) in agg_b.items()}
    result["backward_data_ms"] = median(per_b["backward_data"])
    result["backward_filter_ms"] = median(per_b["backward_filter"])
    bk = result["backward_kernels"]
    filter_kernels = [n for n in bk if n.startswith("backwardFilter") or n.startswith("sliceSum")
                      or n.startswith("reduceFilter")]
    result["backward_data_roofline"] = operator_roofline(
        args.workload, bk, [n for n in bk if n not in filter_kernels], result["backward_data_ms"],
        step.forward_bytes(), "backward-data bytes N*Co*s + L*Ci*s + K*Ci*Co*s + 8P", step.conv_flops(), mfma_peak)
    result["backward_filter_roofline"] = operator_roofline(
        args.workload, bk, filter_kernels, result["backward_filter_ms"], step.backward_filter_bytes(),
        "backward-filter bytes L*Ci*s + N*Co*s + K*Ci*Co*4 + 8P", step.conv_flops(), mfma_peak)
    result["backward_data_tflops"] = step.conv_flops() / (result["backward_data_ms"] * 1e-3) / 1e12
    result["backward_filter_tflops"] = step.conv_flops() / (result["backward_filter_ms"] * 1e-3) / 1e12

    # Not part of the metric: the step without the copy of indice_num (a caller that kept the counts
    # of an identical rulebook).  The forward operator then cannot know yet whether the rulebook's
    # input rows were in cell order: it starts on the pair lists and enqueues the row-map kernels
    # behind them, and the device decides which of the two do the work.
    wall_nr, per_nr = time_ops(torch, [("get_indice_pairs", step.rulebook), ("forward", step.forward)],
                               max(args.steps // 2, 5))
    result["without_count_readback"] = {"ms_per_step": wall_nr * 1e3 / max(args.steps // 2, 5),
                                        "forward_ms": median(per_nr["forward"])}
    # Not part of the metric either: the same voxels in shuffled row order (what a voxelizer that
    # numbers voxels by first point hands over): the rulebook goes through its hash table and
    # forward through a row map.
    shuffled = Step(handle, dict(wl, shuffle=True))
    sh_ops = [("get_indice_pairs", shuffled.rulebook), ("read_counts", shuffled.read_counts),
              ("forward", shuffled.forward)]
    for _ in range(max(args.warmup // 4, 2)):
        for _, fn in sh_ops:
            fn()
    n_sh = max(args.steps // 4, 5)
    _, per_srb = time_ops(torch, [("get_indice_pairs", shuffled.rulebook)], n_sh)
    shuffled.read_counts()
    _, per_sfw = time_ops(torch, [("forward", shuffled.forward)], n_sh)
    result["shuffled_rows"] = {"rulebook_ms": median(per_srb["get_indice_pairs"]),
                               "forward_ms": median(per_sfw["forward"]), "pairs": shuffled.P}
    del shuffled
    if step.sub_m:
        result["graph_replay"] = graph_replay_step(
            torch, m, handle, step, [("get_indice_pairs", step.rulebook), ("forward", step.forward)], args.steps)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(step)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
