"""Forward on a rulebook whose report has not reached the host.

mluOpGetIndicePairs tells the host through pinned memory whether the input rows were in cell
order; a forward call enqueued before that report has arrived (no wait between the two calls, or
both captured into a graph) cannot know.  It then starts on the pair lists all the same and
enqueues the row-map kernels behind them: the first kernel's check of the lists decides on the
device which of the two do the work.  The cases here keep the queue busy in front of the
rulebook, so that the report is certainly missing when forward is called, and check

* rows in order: the list kernels alone produce the result (kernel choice `lists_on_trust` = 1
  enqueues nothing behind them), bit for bit what the call gives after a wait;
* shuffled rows: the lists fail their check, the row-map kernels produce the result;
* that the two ways give the same bits in every dtype, which is what lets the library pick
  between them by what the host happens to know."""
import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import check_close, from_torch, random_voxels, round_to, to_torch

pytestmark = pytest.mark.gpu

LIST_KERNEL = "packFilterCutPairLists"
MAP_KERNELS = ("fillMapPackFilter", "scatterRowMap")


def keep_the_queue_busy():
    """A few milliseconds of work on the current stream."""
    import torch
    a = torch.ones((4096, 4096), device="cuda", dtype=torch.float32)
    for _ in range(6):
        a = (a @ a) * 1e-4
    return a


def make_case(seed, space, L, ci, co, dtype_name, shuffle):
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, 1, space, L, shuffle=shuffle)
    feats = round_to(rng.standard_normal((L, ci)).astype(np.float32), dtype_name)
    b = 1.0 / np.sqrt(27 * ci)
    w = round_to(rng.uniform(-b, b, size=(3, 3, 3, ci, co)).astype(np.float32), dtype_name)
    return idx, feats, w


def rulebook(handle, idx, space):
    import torch
    import mluop_hip
    return mluop_hip.get_indice_pairs(handle, idx, 1, space, (3, 3, 3), list(space), [1, 1, 1], [1, 1, 1],
                                      [1, 1, 1], True)


def forward_after_a_wait(handle, idx_t, space, t_f, t_w, L):
    import torch
    import mluop_hip
    pairs, _, num, _ = rulebook(handle, idx_t, space)
    torch.cuda.synchronize()
    num_host = [int(v) for v in num.cpu().tolist()]
    handle.set_kernel_timing(True)
    out = mluop_hip.indice_conv_forward(handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, pairs, num_host, L, True)
    names = [n for n, _ in handle.kernel_timings()]
    handle.set_kernel_timing(False)
    return out, names, num_host, pairs


def forward_without_a_wait(handle, idx_t, space, t_f, t_w, L, num_host):
    import torch
    import mluop_hip
    torch.cuda.synchronize()
    # (the guard bands other tests switch on are checked after a wait for the GPU: not here)
    guard_bytes, mluop_hip.GUARD_BYTES = mluop_hip.GUARD_BYTES, 0
    try:
        handle.set_kernel_timing(True)
        busy = keep_the_queue_busy()
        pairs, _, _, _ = rulebook(handle, idx_t, space)       # a new pair tensor: a new note, no report yet
        out = mluop_hip.indice_conv_forward(handle, t_f, t_w, mluop_hip.LAYOUT_ARRAY, pairs, num_host, L, True)
        names = [n for n, _ in handle.kernel_timings()]
        handle.set_kernel_timing(False)
        torch.cuda.synchronize()
        del busy
    finally:
        mluop_hip.GUARD_BYTES = guard_bytes
    return out, names


@pytest.mark.parametrize("channels", [(64, 64), (32, 32), (128, 128)])
@pytest.mark.parametrize("dtype_name", ["float16", "float32"])
def test_rows_in_order_run_on_the_lists_before_the_report_arrives(channels, dtype_name):
    import torch
    import mluop_hip
    ci, co = channels
    space, L = (10, 40, 40), 6000
    idx, feats, w = make_case(41 + ci, space, L, ci, co, dtype_name, shuffle=False)
    handle = mluop_hip.make_handle_on_current_stream()
    idx_t = torch.from_numpy(idx).cuda()
    t_f, t_w = to_torch(feats, dtype_name, "cuda"), to_torch(w, dtype_name, "cuda")
    want, names, num_host, pairs = forward_after_a_wait(handle, idx_t, space, t_f, t_w, L)
    assert LIST_KERNEL in names and not any(k in names for k in MAP_KERNELS), names
    check_close(from_torch(want), oracle.forward(feats, w.reshape(27, ci, co), pairs.cpu().numpy(), num_host, L),
                dtype_name, "forward after a wait")
    # the list kernels and the row-map kernels are both enqueued; the result is the lists'
    got, names = forward_without_a_wait(handle, idx_t, space, t_f, t_w, L, num_host)
    assert LIST_KERNEL in names and all(k in names for k in MAP_KERNELS), names
    assert torch.equal(got, want)
    # nothing behind the list kernels: they must have done the work
    handle.set_kernel_choice("lists_on_trust", True)
    got, names = forward_without_a_wait(handle, idx_t, space, t_f, t_w, L, num_host)
    assert LIST_KERNEL in names and not any(k in names for k in MAP_KERNELS), names
    assert torch.equal(got, want)
    # switched off: the row map, as for any rulebook of unknown order
    handle.set_kernel_choice("lists_on_trust", False)
    got, names = forward_without_a_wait(handle, idx_t, space, t_f, t_w, L, num_host)
    assert LIST_KERNEL not in names and all(k in names for k in MAP_KERNELS), names
    assert torch.equal(got, want)
    handle.close()


@pytest.mark.parametrize("channels", [(64, 64), (16, 32)])
def test_shuffled_rows_fall_to_the_row_map_on_the_device(channels):
    import torch
    import mluop_hip
    ci, co = channels
    space, L = (10, 40, 40), 6000
    idx, feats, w = make_case(51 + ci, space, L, ci, co, "float16", shuffle=True)
    handle = mluop_hip.make_handle_on_current_stream()
    idx_t = torch.from_numpy(idx).cuda()
    t_f, t_w = to_torch(feats, "float16", "cuda"), to_torch(w, "float16", "cuda")
    want, names, num_host, pairs = forward_after_a_wait(handle, idx_t, space, t_f, t_w, L)
    assert LIST_KERNEL not in names, names
    check_close(from_torch(want), oracle.forward(feats, w.reshape(27, ci, co), pairs.cpu().numpy(), num_host, L),
                "float16", "forward after a wait")
    got, names = forward_without_a_wait(handle, idx_t, space, t_f, t_w, L, num_host)
    assert LIST_KERNEL in names and all(k in names for k in MAP_KERNELS), names
    assert torch.equal(got, want)
    handle.close()


@pytest.mark.parametrize("dtype_name", ["float16", "bfloat16", "float32"])
@pytest.mark.parametrize("channels", [(64, 64), (32, 32), (128, 128), (16, 16)])
def test_pair_lists_and_row_map_give_the_same_bits(channels, dtype_name):
    """One rulebook through the list kernels (the handle built it and has seen its report) and
    through the row map (the same pairs at an address the handle knows nothing about)."""
    import torch
    import mluop_hip
    ci, co = channels
    space, L = (8, 24, 24), 3000
    idx, feats, w = make_case(61 + ci, space, L, ci, co, dtype_name, shuffle=False)
    handle = mluop_hip.make_handle_on_current_stream()
    idx_t = torch.from_numpy(idx).cuda()
    t_f, t_w = to_torch(feats, dtype_name, "cuda"), to_torch(w, dtype_name, "cuda")
    by_lists, names, num_host, pairs = forward_after_a_wait(handle, idx_t, space, t_f, t_w, L)
    assert LIST_KERNEL in names, names
    other = mluop_hip.make_handle_on_current_stream()
    other.set_kernel_timing(True)
    by_map = mluop_hip.indice_conv_forward(other, t_f, t_w, mluop_hip.LAYOUT_ARRAY, pairs.clone(), num_host, L, True)
    names = [n for n, _ in other.kernel_timings()]
    assert LIST_KERNEL not in names and all(k in names for k in MAP_KERNELS), names
    assert torch.equal(by_lists, by_map)
    handle.close()
    other.close()
