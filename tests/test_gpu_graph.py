"""The submanifold rulebook and the three convolution operators enqueue kernels only (no stream
synchronisation, no allocation, no memset nodes), so a caller can capture them into a HIP graph.
One layer's step is captured once and replayed several times, with ordinary eager calls and
synchronisations in between, and every replay must reproduce the eager results bit for bit."""
import numpy as np
import pytest

from spconv_cases import random_voxels

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows_in_order", [False, True])
def test_captured_step_replays_bit_exactly(rows_in_order):
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(31)
    batch, space, L, ci, co, ks = 2, (12, 24, 24), 5000, 64, 64, (3, 3, 3)
    idx = torch.from_numpy(random_voxels(rng, batch, space, L, shuffle=not rows_in_order)).cuda()
    feats = torch.from_numpy(rng.standard_normal((L, ci)).astype(np.float32)).cuda().half()
    w = torch.from_numpy((rng.standard_normal(ks + (ci, co)) * 0.1).astype(np.float32)).cuda().half()
    dy = torch.from_numpy(rng.standard_normal((L, co)).astype(np.float32)).cuda().half()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        handle = m.make_handle_on_current_stream()      # the handle's queue is the capture stream

        def step(num_host):
            pairs, out_idx, num, n_out = m.get_indice_pairs(handle, idx, batch, space, ks, list(space), [1, 1, 1],
                                                            [1, 1, 1], [1, 1, 1], True)
            out = m.indice_conv_forward(handle, feats, w, m.LAYOUT_ARRAY, pairs, num_host, L, True)
            dx = m.indice_conv_backward_data(handle, dy, w, m.LAYOUT_ARRAY, pairs, num_host, True, ci)
            dw = m.indice_conv_backward_filter(handle, feats, dy, pairs, num_host, ks, True)
            return pairs, num, out, dx, dw

        # eager reference (also the warm-up); indice_num goes to the host once, as a framework does
        pairs0, num0, _, _, _ = step([L] * 27)
        side.synchronize()
        num_host = num0.cpu().tolist()
        eager = [t.clone() for t in step(num_host)]
        side.synchronize()

        # Nothing runs during capture, so the captured forward cannot know whether the rows are
        # in order: list kernels and row-map kernels are both captured, and every replay decides
        # on the device which of them do the work.  For rows in order the test switch leaves the
        # row-map kernels out of the graph, so a replay that reproduces the eager bits shows that
        # the list kernels did the work; the shuffled rows need the row-map kernels.
        if rows_in_order:
            handle.set_kernel_choice("lists_on_trust", True)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = step(num_host)
        handle.set_kernel_choice("lists_on_trust", None)
        for replay in range(4):
            for t in captured:
                t.fill_(0)                               # eager work between the replays
            extra = step(num_host)                       # and an eager step on the same stream
            side.synchronize()
            graph.replay()
            side.synchronize()
            for name, got, want in zip(("pairs", "indice_num", "forward", "backward_data", "backward_filter"),
                                       captured, eager):
                assert torch.equal(got, want), "replay %d: %s" % (replay, name)
            for got, want in zip(extra, eager):
                assert torch.equal(got, want)
    torch.cuda.current_stream().wait_stream(side)
    handle.close()


def test_a_filter_of_175_offsets_is_captured_too():
    """More offsets than the kernels carry counts for in their arguments (128): the counts reach
    device memory through small launches, not through a copy the host waits for, so the three
    operators can be captured with a 5x5x7 filter as well; every replay gives the eager bits."""
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(33)
    batch, space, L, ci, co, ks = 1, (10, 16, 16), 1200, 32, 32, (5, 5, 7)
    idx = torch.from_numpy(random_voxels(rng, batch, space, L)).cuda()
    feats = torch.from_numpy(rng.standard_normal((L, ci)).astype(np.float32)).cuda().half()
    w = torch.from_numpy((rng.standard_normal(ks + (ci, co)) * 0.05).astype(np.float32)).cuda().half()
    dy = torch.from_numpy(rng.standard_normal((L, co)).astype(np.float32)).cuda().half()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        handle = m.make_handle_on_current_stream()
        pairs, _, num, _ = m.get_indice_pairs(handle, idx, batch, space, ks, list(space), [2, 2, 3], [1, 1, 1],
                                              [1, 1, 1], True)
        side.synchronize()
        num_host = num.cpu().tolist()
        assert len(num_host) == 175 and num_host[87] == L

        def step():
            out = m.indice_conv_forward(handle, feats, w, m.LAYOUT_ARRAY, pairs, num_host, L, True)
            dx = m.indice_conv_backward_data(handle, dy, w, m.LAYOUT_ARRAY, pairs, num_host, True, ci)
            dw = m.indice_conv_backward_filter(handle, feats, dy, pairs, num_host, ks, True)
            return out, dx, dw

        eager = [t.clone() for t in step()]
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = step()
        for replay in range(3):
            for t in captured:
                t.fill_(0)
            extra = step()
            side.synchronize()
            graph.replay()
            side.synchronize()
            for name, got, want in zip(("forward", "backward_data", "backward_filter"), captured, eager):
                assert torch.equal(got, want), "replay %d: %s" % (replay, name)
            for got, want in zip(extra, eager):
                assert torch.equal(got, want)
    torch.cuda.current_stream().wait_stream(side)
    handle.close()


def test_two_handles_on_two_streams_do_not_interfere():
    """Each handle owns its queue and its pinned read-back slot: two different problems enqueued
    alternately on two streams (default priority) give the results each gives alone."""
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(32)
    ks = (3, 3, 3)

    def problem(batch, space, L, ci, co, sub_m):
        idx = torch.from_numpy(random_voxels(rng, batch, space, L)).cuda()
        feats = torch.from_numpy(rng.standard_normal((L, ci)).astype(np.float32)).cuda().half()
        w = torch.from_numpy((rng.standard_normal(ks + (ci, co)) * 0.1).astype(np.float32)).cuda().half()
        ospace = list(space) if sub_m else m.regular_output_space(space, ks, [1, 1, 1], [2, 2, 2], [1, 1, 1])
        stride = [1, 1, 1] if sub_m else [2, 2, 2]
        return dict(idx=idx, feats=feats, w=w, batch=batch, space=space, ospace=ospace, stride=stride, sub_m=sub_m)

    def run(handle, p):
        pairs, out_idx, num, n_out = m.get_indice_pairs(handle, p["idx"], p["batch"], p["space"], ks, p["ospace"],
                                                        [1, 1, 1], p["stride"], [1, 1, 1], p["sub_m"])
        num_host = num.cpu().tolist()        # waits for this handle's queue only
        out = m.indice_conv_forward(handle, p["feats"], p["w"], m.LAYOUT_ARRAY, pairs, num_host, n_out, p["sub_m"])
        return pairs, num, out_idx[:n_out].clone(), out

    problems = [problem(2, (12, 24, 24), 6000, 64, 64, True), problem(1, (16, 20, 28), 4000, 32, 64, False)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    handles, alone = [], []
    for s, p in zip(streams, problems):
        with torch.cuda.stream(s):
            handles.append(m.make_handle_on_current_stream())
            alone.append(run(handles[-1], p))
            s.synchronize()
    for rep in range(3):
        together = []
        for s, h, p in zip(streams, handles, problems):
            with torch.cuda.stream(s):
                together.append(run(h, p))
        torch.cuda.synchronize()
        for got, want in zip(together, alone):
            for g, w_ in zip(got, want):
                assert torch.equal(g, w_), "repetition %d" % rep
    for h in handles:
        h.close()


def test_four_host_threads_with_a_handle_each():
    """The reference's convention: one handle per thread and queue, no shared mutable state on
    the operator path except the descriptor pool (locked).  Four host threads, each with its own
    stream and handle, run different problems at the same time (ctypes drops the interpreter lock
    during every call into the library); each result equals the one computed alone."""
    import threading
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(33)
    ks = (3, 3, 3)
    problems = []
    for t, (L, ci, co, sub_m) in enumerate([(5000, 64, 64, True), (3000, 32, 64, False), (7000, 16, 32, True),
                                            (2000, 128, 128, False)]):
        space = (10 + t, 24, 20)
        idx = torch.from_numpy(random_voxels(rng, 1, space, L)).cuda()
        feats = torch.from_numpy(rng.standard_normal((idx.shape[0], ci)).astype(np.float32)).cuda().half()
        w = torch.from_numpy((rng.standard_normal(ks + (ci, co)) * 0.1).astype(np.float32)).cuda().half()
        stride = [1, 1, 1] if sub_m else [2, 2, 2]
        ospace = list(space) if sub_m else m.regular_output_space(space, ks, [1, 1, 1], stride, [1, 1, 1])
        problems.append(dict(idx=idx, feats=feats, w=w, space=space, ospace=ospace, stride=stride, sub_m=sub_m))
    torch.cuda.synchronize()

    def run(handle, p):
        pairs, out_idx, num, n_out = m.get_indice_pairs(handle, p["idx"], 1, p["space"], ks, p["ospace"], [1, 1, 1],
                                                        p["stride"], [1, 1, 1], p["sub_m"])
        num_host = num.cpu().tolist()
        out = m.indice_conv_forward(handle, p["feats"], p["w"], m.LAYOUT_ARRAY, pairs, num_host, n_out, p["sub_m"])
        dx = m.indice_conv_backward_data(handle, out, p["w"], m.LAYOUT_ARRAY, pairs, num_host, p["sub_m"],
                                         p["feats"].shape[1])
        return [t.cpu() for t in (pairs, num, out_idx[:n_out], out, dx)]

    main = m.make_handle_on_current_stream()
    alone = [run(main, p) for p in problems]
    main.close()

    results, errors = [None] * len(problems), []
    start = threading.Barrier(len(problems))

    def worker(i):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                handle = m.make_handle_on_current_stream()
                start.wait(timeout=60)
                for _ in range(5):
                    results[i] = run(handle, problems[i])
                stream.synchronize()
                handle.close()
        except Exception as e:          # reported by the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(problems))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert all(not t.is_alive() for t in threads)
    for i, (got, want) in enumerate(zip(results, alone)):
        for g, w_ in zip(got, want):
            assert torch.equal(g, w_), "thread %d" % i


def test_a_captured_rulebook_files_no_report_in_host_memory():
    """The last kernel of an eager rulebook tells the host, through the handle's pinned memory,
    whether the rows were in cell order.  A captured rulebook must not: its replays would write
    into a slot that by then belongs to another rulebook, or to a handle that is gone.  Seen from
    outside: after a replay (and a wait) a forward call on the captured rulebook still does not
    know the order, so it enqueues the list kernels and the row-map kernels behind them."""
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(35)
    batch, space, L, c, ks = 1, (10, 20, 20), 2000, 32, (3, 3, 3)
    idx = torch.from_numpy(random_voxels(rng, batch, space, L, shuffle=False)).cuda()
    feats = torch.from_numpy(rng.standard_normal((L, c)).astype(np.float32)).cuda().half()
    w = torch.from_numpy((rng.standard_normal(ks + (c, c)) * 0.1).astype(np.float32)).cuda().half()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    guard_bytes, m.GUARD_BYTES = m.GUARD_BYTES, 0
    try:
        with torch.cuda.stream(side):
            handle = m.make_handle_on_current_stream()

            def rulebook():
                return m.get_indice_pairs(handle, idx, batch, space, ks, list(space), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)

            pairs0, _, num0, _ = rulebook()
            side.synchronize()
            num_host = num0.cpu().tolist()
            want = m.indice_conv_forward(handle, feats, w, m.LAYOUT_ARRAY, pairs0, num_host, L, True)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                pairs, _, _, _ = rulebook()
            graph.replay()
            side.synchronize()
            assert torch.equal(pairs, pairs0)
            handle.set_kernel_timing(True)
            got = m.indice_conv_forward(handle, feats, w, m.LAYOUT_ARRAY, pairs, num_host, L, True)
            names = [n for n, _ in handle.kernel_timings()]
            handle.set_kernel_timing(False)
            assert "packFilterCutPairLists" in names and "scatterRowMap" in names, names
            assert torch.equal(got, want)
        torch.cuda.current_stream().wait_stream(side)
        handle.close()
    finally:
        m.GUARD_BYTES = guard_bytes


def test_a_regular_rulebook_is_refused_under_capture_and_the_capture_goes_on():
    """A rulebook that is not submanifold returns its number of output rows through the host
    descriptor, which takes a wait: during capture the call is refused before it enqueues
    anything, and what the caller captures after the refusal replays as usual."""
    import torch
    import mluop_hip as m
    rng = np.random.default_rng(36)
    batch, space, L, ks = 1, (10, 20, 20), 1500, (3, 3, 3)
    idx = torch.from_numpy(random_voxels(rng, batch, space, L, shuffle=False)).cuda()
    ospace = m.regular_output_space(space, ks, [1, 1, 1], [2, 2, 2], [1, 1, 1])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    guard_bytes, m.GUARD_BYTES = m.GUARD_BYTES, 0
    try:
        with torch.cuda.stream(side):
            handle = m.make_handle_on_current_stream()

            def submanifold():
                return m.get_indice_pairs(handle, idx, batch, space, ks, list(space), [1, 1, 1], [1, 1, 1], [1, 1, 1], True)

            def regular():
                return m.get_indice_pairs(handle, idx, batch, space, ks, ospace, [1, 1, 1], [2, 2, 2], [1, 1, 1], False)

            want_pairs, _, want_num, _ = submanifold()
            eager = regular()
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                with pytest.raises(m.MluOpError) as refused:
                    regular()
                pairs, _, num, _ = submanifold()
            assert refused.value.status == m.STATUS_NOT_SUPPORTED, refused.value
            for _ in range(2):
                pairs.fill_(7)
                graph.replay()
                side.synchronize()
                assert torch.equal(pairs, want_pairs) and torch.equal(num, want_num)
            # and outside the capture the handle builds regular rulebooks as before
            again = regular()
            side.synchronize()
            assert again[3] == eager[3] and torch.equal(again[0], eager[0]) and torch.equal(again[2], eager[2])
        torch.cuda.current_stream().wait_stream(side)
        handle.close()
    finally:
        m.GUARD_BYTES = guard_bytes
