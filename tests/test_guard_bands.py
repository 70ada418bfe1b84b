"""The guard bands the Python wrappers put around output tensors and workspaces in the GPU tests."""
import pytest


def test_guard_bands_catch_a_write_outside_the_buffer():
    """The wrappers' guard mode (on for every GPU test): a byte changed in front of or behind an
    output tensor or workspace makes the check after the operator call raise."""
    import torch
    import mluop_hip as m
    old = m.GUARD_BYTES
    m.GUARD_BYTES = 64
    try:
        t = m._output((5, 3), torch.int32, "cpu", "some output")
        ws = m._workspace(100, "cpu")
        assert t.shape == (5, 3) and ws.numel() == 100
        t.fill_(7)
        ws.fill_(9)
        m._guards_intact("an operator")          # nothing outside was touched
        t = m._output((5, 3), torch.int32, "cpu", "some output")
        base = t.untyped_storage()
        raw = torch.empty(0, dtype=torch.uint8).set_(base)
        assert int(raw[0]) == m.GUARD_PATTERN and raw.numel() == 60 + 2 * 64
        raw[64 + 60] = 0                          # first byte behind the payload
        with pytest.raises(AssertionError, match="some output: bytes behind"):
            m._guards_intact("an operator")
        ws = m._workspace(10, "cpu")
        torch.empty(0, dtype=torch.uint8).set_(ws.untyped_storage())[63] = 1
        with pytest.raises(AssertionError, match="workspace: bytes in front"):
            m._guards_intact("an operator")
    finally:
        m.GUARD_BYTES = old
