"""Shared helpers for the sparse-convolution tests: seeded case construction, the
reference harness's dtype round trips, and the accuracy thresholds the reference
grades against (diff1/diff2 <= 3e-3 for half and bfloat16, <= 1e-5 for float;
rulebook exact)."""
import numpy as np

import sparse_conv_oracle as oracle

THRESH = {"float32": 1e-5, "float16": 3e-3, "bfloat16": 3e-3}


def random_voxels(rng, batch, space, L, shuffle=True, duplicates=0):
    """L distinct cells of a (batch, D, H, W) grid, optionally followed by duplicated rows."""
    D, H, W = space
    total = batch * D * H * W
    lin = rng.choice(total, size=min(L, total), replace=False)
    if not shuffle:
        lin = np.sort(lin)
    n = lin // (D * H * W)
    rem = lin % (D * H * W)
    idx = np.stack([n, rem // (H * W), (rem % (H * W)) // W, rem % W], axis=1).astype(np.int32)
    if duplicates:
        pick = rng.integers(0, idx.shape[0], size=duplicates)
        idx = np.concatenate([idx, idx[pick]], axis=0)
        if shuffle:
            idx = idx[rng.permutation(idx.shape[0])]
    return np.ascontiguousarray(idx)


def out_space(space, ks, pad, stride, dil):
    return [(i + 2 * p - d * (k - 1) - 1) // s + 1 for i, k, p, s, d in zip(space, ks, pad, stride, dil)]


def round_to(a, dtype_name):
    """fp32 values as the device tensor type will hold them."""
    if dtype_name == "float16":
        return oracle.round_through_half(a)
    if dtype_name == "bfloat16":
        return oracle.round_through_bf16(a)
    return np.asarray(a, dtype=np.float32)


def to_torch(a_fp32, dtype_name, device):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a_fp32, dtype=np.float32))
    return t.to(device=device, dtype=getattr(torch, dtype_name)).contiguous()


def from_torch(t):
    return t.detach().float().cpu().numpy()


def check_close(dev, ref_fp32, dtype_name, what=""):
    """Grade like the reference harness: the oracle output is rounded through the output
    dtype, then diff1 and diff2 must stay under the dtype's threshold."""
    ref = round_to(ref_fp32, dtype_name)
    d1 = oracle.diff1(dev, ref)
    d2 = oracle.diff2(dev, ref)
    thr = THRESH[dtype_name]
    assert np.isfinite(dev).all(), what + " non-finite output"
    assert d1 <= thr and d2 <= thr, "%s diff1=%.3e diff2=%.3e thr=%.1e" % (what, d1, d2, thr)
    return d1, d2
