"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

# Stated tolerance of the contract: fp16 outputs and gradients within 2e-3
# (relative) of the fp32 oracle evaluated on the same fp16-quantised inputs.
RTOL = 2e-3


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    return t.detach().float().cpu().numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.detach().cpu().numpy()


def q16(a):
    """Round an fp32 array to fp16 and back (what the GPU sees)."""
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def assert_close(got, ref, rtol=RTOL, what="", scale=None):
    """|got - ref| <= rtol * (|ref| + scale), scale defaulting to the RMS of ref: the
    relative tolerance of the contract with an absolute floor for entries near zero."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    if scale is None:
        scale = float(np.sqrt(np.mean(ref ** 2))) if ref.size else 0.0
    err = np.abs(got - ref)
    bound = rtol * (np.abs(ref) + scale)
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside rtol={rtol}; worst at {i}: "
                             f"got {got[i]:.6g} ref {ref[i]:.6g} (scale {scale:.3g}, rel_l2 {rel_l2(got, ref):.3g})")
