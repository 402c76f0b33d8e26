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


def assert_close(got, ref, rtol=RTOL, what="", scale=None, outlier_frac=0.0):
    """|got - ref| <= rtol * (|ref| + scale), scale defaulting to the RMS of ref: the
    relative tolerance of the contract with an absolute floor for entries near zero.
    outlier_frac: fraction of entries allowed outside the band (ReLU masks of
    pre-activations that sit within rounding error of zero may flip)."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    if scale is None:
        scale = float(np.sqrt(np.mean(ref ** 2))) if ref.size else 0.0
    err = np.abs(got - ref)
    bound = rtol * (np.abs(ref) + scale)
    bad = err > bound
    if bad.sum() > outlier_frac * bad.size:
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside rtol={rtol}; worst at {i}: "
                             f"got {got[i]:.6g} ref {ref[i]:.6g} (scale {scale:.3g}, rel_l2 {rel_l2(got, ref):.3g})")


def assert_grad_close(got, ref, what="", rtol=RTOL):
    """Batch-summed weight gradients.  One ReLU mask that lands on the other side of zero
    (see FLIP in the MLP tests) shifts a whole row and column of dW by one sample's
    contribution, so the contract is stated on the norm: relative L2 error <= rtol, and no
    entry further than 5% of the RMS from the oracle."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    scale = float(np.sqrt(np.mean(ref ** 2)))
    r = rel_l2(got, ref)
    worst = float(np.abs(got - ref).max())
    assert r <= rtol, f"{what}: rel_l2 {r:.3g} > {rtol}"
    assert worst <= 0.05 * scale + rtol * float(np.abs(ref).max()), f"{what}: max error {worst:.3g} vs rms {scale:.3g}"
