"""SDF network with the eikonal second-order path (grid + 48-64-16 MLP, loss = mean|sdf| + 0.1 mean(|grad sdf| - 1)^2):
forward, normals and every parameter gradient against the same composition of the oracle's pieces."""
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, assert_grad_close, dev, host, q16, rel_l2

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("kind", ["uniform", "rays"])
def test_sdf_eikonal_step_matches_oracle(oracle, kind):
    from neus2_amd.sdf_net import SdfNet
    rng = np.random.default_rng(7)
    n = 8192
    net = SdfNet(max_batch=n)
    P = q16(rng.uniform(-0.01, 0.01, net.grid.n_params()))  # gradient norms around 1 +- a few tenths; larger tables overflow fp16 gradients
    W = q16(np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")) + rng.normal(0, 0.05, 4096))
    if kind == "uniform":
        x = rng.random((3, n), dtype=np.float32)
    else:
        o = 0.3 + 0.4 * rng.random((n // 64, 1, 3))
        d = rng.standard_normal((n // 64, 1, 3))
        d /= np.linalg.norm(d, axis=-1, keepdims=True)
        x = np.clip(o + d * (np.arange(64).reshape(1, 64, 1) - 32) * (np.sqrt(3.0) / 1024), 0, 1).reshape(-1, 3).T.astype(np.float32).copy()
    dP, dW = dev(P, torch.float16), dev(W, torch.float16)
    gP, gW = torch.zeros_like(dP), torch.zeros_like(dW)
    net.set_params(dP, gP, dW, gW)
    ctx = net.forward(dev(x))
    loss = float(net.loss_backward(ctx, ek_weight=0.1, loss_scale=128.0).item())
    from oracle.sdf_step import sdf_eikonal_step
    ref = sdf_eikonal_step(P, W, x, 0.1, 128.0)
    assert_close(host(ctx["sdf"]), ref["sdf"], what="sdf", outlier_frac=1e-3)
    assert_close(host(ctx["normal"]), ref["normal"], what="normal", outlier_frac=2e-3)
    assert abs(loss - ref["loss"]) <= 2e-3 * abs(ref["loss"])
    assert_grad_close(host(gW), ref["mlp_grad"], what="MLP gradient", rtol=5e-3)
    got = host(gP)
    for l in range(16):
        a, b = int(ref["offset"][l]) * 2, int(ref["offset"][l + 1]) * 2
        assert rel_l2(got[a:b], ref["grid_grad"][a:b]) < 5e-3, (l, rel_l2(got[a:b], ref["grid_grad"][a:b]))
