"""Pins the oracle's MLP, SH and Adam functions."""
import os

import numpy as np
import pytest
import torch
from scipy import special

from torch_ref import mlp_forward as t_mlp_forward

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _setup(oracle, in_w, width, n_hidden, out_w, n, seed):
    rng = np.random.default_rng(seed)
    m = oracle.Mlp(in_w, width, n_hidden, out_w)
    W = (rng.standard_normal(m.n_params) * 0.3).astype(np.float32)
    x = rng.standard_normal((in_w, n)).astype(np.float32)
    return m, W, x, rng


@pytest.mark.parametrize("shape", [(48, 64, 1, 16), (48, 64, 2, 16), (32, 64, 1, 16), (16, 32, 3, 8)])
def test_mlp_forward_backward_vs_torch(oracle, shape):
    m, W, x, rng = _setup(oracle, *shape, n=257, seed=1)
    y, h = m.forward(W, x)
    tW = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in m.split(W)]
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ty = t_mlp_forward(tW, tx)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-4, atol=1e-4)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    (ty * torch.tensor(dy, dtype=torch.float64)).sum().backward()
    dx, dW = m.backward(W, x, h, dy)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(dW, np.concatenate([w.grad.numpy().ravel() for w in tW]), rtol=1e-4, atol=2e-3)
    # Ignore mode: no weight gradient requested
    dx2, none = m.backward(W, x, h, dy, want_dW=False)
    assert none is None
    np.testing.assert_array_equal(dx, dx2)


@pytest.mark.parametrize("shape", [(48, 64, 1, 16), (48, 64, 2, 16), (16, 32, 3, 8)])
def test_mlp_backward_backward_input_vs_double_backward(oracle, shape):
    m, W, x, rng = _setup(oracle, *shape, n=200, seed=2)
    y, h = m.forward(W, x)
    g = rng.standard_normal(y.shape).astype(np.float32)
    v = rng.standard_normal(x.shape).astype(np.float32)
    tW = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in m.split(W)]
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tg = torch.tensor(g, dtype=torch.float64, requires_grad=True)
    ty = t_mlp_forward(tW, tx)
    (q,) = torch.autograd.grad(ty, tx, tg, create_graph=True)
    s = (q * torch.tensor(v, dtype=torch.float64)).sum()
    grads = torch.autograd.grad(s, tW + [tg])
    dW, out = m.backward_backward_input(W, h, v, g)
    np.testing.assert_allclose(dW, np.concatenate([w.numpy().ravel() for w in grads[:-1]]), rtol=1e-4, atol=3e-3)
    np.testing.assert_allclose(out, grads[-1].numpy(), rtol=1e-4, atol=1e-4)
    base = rng.standard_normal(m.n_params).astype(np.float32)
    dW2, _ = m.backward_backward_input(W, h, v, g, dW=base.copy())
    np.testing.assert_allclose(dW2, base + dW, rtol=1e-5, atol=1e-4)


def test_geometric_init_fixture_is_a_sphere(oracle):
    """utils/mlp_weights.txt with zero grid features: sdf ~ |x - 0.5| (statistical, 64 neurons)."""
    W = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))
    assert W.size == 4096
    W0 = W[:64 * 48].reshape(64, 48)
    assert np.all(W0[:, 3:] == 0) and np.abs(W0[:, :3]).max() > 0
    np.testing.assert_allclose(W[64 * 48:64 * 48 + 64], np.sqrt(np.pi) / 8, atol=5e-5)
    m = oracle.Mlp(48, 64, 1, 16)
    rng = np.random.default_rng(0)
    p = rng.random((3, 4000)).astype(np.float32)
    x = np.zeros((48, 4000), np.float32)
    x[:3] = p - 0.5
    y, h = m.forward(W, x)
    r = np.linalg.norm(p - 0.5, axis=0)
    # 64 random neurons only approximate the cone |x - 0.5|: check slope, offset and correlation
    slope, icpt = np.polyfit(r, y[0], 1)
    assert abs(slope - 1) < 0.15 and abs(icpt) < 0.02
    assert np.corrcoef(y[0], r)[0, 1] > 0.75
    np.testing.assert_allclose(y[1:], np.broadcast_to(y[0], y[1:].shape), rtol=1e-3, atol=1e-4)  # all W1 rows equal
    e0 = np.zeros_like(y)
    e0[0] = 1
    dx, _ = m.backward(W, x, h, e0, want_dW=False)
    n = dx[:3]
    norm = np.linalg.norm(n, axis=0)
    assert abs(norm.mean() - 1) < 0.25
    far = r > 0.2
    cos = (n * (p - 0.5)).sum(0)[far] / (norm[far] * r[far])
    assert cos.mean() > 0.8


def test_sh4_matches_scipy(oracle):
    rng = np.random.default_rng(3)
    d = rng.standard_normal((3, 500))
    d /= np.linalg.norm(d, axis=0)
    out = oracle.sh4(((d + 1) / 2).astype(np.float32))
    x, y, z = d
    theta, phi = np.arccos(np.clip(z, -1, 1)), np.arctan2(y, x)
    k = 0
    for l in range(4):
        for m in range(-l, l + 1):
            Y = special.sph_harm_y(l, abs(m), theta, phi)
            # real harmonics that keep the Condon-Shortley phase of the complex ones
            if m < 0:
                ref = np.sqrt(2) * Y.imag
            elif m == 0:
                ref = Y.real
            else:
                ref = np.sqrt(2) * Y.real
            np.testing.assert_allclose(out[k], ref, atol=2e-5, err_msg=f"l={l} m={m}")
            k += 1


def test_adam_matches_torch_on_matrix_params(oracle):
    rng = np.random.default_rng(4)
    n = 1000
    w0 = rng.standard_normal(n).astype(np.float32)
    w, m1, m2 = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    steps = np.zeros(n, np.uint32)
    tw = torch.tensor(w0.astype(np.float64), requires_grad=True)
    # l2_reg as a gradient term == torch's (coupled) weight_decay
    opt = torch.optim.Adam([tw], lr=1e-3, betas=(0.9, 0.99), eps=1e-15, weight_decay=1e-6)
    for it in range(5):
        g = rng.standard_normal(n).astype(np.float32)
        tw.grad = torch.tensor(g.astype(np.float64))
        opt.step()
        oracle.adam_step(w, g * 128.0, m1, m2, steps, n_matrix_params=n)
        np.testing.assert_allclose(w, tw.detach().numpy(), rtol=2e-5, atol=2e-6)
    assert (steps == 5).all()


def test_adam_non_matrix_rules(oracle):
    n = 8
    w = np.ones(n, np.float32)
    m1, m2, steps = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint32)
    g = np.array([0, 1, 0, 1, 0, 1, 0, 1], np.float32) * 128
    oracle.adam_step(w, g, m1, m2, steps, n_matrix_params=4)
    # matrix params always step (l2 pulls them even at g == 0); non-matrix with g == 0 are untouched
    assert steps.tolist() == [1, 1, 1, 1, 0, 1, 0, 1]
    assert w[4] == 1 and w[6] == 1 and m1[4] == 0
    assert w[0] < 1  # l2_reg
    # first step of Adam moves by ~lr regardless of gradient magnitude
    np.testing.assert_allclose(1 - w[5], 1e-3, rtol=1e-3)
    # second call: the skipped params still have step 0 -> their first update is bias-corrected as t=1
    oracle.adam_step(w, np.full(n, 128, np.float32), m1, m2, steps, n_matrix_params=4)
    assert steps.tolist() == [2, 2, 2, 2, 1, 2, 1, 2]
    np.testing.assert_allclose(1 - w[4], 1e-3, rtol=1e-3)


def test_round_fp16_matches_numpy(oracle):
    rng = np.random.default_rng(9)
    a = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-9, 5, 20000),
                        [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 6.1e-5, 6.0e-5, 5.96e-8, 2.9e-8, 3.0e-8,
                         1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, np.inf, -np.inf]]).astype(np.float32)
    with np.errstate(over="ignore"):
        ref = a.astype(np.float16).astype(np.float32)
    got = oracle.round_fp16(a)
    np.testing.assert_array_equal(got, ref)


def test_mlp_forward_fp16_hidden_option(oracle):
    m, W, x, _ = _setup(oracle, 48, 64, 2, 16, n=64, seed=5)
    y0, h0 = m.forward(W, x)
    y1, h1 = m.forward(W, x, round_hidden=True)
    np.testing.assert_array_equal(h1[0], h0[0].astype(np.float16).astype(np.float32))
    assert np.abs(y1 - y0).max() < 2e-2 and not np.array_equal(y1, y0)
