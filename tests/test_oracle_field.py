"""Pins the oracle's NeuS-field composition (forward, normals, first + second order backward)."""
import numpy as np
import pytest
import torch

from torch_ref import grid_forward as t_grid_forward
from torch_ref import mlp_forward as t_mlp_forward

SH_C = [0.28209479177387814, 0.48860251190291987, 1.0925484305920792, 0.94617469575755997, 0.31539156525251999,
        0.54627421529603959, 0.59004358992664352, 2.8906114426405538, 0.45704579946446572, 0.3731763325901154,
        1.4453057213202769]


def t_sh4(d):
    x, y, z = d[0] * 2 - 1, d[1] * 2 - 1, d[2] * 2 - 1
    c = SH_C
    return torch.stack([
        torch.full_like(x, c[0]), -c[1] * y, c[1] * z, -c[1] * x, c[2] * x * y, -c[2] * y * z, c[3] * z * z - c[4],
        -c[2] * x * z, c[5] * (x * x - y * y), c[6] * y * (-3 * x * x + y * y), c[7] * x * y * z,
        c[8] * y * (1 - 5 * z * z), c[9] * z * (5 * z * z - 3), c[8] * x * (1 - 5 * z * z), c[10] * z * (x * x - y * y),
        c[6] * x * (-x * x + 3 * y * y)])


def make_field(seed=0):
    from oracle.field import Field
    f = Field(n_levels=4, log2_hashmap_size=9, base_resolution=4, per_level_scale=1.7, fp16=False)
    assert f.sdf_in_w == 16 and f.enc_w == 8
    rng = np.random.default_rng(seed)
    p = np.zeros(f.n_params, np.float32)
    p[:f.off_grid] = rng.standard_normal(f.off_grid) * 0.25
    p[f.off_grid:f.off_var] = rng.uniform(-0.5, 0.5, f.grid.n_params)
    p[f.off_var] = 0.3
    return f, p, rng


def torch_forward(f, tp, coords, idx):
    """Independent forward: returns (rgb_out[16,N], sdf_out0 + bias, normal[3,N])."""
    n = coords.shape[0]
    Ws = [tp[0:64 * f.sdf_in_w].view(64, f.sdf_in_w), tp[64 * f.sdf_in_w:f.off_rgb].view(16, 64)]
    o = f.off_rgb
    Wr = [tp[o:o + 64 * 48].view(64, 48), tp[o + 64 * 48:o + 64 * 48 + 4096].view(64, 64),
          tp[o + 64 * 48 + 4096:f.off_grid].view(16, 64)]
    G = tp[f.off_grid:f.off_var]
    xyz = torch.tensor(coords[:, 0:3].T.copy(), dtype=torch.float64, requires_grad=True)
    dirs = torch.tensor(coords[:, 4:7].T.copy(), dtype=torch.float64)
    enc = t_grid_forward(G, xyz, f.grid.scale, f.grid.offset, idx)
    pad = torch.zeros((f.sdf_in_w - 3 - f.enc_w, n), dtype=torch.float64)
    sdf_in = torch.cat([xyz - 0.5, enc, pad], 0)
    sdf_out = t_mlp_forward(Ws, sdf_in)
    (normal,) = torch.autograd.grad(sdf_out[0].sum(), xyz, create_graph=True)
    rgb_in = torch.cat([sdf_out, t_sh4(dirs), xyz, normal, torch.zeros((10, n), dtype=torch.float64)], 0)
    rgb_out = t_mlp_forward(Wr, rgb_in)
    return rgb_out, sdf_out[0] + float(f.sdf_bias), normal


def test_field_forward_and_backward_match_autograd():
    f, p, rng = make_field()
    n = 96
    coords = rng.random((n, 7)).astype(np.float32)
    out, ctx = f.forward(p, coords)
    idx, _ = f.grid.indices(ctx["xyz"])
    tp = torch.tensor(p.astype(np.float64), requires_grad=True)
    rgb_out, sdf, normal = torch_forward(f, tp, coords, idx)
    np.testing.assert_allclose(out[0:3], rgb_out[0:3].detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(out[3], sdf.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(out[4:7], normal.detach().numpy(), rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(out[7], 0.3, atol=1e-7)
    np.testing.assert_allclose(out[8:11], coords[:, 4:7].T, atol=1e-7)
    # backward: the loss functional the reference's backward_impl differentiates
    dL = rng.standard_normal((16, n)).astype(np.float32)
    B = 37  # eikonal batch-size divisor, independent of n on purpose
    tl = torch.tensor(dL.astype(np.float64))
    loss = (tl[0:3] * rgb_out[0:3]).sum() + (tl[3] * sdf).sum() + (tl[7] * tp[f.off_var]).sum() \
        + ((tl[4:7] / B + tl[8:11]) * normal).sum()
    (ref,) = torch.autograd.grad(loss, tp)
    got = f.backward(p, ctx, dL, ek_batch_size=B)
    ref = ref.numpy()
    for name, a, b in (("sdf mlp", f.off_sdf, f.off_rgb), ("rgb mlp", f.off_rgb, f.off_grid),
                       ("grid", f.off_grid, f.off_var), ("variance", f.off_var, f.n_params)):
        scale = np.abs(ref[a:b]).max() + 1e-12
        np.testing.assert_allclose(got[a:b] / scale, ref[a:b] / scale, rtol=2e-4, atol=2e-5, err_msg=name)
    # the second-order terms matter: without them the SDF-MLP gradient is visibly different
    assert np.abs(ref[f.off_sdf:f.off_rgb]).max() > 0


def test_second_order_terms_are_needed():
    """Dropping the eikonal/normal path (rows 4..6, 8..10 and the colour net's normal input) changes the gradients:
    guards against a backward that silently ignores the second-order pieces."""
    f, p, rng = make_field(1)
    n = 64
    coords = rng.random((n, 7)).astype(np.float32)
    out, ctx = f.forward(p, coords)
    dL = np.zeros((16, n), np.float32)
    dL[4:7] = rng.standard_normal((3, n))
    g = f.backward(p, ctx, dL, ek_batch_size=n)
    assert np.abs(g[f.off_grid:f.off_var]).max() > 0 and np.abs(g[f.off_sdf:f.off_rgb]).max() > 0
    assert np.all(g[f.off_rgb:f.off_grid] == 0)


def test_sdf_and_density(oracle):
    from oracle.field import Field
    f = Field(n_levels=4, log2_hashmap_size=9, base_resolution=4, per_level_scale=1.7, fp16=False)
    rng = np.random.default_rng(2)
    p = (rng.standard_normal(f.n_params) * 0.2).astype(np.float32)
    p[f.off_var] = 0.3
    coords = rng.random((40, 7)).astype(np.float32)
    out, _ = f.forward(p, coords)
    sdf = f.sdf_values(p, coords[:, :3].T.copy())
    np.testing.assert_allclose(sdf[0], out[3], rtol=1e-6, atol=1e-6)
    s = np.exp(3.0)
    sg = 1 / (1 + np.exp(-s * sdf[0].astype(np.float64)))
    np.testing.assert_allclose(f.density(p, coords[:, :3].T.copy())[0], s * sg * (1 - sg), rtol=1e-4)
