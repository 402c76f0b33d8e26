"""Parity at the benchmark's full sizes (2^18-sample batches, the 512^3 lattice), through the C ABI.

The smaller tests compare everything with the oracle; here the launches have the shapes the benchmark uses (all
workgroup counts, the bucketed scatter with every level's real bucket plan, several lattice chunks) and are checked
 * directly against the oracle where it finishes in seconds (its C core is OpenMP code),
 * and through size-independent properties: the corner weights of a point sum to one, so a level's gradient entries
   add up to the column sums of dL_dy (a checksum of checksums); the scatter is linear in dL_dy; lattice values do not
   depend on how the lattice is cut into chunks.
"""
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, assert_grad_close, dev, host, q16, rel_l2

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
N = 1 << 18
CFG = dict(n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447)


@pytest.fixture(scope="module")
def grid(oracle):
    from neus2_amd.tcnn_api import GridEncoding
    og = oracle.Grid(CFG["n_levels"], CFG["log2_hashmap_size"], CFG["base_resolution"], CFG["per_level_scale"])
    gg = GridEncoding(**CFG)
    rng = np.random.default_rng(2)
    params = q16(rng.uniform(-1, 1, og.n_params))
    dp = dev(params, torch.float16)
    dg = torch.zeros_like(dp)
    gg.set_params(dp, dg)
    assert gg.reserve_scatter_workspace(N)
    xyz = rng.random((3, N), dtype=np.float32)
    dy = q16(rng.standard_normal((32, N)))
    return og, gg, params, dg, xyz, dy, rng


def level_slices(og):
    return [(2 * int(og.offset[l]), 2 * int(og.offset[l + 1])) for l in range(og.n_levels)]


def test_grid_forward_2p18_against_oracle(grid):
    """The benchmark's grid-only configuration: 2^18 uniform points, every value and derivative against the oracle."""
    og, gg, params, dg, xyz, dy, rng = grid
    ref_y, ref_j = og.forward(params, xyz, want_dy_dx=True)
    y, ctx = gg.forward(dev(xyz), prepare_input_gradients=True)
    assert_close(host(y), ref_y, what="grid output at 2^18")
    assert_close(host(ctx), ref_j, rtol=1e-4, what="dy_dx at 2^18")
    idx = host(gg.corner_indices(dev(xyz)))
    ref_idx, _ = og.indices(xyz)
    assert np.array_equal(idx, ref_idx)  # bit exact: 2^18 x 16 x 8 indices


def test_grid_scatter_2p18_against_oracle_and_checksums(grid):
    from neus2_amd.tcnn_api import GRAD_OVERWRITE
    og, gg, params, dg, xyz, dy, rng = grid
    d_xyz = dev(xyz)
    ref, _ = og.backward(params, xyz, dy, want_dx=False)
    dg.fill_(9.0)
    gg.backward(None, d_xyz, dev(dy, torch.float16), mode=GRAD_OVERWRITE)
    got = host(dg)
    col = dy.astype(np.float64).sum(1)  # [32]: per level and feature
    for l, (a, b) in enumerate(level_slices(og)):
        # sorted path: fp32 / fixed-point accumulation, one rounding to fp16 per entry
        assert rel_l2(got[a:b], ref[a:b]) < RTOL, (l, rel_l2(got[a:b], ref[a:b]))
        # weights of a point's 8 corners sum to 1: the level's entries add up to the column sums of dL_dy.
        # Every entry carries one fp16 rounding (relative 2^-11), random in sign.
        for f in range(2):
            s = got[a + f:b:2].astype(np.float64).sum()
            slack = 2.0 ** -11 * np.sqrt((got[a + f:b:2].astype(np.float64) ** 2).sum()) * 6 + 1e-3
            assert abs(s - col[2 * l + f]) < slack, (l, f, s, col[2 * l + f], slack)
    # linearity in dL_dy: scatter(2 dy1 - dy2) = 2 scatter(dy1) - scatter(dy2)
    dy2 = q16(rng.standard_normal((32, N)))
    gg.backward(None, d_xyz, dev(dy2, torch.float16), mode=GRAD_OVERWRITE)
    got2 = host(dg)
    gg.backward(None, d_xyz, dev(q16(2 * dy - dy2), torch.float16), mode=GRAD_OVERWRITE)
    got3 = host(dg)
    assert rel_l2(got3, 2 * got - got2) < 2 * RTOL


def test_field_step_2p18_against_oracle(oracle):
    """The benchmark's SDF-net configuration at 2^18 samples: forward, normals, first- and second-order backward of the whole
    field against the oracle's field."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, NerfNetwork
    from oracle.field import Field
    of, gf = Field(fp16=True), NerfNetwork()
    rng = np.random.default_rng(3)
    p = np.zeros(of.n_params, np.float32)
    p[:of.off_rgb] = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))
    p[of.off_rgb:of.off_grid] = rng.standard_normal(of.off_grid - of.off_rgb) * 0.2
    p[of.off_grid:of.off_var] = rng.uniform(-0.05, 0.05, of.grid.n_params)
    p[of.off_var] = 0.3
    p = q16(p)
    dp = dev(p, torch.float16)
    dg = torch.zeros_like(dp)
    gf.set_params(dp, dg)
    coords = rng.random((N, 7)).astype(np.float32)
    d = rng.standard_normal((N, 3))
    coords[:, 4:7] = (d / np.linalg.norm(d, axis=1, keepdims=True) + 1) / 2
    coords[:, 3] = 0
    # batch-summed gradients must stay inside the fp16 range of the gradient buffer
    dL = q16(rng.standard_normal((16, N)) * np.array([.02, .02, .02, .02, .5, .5, .5, .02, .001, .001, .001, 0, 0, 0, 0, 0])[:, None])
    ref_out, ctx = of.forward(p, coords)
    ref = of.backward(p, ctx, dL, ek_batch_size=N)
    d_coords = dev(coords)
    out = host(gf.forward(d_coords)).T
    for name, rows in (("rgb", slice(0, 3)), ("sdf", slice(3, 4)), ("normal", slice(4, 7)), ("variance", slice(7, 8))):
        assert_close(out[rows], ref_out[rows], what=f"field output {name} at 2^18", outlier_frac=2e-4)
    gf.backward(d_coords, dev(np.ascontiguousarray(dL.T), torch.float16), ek_batch_size=N, mode=GRAD_OVERWRITE)
    got = host(dg)
    assert_grad_close(got[of.off_sdf:of.off_rgb], ref[of.off_sdf:of.off_rgb], what="SDF MLP gradients at 2^18", rtol=2 * RTOL)
    assert_grad_close(got[of.off_rgb:of.off_grid], ref[of.off_rgb:of.off_grid], what="colour MLP gradients at 2^18", rtol=2 * RTOL)
    for l in range(16):
        a = of.off_grid + 2 * int(of.grid.offset[l])
        b = of.off_grid + 2 * int(of.grid.offset[l + 1])
        assert rel_l2(got[a:b], ref[a:b]) < 2 * RTOL, (l, rel_l2(got[a:b], ref[a:b]))


def test_lattice_512_chunks_and_subsample(oracle):
    """The benchmark's mesh-inference configuration: the SDF over the 512^3 lattice in 2^22-point chunks.  A random subsample
    is compared with the oracle; cutting the lattice into other chunk sizes gives the same bits."""
    from neus2_amd.mesh import density_on_grid
    from neus2_amd.tcnn_api import NerfNetwork
    from neus2_amd.training import initial_parameters
    from oracle.field import Field
    net = NerfNetwork()
    p = q16(initial_parameters(net.param_offsets(), 48, seed=1, sdf_mlp_weights=np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))))
    params = dev(p, torch.float16)
    net.set_params(params, None)
    net.reserve(1 << 22)
    R = 512
    d = density_on_grid(net._h, (R, R, R), chunk=1 << 22)
    assert tuple(d.shape) == (R, R, R)
    rng = np.random.default_rng(5)
    pick = rng.integers(0, R ** 3, 8192)
    x, y, z = pick % R, (pick // R) % R, pick // (R * R)
    pos = np.stack([x, y, z]).astype(np.float32) * np.float32(1.0 / R)
    want = Field(fp16=True).sdf_values(p, pos)[0]
    got = host(d.view(-1)[torch.from_numpy(pick).cuda()])
    assert_close(got, want, rtol=RTOL, what="SDF on the 512^3 lattice", outlier_frac=1e-3)
    # the geometric initialisation: a sphere of radius ~0.1 around the centre
    r = np.linalg.norm(pos - 0.5, axis=0)
    assert np.corrcoef(got, r)[0, 1] > 0.75  # 64 random neurons: a lumpy sphere
    sub = d[:64].clone()  # 64 z-slices = 2^24 points
    del d
    for chunk in (1 << 20, (1 << 21) + 8 * 977):  # the second one does not divide the lattice
        e = density_on_grid(net._h, (R, R, 64), (0, 0, 0), (1, 1, 64 / R), chunk=chunk)
        assert torch.equal(e, sub), chunk
        del e


def test_sdf_eikonal_step_2p18_against_oracle(oracle):
    """BASELINE configuration 3 at its full size, through the entry points that configuration's benchmark times
    (n2_sdf_pack_input, n2_grid_forward with the Jacobian, n2_mlp_forward_and_input_gradient, n2_sdf_eikonal_loss,
    n2_mlp_backward, n2_grid_backward_fused, n2_mlp_backward_backward_input): 2^18 points uniform in the unit cube, the
    SDF, the normals, the loss, the MLP's weight gradients and the encoding's gradients level by level against the oracle's
    composition, at the tolerances of the small test (nerf_network.h:184-238, 402-429, 534-571)."""
    from neus2_amd.sdf_net import SdfNet
    from oracle.sdf_step import sdf_eikonal_step
    rng = np.random.default_rng(70)
    n = 1 << 18
    net = SdfNet(max_batch=n)
    P = q16(rng.uniform(-0.01, 0.01, net.grid.n_params()))
    W = q16(np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")) + rng.normal(0, 0.05, 4096))
    x = rng.random((3, n), dtype=np.float32)
    dP, dW = dev(P, torch.float16), dev(W, torch.float16)
    gP, gW = torch.zeros_like(dP), torch.zeros_like(dW)
    net.set_params(dP, gP, dW, gW)
    ctx = net.forward(dev(x))
    loss = float(net.loss_backward(ctx, ek_weight=0.1, loss_scale=128.0).item())
    ref = sdf_eikonal_step(P, W, x, 0.1, 128.0)
    assert_close(host(ctx["sdf"]), ref["sdf"], what="sdf", outlier_frac=1e-3)
    assert_close(host(ctx["normal"]), ref["normal"], what="normal", outlier_frac=2e-3)
    assert abs(loss - ref["loss"]) <= 2e-3 * abs(ref["loss"])
    assert_grad_close(host(gW), ref["mlp_grad"], what="MLP gradient", rtol=5e-3)
    got = host(gP)
    for l in range(16):
        a, b = int(ref["offset"][l]) * 2, int(ref["offset"][l + 1]) * 2
        assert rel_l2(got[a:b], ref["grid_grad"][a:b]) < 5e-3, (l, rel_l2(got[a:b], ref["grid_grad"][a:b]))
    # a second run of the same step leaves the same bits (sorted scatter, fixed-order sums)
    g1 = gP.clone()
    w1 = gW.clone()
    ctx = net.forward(dev(x))
    net.loss_backward(ctx, ek_weight=0.1, loss_scale=128.0)
    assert torch.equal(g1, gP) and torch.equal(w1, gW)
