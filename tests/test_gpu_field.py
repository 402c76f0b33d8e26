"""GPU parity of the NeuS field (NerfNetwork forward / backward / sdf / density) against the oracle."""
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, assert_grad_close, dev, host, q16, rel_l2

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FLIP = 2e-4


def make(oracle, seed=0, geometric_init=False, **cfg):
    from neus2_amd.tcnn_api import NerfNetwork
    from oracle.field import Field
    of = Field(fp16=True, **cfg)
    gf = NerfNetwork(**cfg)
    assert gf.n_params() == of.n_params
    assert gf.param_offsets() == [of.off_sdf, of.off_rgb, of.off_grid, of.off_var, of.n_params]
    rng = np.random.default_rng(seed)
    p = np.zeros(of.n_params, np.float32)
    if geometric_init and of.sdf_in_w == 48:
        p[:of.off_rgb] = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))
        p[of.off_grid:of.off_var] = rng.uniform(-1e-4, 1e-4, of.grid.n_params)
    else:
        p[:of.off_rgb] = rng.standard_normal(of.off_rgb) * 0.2
        p[of.off_grid:of.off_var] = rng.uniform(-0.5, 0.5, of.grid.n_params)
    p[of.off_rgb:of.off_grid] = rng.standard_normal(of.off_grid - of.off_rgb) * 0.2
    p[of.off_var] = 0.3
    p = q16(p)
    dp = dev(p, torch.float16)
    dg = torch.zeros_like(dp)
    gf.set_params(dp, dg)
    return of, gf, p, dp, dg, rng


def rand_coords(rng, n):
    c = rng.random((n, 7)).astype(np.float32)
    d = rng.standard_normal((n, 3))
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    c[:, 4:7] = (d + 1) / 2
    c[:, 3] = 0
    return c


@pytest.mark.parametrize("geo", [False, True])
def test_forward_full_config(oracle, geo):
    of, gf, p, *_, rng = make(oracle, seed=1, geometric_init=geo)
    n = 4096
    coords = rand_coords(rng, n)
    ref, _ = of.forward(p, coords)
    out = host(gf.forward(dev(coords))).T
    # rows 11..15 are unused colour-net outputs but still defined: compare everything
    for name, rows in (("rgb", slice(0, 3)), ("sdf", slice(3, 4)), ("normal", slice(4, 7)), ("variance", slice(7, 8)),
                       ("dir", slice(8, 11)), ("tail", slice(11, 16))):
        assert_close(out[rows], ref[rows], what=f"field output {name}", outlier_frac=FLIP)
    if geo:
        r = np.linalg.norm(coords[:, :3] - 0.5, axis=1)
        assert np.corrcoef(out[3], r)[0, 1] > 0.75  # the sphere of the geometric init


def test_backward_full_config(oracle):
    of, gf, p, dp, dg, rng = make(oracle, seed=2)
    n = 8192
    coords = rand_coords(rng, n)
    # magnitudes chosen so that batch-summed gradients stay inside the fp16 range of the gradient buffer
    dL = q16(rng.standard_normal((16, n)) * np.array([.1, .1, .1, .1, 3, 3, 3, .1, .003, .003, .003, 0, 0, 0, 0, 0])[:, None])
    ref_out, ctx = of.forward(p, coords)
    ref = of.backward(p, ctx, dL, ek_batch_size=n)
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE
    d_coords = dev(coords)
    gf.forward(d_coords)
    dg.fill_(5.0)
    d_dL = dev(np.ascontiguousarray(dL.T), torch.float16)
    gf.backward(d_coords, d_dL, ek_batch_size=n, mode=GRAD_OVERWRITE)
    got = host(dg)
    assert_grad_close(got[of.off_sdf:of.off_rgb], ref[of.off_sdf:of.off_rgb], what="SDF MLP gradients (1st + 2nd order)",
                      rtol=2 * RTOL)
    assert_grad_close(got[of.off_rgb:of.off_grid], ref[of.off_rgb:of.off_grid], what="colour MLP gradients", rtol=2 * RTOL)
    # one fp16 rounding of a sum accumulated in fp32
    var_floor = 1e-5 * float(np.abs(dL[7]).sum()) + 1e-6
    assert abs(got[of.off_var] - ref[of.off_var]) <= RTOL * abs(ref[of.off_var]) + var_floor, (got[of.off_var], ref[of.off_var])
    for l in range(16):
        a = of.off_grid + 2 * int(of.grid.offset[l])
        b = of.off_grid + 2 * int(of.grid.offset[l + 1])
        k = 8.0 * n / max(1, int(of.grid.entries[l]))
        tol = 2 * RTOL * max(1.0, np.sqrt(k))
        assert rel_l2(got[a:b], ref[a:b]) < tol, (l, rel_l2(got[a:b], ref[a:b]), tol)
    # Accumulate doubles everything
    gf.backward(d_coords, d_dL, ek_batch_size=n, mode=GRAD_ACCUMULATE)
    got2 = host(dg)
    assert rel_l2(got2[:of.off_grid], 2 * ref[:of.off_grid]) < 3 * RTOL
    assert rel_l2(got2[of.off_grid:of.off_var], 2 * ref[of.off_grid:of.off_var]) < 2e-2
    # ... the variance gradient too (every backward sums its own batch, nothing is left over from the first call)
    assert abs(got2[of.off_var] - 2 * ref[of.off_var]) <= 3 * RTOL * abs(ref[of.off_var]) + 2 * var_floor, (got2[of.off_var], ref[of.off_var])


def test_backward_reference_14_level_config(oracle):
    """configs/nerf/base.json ships 14 levels -> SDF net input width 32 (the second weight fixture)."""
    cfg = dict(n_levels=14, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.4472692012786865)
    of, gf, p, dp, dg, rng = make(oracle, seed=3, **cfg)
    assert of.sdf_in_w == 32
    n = 2048
    coords = rand_coords(rng, n)
    dL = q16(rng.standard_normal((16, n)))
    ref_out, ctx = of.forward(p, coords)
    out = host(gf.forward(dev(coords))).T
    assert_close(out[:11], ref_out[:11], what="14-level output", outlier_frac=FLIP)
    ref = of.backward(p, ctx, dL, ek_batch_size=1 << 18)
    gf.backward(dev(coords), dev(np.ascontiguousarray(dL.T), torch.float16), ek_batch_size=1 << 18)
    got = host(dg)
    assert_grad_close(got[:of.off_grid], ref[:of.off_grid], what="MLP gradients", rtol=2 * RTOL)
    assert rel_l2(got[of.off_grid:of.off_var], ref[of.off_grid:of.off_var]) < 1e-2


def test_sdf_and_density(oracle):
    of, gf, p, *_, rng = make(oracle, seed=4)
    n = 4096
    xyz = rng.random((3, n), dtype=np.float32)
    ref = of.sdf_values(p, xyz)
    got = host(gf.sdf(dev(xyz)))
    assert_close(got, ref, what="NerfNetwork::sdf", outlier_frac=FLIP)
    refd = of.density(p, xyz)
    gotd = host(gf.density(dev(xyz)))
    assert_close(gotd[0], refd[0], rtol=5e-3, what="NerfNetwork::density")
    # the row-per-point layout gives the same answer
    rows = np.zeros((n, 7), np.float32)
    rows[:, :3] = xyz.T
    assert torch.equal(gf.sdf(dev(rows)), gf.sdf(dev(xyz)))


def test_field_errors(oracle):
    from neus2_amd.tcnn_api import N2Error, NerfNetwork
    gf = NerfNetwork()
    c = torch.rand((64, 7), device="cuda")
    with pytest.raises(N2Error, match="set_params"):
        gf.forward(c)
    gf.set_params(torch.zeros(gf.n_params(), dtype=torch.float16, device="cuda"), None)
    gf.forward(c)
    with pytest.raises(N2Error, match="gradient buffer"):
        gf.backward(c, torch.zeros((64, 16), dtype=torch.float16, device="cuda"))
    with pytest.raises(N2Error, match="multiple of 8"):
        gf.forward(torch.rand((12, 7), device="cuda"))
    assert gf.forward(torch.rand((0, 7), device="cuda")).shape == (0, 16)


def test_select_equals_forward_on_the_selected_samples(oracle):
    """n2_field_select: backward over samples picked from the last forward (with repeats and gaps, odd and even counts)
    gives exactly the gradients of a forward over those samples' coordinates followed by the same backward."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, N2Error
    of, gf, p, dp, dg, rng = make(oracle, seed=6)
    n_src = 6000
    coords = rand_coords(rng, n_src)
    d_coords = dev(coords)
    for n in (4096, 5000):  # (smaller batches scatter with fp16 atomics, whose order of arrival is not reproducible)
        idx = np.sort(rng.integers(0, n_src, n)).astype(np.int32)
        idx[-40:] = idx[:40]  # roll-over style repeats, out of order
        dL = q16(rng.standard_normal((n, 16)) * np.array([.1, .1, .1, .1, 3, 3, 3, .1, .003, .003, .003, 0, 0, 0, 0, 0]))
        d_dL = dev(dL, torch.float16)
        sub = dev(coords[idx])
        gf.forward(sub)
        dg.fill_(3.0)
        gf.backward(sub, d_dL, ek_batch_size=n, mode=GRAD_OVERWRITE)
        want = dg.clone()
        gf.forward(d_coords)
        gf.select(dev(idx, torch.int32), n_src)
        dg.fill_(3.0)  # (the three spare variance slots are never written)
        gf.backward(sub, d_dL, ek_batch_size=n, mode=GRAD_OVERWRITE)
        assert torch.equal(dg, want), n
    # the batch of a backward must be the selection (or the forward) that precedes it
    with pytest.raises(N2Error):
        gf.backward(d_coords, dev(q16(rng.standard_normal((n_src, 16))), torch.float16), ek_batch_size=n_src)
    with pytest.raises(N2Error):
        gf.select(dev(idx, torch.int32), n_src + 8)


def test_padding_rows_follow_the_batch_size(oracle):
    """The inputs of the two networks are padded to 48 rows; the padding rows are cleared once per batch size and never
    written again.  Starting from a workspace full of NaNs, batches of changing sizes (the rows move with the row pitch),
    the SDF-only path and a backward through a selection all agree with the oracle."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE
    of, gf, p, dp, dg, rng = make(oracle, seed=11)
    gf.reserve(8192)
    gf._ws.fill_(0xFF)  # every fp16 of the workspace is a NaN
    for n in (4096, 2048, 8192, 4096):
        coords = rand_coords(rng, n)
        ref, ctx = of.forward(p, coords)
        out = host(gf.forward(dev(coords))).T
        assert np.isfinite(out[:11]).all(), n
        assert_close(out[:11], ref[:11], what=f"field output at n={n}", outlier_frac=FLIP)
        xyz = np.ascontiguousarray(coords[: n // 2, :3])
        sdf = host(gf.sdf(dev(xyz)))
        assert np.isfinite(sdf[0]).all()
        assert_close(sdf[0], of.sdf_values(p, xyz.T.copy())[0], what=f"sdf at n={n // 2}", outlier_frac=FLIP)
    # a backward through a selection of half the last batch
    n = 4096
    coords = rand_coords(rng, n)
    gf.forward(dev(coords))
    pick = np.sort(rng.choice(n, n // 2, replace=False)).astype(np.int32)
    gf.select(torch.from_numpy(pick).cuda(), n)
    dL = q16(rng.standard_normal((16, n // 2)) * np.array([.1, .1, .1, .1, 3, 3, 3, .1, .003, .003, .003, 0, 0, 0, 0, 0])[:, None])
    sub = np.ascontiguousarray(coords[pick])
    _, ctx = of.forward(p, sub)
    ref = of.backward(p, ctx, dL, ek_batch_size=n // 2)
    gf.backward(dev(sub), dev(np.ascontiguousarray(dL.T), torch.float16), ek_batch_size=n // 2, mode=GRAD_OVERWRITE)
    got = host(dg)
    assert np.isfinite(got).all()
    assert_grad_close(got[of.off_sdf:of.off_rgb], ref[of.off_sdf:of.off_rgb], what="SDF MLP gradients", rtol=2 * RTOL)
    assert_grad_close(got[of.off_rgb:of.off_grid], ref[of.off_rgb:of.off_grid], what="colour MLP gradients", rtol=2 * RTOL)


def test_direction_encoding_rows(oracle):
    """The degree-4 spherical-harmonics rows of the colour net's input on their own: with every other input column of
    the colour net's first layer zeroed, the output depends on the direction only through the 16 SH rows, and a net whose
    hidden layers pass values through unchanged hands them to the output."""
    from neus2_amd.tcnn_api import NerfNetwork
    from oracle.field import Field
    of, gf = Field(fp16=True), NerfNetwork()
    rng = np.random.default_rng(4)
    p = np.zeros(of.n_params, np.float32)
    # colour net: W0 [64][48] picks SH row k (input column 16 + k) into neurons 2k (+) and 2k + 1 (-), the second layer is
    # the identity, the output layer recombines relu(x) - relu(-x) = x for the first 16 SH values
    W0 = np.zeros((64, 48), np.float32)
    W1 = np.eye(64, dtype=np.float32)
    Wo = np.zeros((16, 64), np.float32)
    for k in range(16):
        W0[2 * k, 16 + k], W0[2 * k + 1, 16 + k] = 1.0, -1.0
        Wo[k, 2 * k], Wo[k, 2 * k + 1] = 1.0, -1.0
    p[of.off_rgb:of.off_grid] = np.concatenate([W0.ravel(), W1.ravel(), Wo.ravel()])
    p[of.off_sdf:of.off_rgb] = rng.standard_normal(of.off_rgb) * 0.1
    p[of.off_grid:of.off_var] = rng.uniform(-0.1, 0.1, of.grid.n_params)
    p = q16(p)
    dp = dev(p, torch.float16)
    gf.set_params(dp, torch.zeros_like(dp))
    n = 4096
    coords = rand_coords(rng, n)
    out = host(gf.forward(dev(coords))).T
    sh = oracle.sh4(np.ascontiguousarray(coords[:, 4:7].T))           # pinned by scipy.special.sph_harm_y
    # rows 0..2 and 11..15 of the output are the colour net's own rows (3..10 are overwritten by sdf, normal, ...)
    for r in (0, 1, 2, 11, 12, 13, 14, 15):
        assert_close(out[r], q16(sh[r]), rtol=RTOL, what=f"SH row {r}", scale=1.0)
