"""GPU parity of NeuS compositing / loss / backward / compaction against the oracle."""
import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, dev, host, q16
from test_oracle_composite import make_rays

pytestmark = pytest.mark.gpu


def run_both(oracle, numsteps, out, coords, target, cap, **kw):
    from neus2_amd.tcnn_api import composite_loss
    out = q16(out)
    ref = oracle.composite_loss(numsteps, out, coords, target, cap, **kw)
    d_ns = dev(numsteps.astype(np.int32))
    got = composite_loss(d_ns, dev(out, torch.float16), dev(coords), dev(target), cap, **kw)
    got["numsteps"] = host(d_ns).view(np.uint32)
    return ref, got


def compare(ref, got, numsteps, max_count_mismatch=0):
    rn, gn = ref["numsteps"], got["numsteps"]
    # a transmittance within rounding of the 1e-4 cut-off may end a ray one sample apart
    same = rn[:, 0] == gn[:, 0]
    assert (~same).sum() <= max_count_mismatch, (~same).sum()
    if same.all():
        assert np.array_equal(rn, gn)
        assert int(host(got["counter"])[0]) == ref["counter"]
        np.testing.assert_array_equal(host(got["coords"]), ref["coords"])
    n_rays = rn.shape[0]
    assert_close(host(got["loss"])[same], ref["loss"][same], rtol=RTOL, what="per-ray loss")
    g, r = host(got["dloss"]), ref["dloss"]
    rows_g, rows_r = [], []
    for i in np.nonzero(same)[0]:
        k = int(rn[i, 0])
        rows_g.append(g[int(gn[i, 1]):int(gn[i, 1]) + k])
        rows_r.append(r[int(rn[i, 1]):int(rn[i, 1]) + k])
    G, R = np.concatenate(rows_g), np.concatenate(rows_r)
    for name, sl in (("rgb", slice(0, 3)), ("sdf", slice(3, 4)), ("eikonal", slice(4, 7)), ("variance", slice(7, 8)),
                     ("normal", slice(8, 11))):
        # fp16 output with gradients spanning decades: relative band plus half an fp16 subnormal step
        assert_close(G[:, sl], R[:, sl], rtol=2 * RTOL, what=f"dloss {name}", scale=float(np.abs(R[:, sl]).mean()) + 6e-8,
                     outlier_frac=1e-4)
    assert (G[:, 11:] == 0).all()


@pytest.mark.parametrize("sharp", [False, True])
def test_composite_matches_oracle(oracle, sharp):
    rng = np.random.default_rng(3 + sharp)
    numsteps, out, coords, target = make_rays(rng, 3000, lo=1, hi=150, sharp=sharp)
    ref, got = run_both(oracle, numsteps, out, coords, target, 1 << 18, background=(0.3, 0.6, 0.9), ek_loss_weight=0.01)
    compare(ref, got, numsteps, max_count_mismatch=1)
    if sharp:
        assert (ref["numsteps"][:, 0] < numsteps[:, 0]).mean() > 0.1  # early termination is exercised


def test_long_rays_cross_wave_chunks(oracle):
    rng = np.random.default_rng(5)
    numsteps, out, coords, target = make_rays(rng, 64, lo=60, hi=700)
    out[:, 3] = np.abs(out[:, 3]) * 0.2 + 0.006   # stay outside the surface: low alpha, rays run long
    ref, got = run_both(oracle, numsteps, out, coords, target, 1 << 16)
    assert (ref["numsteps"][:, 0] > 128).sum() > 10, ref["numsteps"][:, 0]  # several 64-sample chunks per ray
    compare(ref, got, numsteps, max_count_mismatch=1)


def test_many_rays_use_the_offset_scan(oracle):
    """Beyond 8192 rays the places of the rays in the compacted batch come from a scan kernel (several rounds of 4096 rays
    plus a ragged last one) instead of sums inside the backward kernel."""
    rng = np.random.default_rng(12)
    numsteps, out, coords, target = make_rays(rng, 21003, lo=0, hi=40, sharp=True)
    # the gradients scale with loss_scale / n_rays: 1024 keeps them where the other cases' 128 does at 3000 rays
    ref, got = run_both(oracle, numsteps, out, coords, target, 1 << 19, ek_loss_weight=0.01, loss_scale=1024.0)
    compare(ref, got, numsteps, max_count_mismatch=2)
    same = ref["numsteps"][:, 0] == got["numsteps"][:, 0]
    if not same.all():  # places follow the kept counts: compare them where no count before a ray differs
        upto = int(np.argmin(same))
        assert np.array_equal(ref["numsteps"][:upto], got["numsteps"][:upto])


def test_budget_clamp_and_ray_counter(oracle):
    from neus2_amd.tcnn_api import composite_loss
    rng = np.random.default_rng(6)
    numsteps, out, coords, target = make_rays(rng, 500, lo=2, hi=60)
    full = oracle.composite_loss(numsteps, q16(out), coords, target, 1 << 16)
    cap = int(full["counter"]) // 2 // 8 * 8
    ref, got = run_both(oracle, numsteps, out, coords, target, cap)
    compare(ref, got, numsteps)
    assert int(host(got["counter"])[0]) > cap
    # only the first 100 rays are live
    live = torch.tensor([100], dtype=torch.int32, device="cuda")
    d_ns = dev(numsteps.astype(np.int32))
    got2 = composite_loss(d_ns, dev(q16(out), torch.float16), dev(coords), dev(target), 1 << 16, ray_counter=live,
                          n_rays_norm=500)
    ref2 = oracle.composite_loss(numsteps[:100], q16(out), coords, target[:100], 1 << 16, n_rays_norm=500)
    assert int(host(got2["counter"])[0]) == ref2["counter"]
    ns2 = host(d_ns).view(np.uint32)
    assert np.array_equal(ns2[:100], ref2["numsteps"]) and (ns2[100:, 0] == 0).all()


def test_fill_rollover(oracle):
    from neus2_amd.tcnn_api import fill_rollover
    rng = np.random.default_rng(7)
    a = rng.standard_normal((4096, 7)).astype(np.float32)
    h = q16(rng.standard_normal((4096, 16)))
    for n_in in (0, 1, 1000, 4095, 4096, 5000):
        cnt = torch.tensor([n_in], dtype=torch.int32, device="cuda")
        ra = oracle.fill_rollover(a.copy(), n_in)
        ga = fill_rollover(dev(a), cnt)
        np.testing.assert_array_equal(host(ga), ra)
        rh = oracle.fill_rollover(h.copy(), n_in, rescale=True)
        gh = fill_rollover(dev(h, torch.float16), cnt)
        np.testing.assert_allclose(host(gh), rh, rtol=1e-3, atol=1e-6)


def test_empty(oracle):
    from neus2_amd.tcnn_api import composite_loss
    r = composite_loss(torch.zeros((0, 2), dtype=torch.int32, device="cuda"), torch.zeros((0, 16), dtype=torch.float16, device="cuda"),
                       torch.zeros((0, 7), device="cuda"), torch.zeros((0, 3), device="cuda"), 64)
    assert int(host(r["counter"])[0]) == 0


def test_cos_anneal_ratio_below_one(oracle):
    """cos_anneal_ratio < 1 blends the two cosine terms (nerf_network.h:1109-1118, src/testbed_nerf.cu:1583-1590)."""
    rng = np.random.default_rng(8)
    numsteps, out, coords, target = make_rays(rng, 1500, lo=1, hi=120, sharp=True)
    results = {}
    for ratio in (0.5, 0.0):
        ref, got = run_both(oracle, numsteps, out, coords, target, 1 << 18, cos_anneal_ratio=ratio, ek_loss_weight=0.01)
        compare(ref, got, numsteps, max_count_mismatch=1)
        results[ratio] = ref["dloss"]
    ref1 = oracle.composite_loss(numsteps, q16(out), coords, target, 1 << 18, cos_anneal_ratio=1.0, ek_loss_weight=0.01)
    assert not np.allclose(results[0.5][:, 3], ref1["dloss"][:, 3])  # the ratio matters for these rays
