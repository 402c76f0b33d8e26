"""Pins the oracle's NeuS compositing / loss / backward with closed-form cases and finite differences."""
import numpy as np
import pytest


def make_rays(rng, n_rays, lo=3, hi=40, sharp=False):
    counts = rng.integers(lo, hi, n_rays).astype(np.uint32)
    base = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint32)
    S = int(counts.sum())
    out = np.zeros((S, 16), np.float32)
    coords = np.zeros((S, 7), np.float32)
    coords[:, :3] = rng.random((S, 3))
    for i in range(n_rays):
        d = rng.standard_normal(3)
        d /= np.linalg.norm(d)
        sl = slice(int(base[i]), int(base[i] + counts[i]))
        m = int(counts[i])
        out[sl, 8:11] = (d + 1) / 2
        coords[sl, 4:7] = (d + 1) / 2
        # an sdf that crosses zero along the ray, normals roughly facing the camera
        t = np.linspace(0.02, -0.02, m) * (3 if sharp else 1) + rng.standard_normal(m) * 0.002
        out[sl, 3] = t
        nrm = -d[None, :] * (0.7 + 0.6 * rng.random((m, 1))) + rng.standard_normal((m, 3)) * 0.3
        out[sl, 4:7] = nrm
    out[:, 0:3] = rng.standard_normal((S, 3))
    out[:, 7] = 0.3 + (0.25 if sharp else 0.0)
    numsteps = np.stack([counts, base], 1).astype(np.uint32)
    target = rng.random((n_rays, 3)).astype(np.float32)
    return numsteps, out, coords, target


def huber_total(rgb_ray, target):
    d = rgb_ray.astype(np.float64) - target
    ad = np.abs(d)
    return np.where(ad > 0.1, ad - 0.05, 5.0 * d * d).sum() / 5.0


def test_all_alpha_zero_gives_background(oracle):
    """sdf far outside (prev and next cdf both ~1): alpha = 1e-5/(1+1e-5) ~ 0, T ~ 1, colour = background."""
    n = 5
    numsteps = np.array([[4, 4 * i] for i in range(n)], np.uint32)
    out = np.zeros((4 * n, 16), np.float32)
    out[:, 3] = 5.0
    out[:, 7] = 0.3
    out[:, 8:11] = [1.0, 0.5, 0.5]
    out[:, 4:7] = [-1, 0, 0]
    coords = np.zeros((4 * n, 7), np.float32)
    r = oracle.composite_loss(numsteps, out, coords, np.zeros((n, 3), np.float32), 64, background=(0.2, 0.4, 0.6))
    np.testing.assert_allclose(r["rgb_ray"], np.tile([0.2, 0.4, 0.6], (n, 1)), atol=1e-4)
    assert r["counter"] == 4 * n and (r["numsteps"][:, 0] == 4).all()
    np.testing.assert_array_equal(r["numsteps"][:, 1], 4 * np.arange(n))


def test_constant_alpha_geometric_transmittance(oracle):
    """Identical samples along a ray: T_i = (1-alpha)^i, rgb_ray = c*(1-(1-alpha)^n) + bg*(1-alpha)^n."""
    m = 12
    out = np.zeros((m, 16), np.float32)
    out[:, 3] = 0.0005
    out[:, 7] = 0.3
    out[:, 8:11] = [1.0, 0.5, 0.5]   # dir = +x
    out[:, 4:7] = [-1.0, 0, 0]       # cos = -1 -> iter_cos = -1
    out[:, 0:3] = [0.3, -0.2, 1.0]
    coords = np.zeros((m, 7), np.float32)
    numsteps = np.array([[m, 0]], np.uint32)
    r = oracle.composite_loss(numsteps, out, coords, np.zeros((1, 3), np.float32), 64, background=(1.0, 1.0, 1.0))
    s = np.exp(np.float64(np.float16(3.0)))
    dt = oracle.MIN_STEP
    sig = lambda x: 1 / (1 + np.exp(-x))
    prev, nxt = sig((0.0005 + dt / 2) * s), sig((0.0005 - dt / 2) * s)
    alpha = (prev - nxt + 1e-5) / (prev + 1e-5)
    c = sig(np.array([0.3, -0.2, 1.0]))
    want = c * (1 - (1 - alpha) ** m) + (1 - alpha) ** m
    np.testing.assert_allclose(r["rgb_ray"][0], want, rtol=2e-5)


def test_single_sample_ray_and_early_stop(oracle):
    # one opaque sample (alpha clamps to 1 when next cdf ~ 0): the ray stops, later samples are dropped
    m = 6
    out = np.zeros((m, 16), np.float32)
    out[:, 7] = 0.6
    out[:, 8:11] = [1.0, 0.5, 0.5]
    out[:, 4:7] = [-1.0, 0, 0]
    out[0, 3] = 0.02   # outside
    out[1, 3] = -0.02  # deep inside: prev ~ 0, alpha ~ clamp -> T falls below 1e-4 soon
    out[2:, 3] = -0.05
    coords = np.zeros((m, 7), np.float32)
    numsteps = np.array([[m, 0]], np.uint32)
    r = oracle.composite_loss(numsteps, out, coords, np.full((1, 3), 0.5, np.float32), 64, background=(9.0, 9.0, 9.0))
    kept = int(r["numsteps"][0, 0])
    assert 1 <= kept < m            # cut short
    assert r["rgb_ray"].max() < 1.5  # background not added when the ray was cut short
    assert (r["dloss"][kept:] == 0).all()


def test_gate_zeroes_geometry_gradients(oracle):
    """p_div_c outside (0,1) -> sdf / variance / normal gradients are exactly zero, colour gradient is not."""
    m = 3
    out = np.zeros((m, 16), np.float32)
    out[:, 7] = 0.3
    out[:, 8:11] = [1.0, 0.5, 0.5]
    out[:, 4:7] = [1.0, 0, 0]   # facing away: cos > 0 -> iter_cos = 0 -> p = 0 -> p_div_c = 1e-5/(c+1e-5) in (0,1)
    out[:, 3] = -1.0            # but deep inside: prev cdf ~ 0 -> p_div_c = 1e-5/(~0 + 1e-5) ~ 1 -> clamp gate
    out[:, 7] = 1.0
    coords = np.zeros((m, 7), np.float32)
    r = oracle.composite_loss(np.array([[m, 0]], np.uint32), out, coords, np.zeros((1, 3), np.float32), 8)
    g = r["dloss"][0]
    assert g[3] == 0 and g[7] == 0 and (g[8:11] == 0).all()
    assert np.abs(g[0:3]).max() > 0


def test_compaction_ranges_and_clamp(oracle):
    rng = np.random.default_rng(0)
    numsteps, out, coords, target = make_rays(rng, 50)
    full = oracle.composite_loss(numsteps, out, coords, target, 1 << 14)
    kept = full["numsteps"][:, 0]
    assert full["counter"] == kept.sum()
    np.testing.assert_array_equal(full["numsteps"][:, 1], np.concatenate([[0], np.cumsum(kept)[:-1]]))
    # compacted coords are the first kept[i] coords of each ray
    for i in (0, 7, 49):
        b, cb, k = int(numsteps[i, 1]), int(full["numsteps"][i, 1]), int(kept[i])
        np.testing.assert_array_equal(full["coords"][cb:cb + k], coords[b:b + k])
    # a smaller budget clamps the tail: max - min(max, base)
    cap = int(kept.sum()) // 2
    half = oracle.composite_loss(numsteps, out, coords, target, cap)
    assert half["counter"] == full["counter"]
    want = np.minimum(cap - np.minimum(cap, full["numsteps"][:, 1]), kept)
    np.testing.assert_array_equal(half["numsteps"][:, 0], want)
    np.testing.assert_array_equal(half["dloss"][:cap], full["dloss"][:cap])


@pytest.mark.parametrize("anneal", [1.0])
def test_backward_matches_finite_differences(oracle, anneal):
    rng = np.random.default_rng(1)
    n_rays = 6
    numsteps, out, coords, target = make_rays(rng, n_rays, lo=4, hi=12)
    kw = dict(max_compacted=256, loss_scale=128.0, ek_loss_weight=0.0, cos_anneal_ratio=anneal,
              background=(0.1, 0.2, 0.3), exact_inv_s=True)
    r = oracle.composite_loss(numsteps, out, coords, target, **kw)
    assert (r["numsteps"][:, 0] == numsteps[:, 0]).all(), "test wants rays that are not cut short"
    scale = 128.0 / n_rays
    h = 2e-3

    def L(o):
        return huber_total(oracle.composite_loss(numsteps, o, coords, target, **kw)["rgb_ray"], target)

    checked = 0
    for ray in range(n_rays):
        b, m = int(numsteps[ray, 1]), int(numsteps[ray, 0])
        cb = int(r["numsteps"][ray, 1])
        for j in (0, m // 2, m - 1):
            for col, gcol in ((0, 0), (2, 2), (3, 3), (7, 7), (4, 8), (5, 9), (6, 10)):
                op, om = out.copy(), out.copy()
                hh = h * (0.05 if col == 3 else 1.0)   # sdf lives on a 1e-2 scale
                op[b + j, col] += hh
                om[b + j, col] -= hh
                fd = (L(op) - L(om)) / (2 * hh)
                got = r["dloss"][cb + j, gcol] / scale
                assert abs(got - fd) <= 2e-2 * abs(fd) + 2e-4, (ray, j, col, got, fd)
                checked += 1
    assert checked > 100


def test_eikonal_rows(oracle):
    rng = np.random.default_rng(2)
    numsteps, out, coords, target = make_rays(rng, 4)
    r = oracle.composite_loss(numsteps, out, coords, target, 512, ek_loss_weight=0.01, loss_scale=128.0)
    for ray in range(4):
        b, cb, k = int(numsteps[ray, 1]), int(r["numsteps"][ray, 1]), int(r["numsteps"][ray, 0])
        n = out[b:b + k, 4:7].astype(np.float64)
        want = 0.01 * 2 * 128.0 * (1 - 1 / np.sqrt((n * n).sum(1) + 1e-6))[:, None] * n
        np.testing.assert_allclose(r["dloss"][cb:cb + k, 4:7], want, rtol=1e-4, atol=1e-6)
        assert (r["dloss"][cb:cb + k, 11:] == 0).all()


def test_fill_rollover(oracle):
    a = np.arange(40, dtype=np.float32).reshape(10, 4)
    b = a.copy()
    oracle.fill_rollover(b, 3)
    np.testing.assert_array_equal(b[:3], a[:3])
    for i in range(3, 10):
        np.testing.assert_array_equal(b[i], a[i % 3])
    c = a.copy()
    oracle.fill_rollover(c, 3, rescale=True)
    np.testing.assert_array_equal(c[:3], a[:3])
    np.testing.assert_allclose(c[5], a[2] * 3 / 10, rtol=1e-6)
    d = a.copy()
    oracle.fill_rollover(d, 0)
    np.testing.assert_array_equal(d, a)
    oracle.fill_rollover(d, 12)
    np.testing.assert_array_equal(d, a)
