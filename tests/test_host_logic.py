"""Host-side logic that needs no GPU: ray budget feedback, parameter initialisation, scene helpers."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_ray_budget_feedback():
    from neus2_amd.training import RayBudget
    b = RayBudget(1 << 18, 1 << 16, 16 << 18, rays_per_batch=4096)
    assert b.n_inference() == 16 << 18  # nothing measured yet: worst case (src/testbed_nerf.cu:3751-3753)
    assert b.update(4000, 500000, 131072)
    assert b.rays_per_batch == 8192 and b.n_inference() == 500096  # 2x rays, samples rounded up to 128
    assert b.update(8000, 10 ** 9, 262144)
    assert b.n_inference() == 16 << 18 and b.rays_per_batch == 8192
    assert not b.update(0, 0, 0)  # nothing generated: the reference stops training here
    b.update(8000, 1000, 10)
    assert b.rays_per_batch == 1 << 16  # clamped to the maximum


def test_initial_parameters_layout():
    from neus2_amd.training import initial_parameters
    W = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))
    offs = [0, 4096, 12288, 12288 + 12599920, 12288 + 12599920 + 4]
    p = initial_parameters(offs, 48, seed=1, sdf_mlp_weights=W)
    assert p.dtype == np.float32 and p.size == offs[4]
    np.testing.assert_array_equal(p[:4096], W)
    assert np.abs(p[4096:12288]).max() <= np.sqrt(6 / (16 + 64)) + 1e-6 and p[4096:12288].std() > 0.05  # widest: the 16x64 layer
    g = p[12288:offs[3]]
    assert np.abs(g).max() <= 1e-4 and abs(g.mean()) < 1e-6
    np.testing.assert_array_equal(p[offs[3]:], np.float32(0.3))
    from neus2_amd.capi import N2Error
    with pytest.raises(N2Error):
        initial_parameters(offs, 48, sdf_mlp_weights=W[:100])


def test_scene_cameras_look_at_the_centre():
    from neus2_amd import scene
    cams = scene.cameras_on_sphere(16, 32)
    for c in cams:
        X = c["xform"].reshape(3, 4)
        R, o = X[:, :3], X[:, 3]
        np.testing.assert_allclose(R.T @ R, np.eye(3), atol=1e-5)
        np.testing.assert_allclose(np.linalg.norm(o - 0.5), 2.0, rtol=1e-5)
        np.testing.assert_allclose(R[:, 2], (0.5 - o) / 2.0, atol=1e-5)
    img = scene.render_sphere_images(cams[:2])
    a = img[:, 3].reshape(2, 32, 32)
    assert a[:, 16, 16].all() and not a[:, 0, 0].any()  # sphere in the middle, empty corners


def test_trainer_config_struct_matches_header():
    """ctypes mirror vs the C declaration: same field count and 4-byte packing."""
    import ctypes
    from neus2_amd import capi
    assert ctypes.sizeof(capi.FieldConfig) == 32 and ctypes.sizeof(capi.AdamConfig) == 20
    assert ctypes.sizeof(capi.CompositeConfig) == 28 and ctypes.sizeof(capi.Camera) == 80
    assert ctypes.sizeof(capi.TrainerConfig) == 32 + 20 + 28 + 28
    assert ctypes.sizeof(capi.OccupancyBuffers) == 6 * 8 + 3 * 4 + 4 + 2 * 8 and ctypes.sizeof(capi.TrainerOptimizerBuffers) == 5 * 8 + 16
    L = capi.lib()
    cfg = capi.TrainerConfig()
    assert L.n2_trainer_workspace_bytes(ctypes.byref(cfg)) == 0  # all-zero config is rejected on the host
    from neus2_amd.training import default_config
    n = L.n2_trainer_workspace_bytes(ctypes.byref(default_config()))
    assert 3 * 2 ** 30 < n < 6 * 2 ** 30


def test_exponential_decay_schedule(oracle):
    """Host mirror of tcnn's ExponentialDecay (configs/nerf/base.json:8-12) against the oracle's step-by-step loop."""
    from neus2_amd.training import ExponentialDecay
    sched = ExponentialDecay(1e-3, decay_start=20, decay_interval=10, decay_base=0.33)
    for t in range(1, 75):
        lr = sched.after_step(t)
        want = oracle.exponential_decay_lr(1e-3, t, 20, 10, 0.33)
        assert abs(lr - want) <= 1e-7 * want, (t, lr, want)
    # closed form: the rate has been multiplied once at each of the steps 20, 30, ..., 70
    assert abs(sched.learning_rate - 1e-3 * 0.33 ** 6) < 1e-9
    # the published defaults leave the first 19999 steps alone
    d = ExponentialDecay()
    assert all(d.after_step(t) == d.learning_rate for t in (1, 100, 19999)) and abs(d.after_step(20000) - 3.3e-4) < 1e-9


def test_ema_oracle_closed_forms(oracle):
    rng = np.random.default_rng(0)
    decay = 0.95
    # constant weights: the bias-corrected average equals them at every step
    w = rng.standard_normal(1000).astype(np.float16).astype(np.float32)
    tmp = np.zeros_like(w)
    for t in range(1, 30):
        ema = oracle.ema_step(w, tmp, t, decay)
        np.testing.assert_allclose(tmp, w, rtol=2e-6, atol=1e-9)
        np.testing.assert_array_equal(ema, tmp.astype(np.float16).astype(np.float32))
    # changing weights: sum of (1 - d) d^(t-k) w_k over the steps, divided by 1 - d^t
    ws = rng.standard_normal((12, 64)).astype(np.float16).astype(np.float32)
    tmp = np.zeros(64, np.float32)
    for t in range(1, 13):
        oracle.ema_step(ws[t - 1], tmp, t, decay)
        k = np.arange(1, t + 1)
        want = ((1 - decay) * decay ** (t - k)[:, None] * ws[:t].astype(np.float64)).sum(0) / (1 - decay ** t)
        np.testing.assert_allclose(tmp, want, rtol=1e-5, atol=1e-6)


def test_level_mask_closed_forms(oracle):
    """tcnn's cut: level >= fraction * n_levels + 1e-3, so a level EQUAL to the limit stays on.  Fractions 0, 1/2, 1
    and > 1 on 16 and 14 levels."""
    m = oracle.level_mask(16, 1, 1.0)
    assert not m.any()
    assert oracle.level_mask(16, 1, 0.5)[:, 0].tolist() == [False] * 9 + [True] * 7
    assert oracle.level_mask(16, 1, 0.0)[:, 0].tolist() == [False] + [True] * 15     # level 0 survives: 0 < 0 + 1e-3
    assert not oracle.level_mask(14, 1, 1.7).any()
    assert oracle.level_mask(14, 1, 0.25)[:, 0].sum() == 10                           # limit 3.5: levels 0..3 stay
    per_point = oracle.level_mask(16, 3, np.array([0.0, 0.5, 2.0], np.float32))
    assert per_point.sum(0).tolist() == [15, 7, 0]
    assert oracle.level_mask(16, 2, 1.0, valid_levels=3).sum(0).tolist() == [13, 13]


def test_progressive_levels_schedule(oracle):
    """base.json: 14 levels, base 0.2, +0.02 per 100 steps -> 2 levels at the start, all 14 from step 4000 on."""
    f = lambda step: oracle.progressive_levels(14, 0.2, 0.02, 100, step)
    assert f(0) == 2 and f(99) == 2 and f(100) == 3 and f(4000) == 14 and f(10 ** 6) == 14
    steps = [f(s) for s in range(0, 5000, 100)]
    assert steps == sorted(steps)
    assert oracle.progressive_levels(16, 0.2, 0.02, 0, 5) == 16   # base_training_step 0: off


def test_progressive_levels_tables_of_the_shipped_configs(oracle):
    """The level schedule the adopted reading gives for the keys the reference ships (configs/nerf/base.json:31,36-38 and
    configs/nerf/dtu.json:30,35-37: 14 levels, base 0.2, +0.02 per 100 resp. 200 steps), as (first step, levels in use):
    closed form floor((0.2 + 0.02 (step // T)) 14 + 1e-3), i.e. level k + 1 joins at the first multiple of T with
    0.02 (step // T) >= (k + 1) / 14 - 0.2 up to fp32 rounding."""
    def table(period):
        out, prev = [], None
        for s in range(0, 40 * period + 1, period):
            lv = oracle.progressive_levels(14, 0.2, 0.02, period, s)
            assert lv == oracle.progressive_levels(14, 0.2, 0.02, period, s + period - 1)  # constant inside a period
            if lv != prev:
                out.append((s, lv))
                prev = lv
        return out
    base = [(0, 2), (100, 3), (500, 4), (800, 5), (1200, 6), (1500, 7), (1900, 8), (2300, 9), (2600, 10), (3000, 11), (3300, 12),
            (3700, 13), (4000, 14)]
    assert table(100) == base
    assert table(200) == [(2 * s, lv) for s, lv in base]
    # the same schedule by the closed form in exact arithmetic: levels = floor(2.8 + 0.28 k) for k = step // T < 40
    # (no k puts 2.8 + 0.28 k within the fp32 rounding and the 1e-3 guard of an integer except k = 40, which gives 14)
    import fractions
    for k in range(0, 41):
        exact = min(14, int(fractions.Fraction(14, 5) + fractions.Fraction(7, 25) * k))
        assert oracle.progressive_levels(14, 0.2, 0.02, 100, 100 * k) == exact, k
