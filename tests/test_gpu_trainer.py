"""The full training step on the GPU against the oracle pipeline (wiring test; every stage has its own parity test)."""
import os

import numpy as np
import pytest
import torch

from gpu_util import dev, host, q16
from neus2_amd import scene
from test_oracle_sampler import oc_cams

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def cos_sim(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float((a * b).sum() / max(np.linalg.norm(a) * np.linalg.norm(b), 1e-300))


@pytest.fixture(scope="module")
def setup(oracle):
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield()
    T = 4096
    cfg = default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=16 * T, background=(1.0, 1.0, 1.0))
    tr = Trainer(cfg)
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(bits))
    return tr, cams, rgba, bits, T


def test_one_step_matches_oracle_pipeline(oracle, setup):
    from oracle.field import Field
    tr, cams, rgba, bits, T = setup
    # Xavier everywhere: with the geometric-init weights the first layer's encoding columns are
    # zero, so the grid would receive an exactly zero gradient in the first step
    tr.initialize_params(seed=5, sdf_mlp_weights=None)
    master0 = host(tr.master).copy()
    params16 = host(tr.params)
    np.testing.assert_array_equal(params16, q16(master0))
    n_rays, seed = 300, 11
    n_inf = 16 * T
    tr.step(n_rays=n_rays, n_inference=n_inf, seed=seed)
    c = tr.read_counters()
    # ---- every stage against the oracle on the GPU's own input to that stage ----
    from oracle.step import verify_step
    gpu = {k: host(v) for k, v in tr.last_step(c["rays"], c["samples"], n_inf).items()}
    got_grad = host(tr.grads)
    of = Field(fp16=True)
    res = verify_step(of, params16, oc_cams(oracle, cams), rgba, bits, n_rays, 0, seed, n_inf, T, c, gpu, got_grad, background=(1.0, 1.0, 1.0))
    assert res["compacted"] > T // 2, res
    # ---- Adam on the GPU's own gradients ----
    w, m1, m2 = master0.copy(), np.zeros_like(master0), np.zeros_like(master0)
    steps = np.zeros(master0.size, np.uint32)
    oracle.adam_step(w, got_grad, m1, m2, steps, n_matrix_params=of.n_matrix_params)
    np.testing.assert_allclose(host(tr.master), w, rtol=1e-5, atol=1e-7)
    np.testing.assert_array_equal(host(tr.params), q16(host(tr.master)))


def test_a_small_batch_rolls_over_several_times(oracle, setup):
    """Few rays: the kept samples fill less than half of the batch, so every kept sample is copied (and its output
    gradient rescaled) more than once; every stage of the step against the oracle, as above."""
    from oracle.field import Field
    from oracle.step import verify_step
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    _, cams, rgba, bits, T = setup
    tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=16 * T, background=(1.0, 1.0, 1.0)))
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(bits))
    tr.initialize_params(seed=7, sdf_mlp_weights=None)
    params16 = host(tr.params)
    n_rays, seed, n_inf = 40, 3, 16 * T
    tr.step(n_rays=n_rays, n_inference=n_inf, seed=seed)
    c = tr.read_counters()
    assert 0 < c["compacted"] < T // 2, c
    gpu = {k: host(v) for k, v in tr.last_step(c["rays"], c["samples"], n_inf).items()}
    res = verify_step(Field(fp16=True), params16, oc_cams(oracle, cams), rgba, bits, n_rays, 0, seed, n_inf, T, c, gpu,
                      host(tr.grads), background=(1.0, 1.0, 1.0))
    assert res["compacted"] == c["compacted"]


def test_training_reduces_the_loss(setup):
    """End-to-end: a sign error anywhere in the first- or second-order backward would stop this from converging."""
    tr, cams, rgba, bits, T = setup
    W = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))
    tr.cfg.adam.learning_rate = 1e-2  # the reference's DTU recipe (README.md:90, configs/nerf/dtu.json:15)
    from neus2_amd.training import Trainer
    tr2 = Trainer(tr.cfg)
    tr2.set_scene(*[tr._scene[0], len(cams), tr._scene[1], tr._scene[2]])
    tr2.initialize_params(seed=6, sdf_mlp_weights=W)
    tr2.budget.rays_per_batch = 256
    losses = []
    for it in range(1600):
        tr2.step()
        if it % 20 == 19:
            c, ok = tr2.update_budget()
            assert ok, c
            losses.append(c["loss"])
    losses = np.array(losses)
    assert np.isfinite(losses).all()
    early, late = losses[5:15].mean(), losses[-10:].mean()
    assert late < 0.75 * early, (early, late)
    # the ray budget steers the compacted batch towards the target
    assert 0.5 * T < c["compacted"] < 2.0 * T, c
    assert np.isfinite(host(tr2.master)).all()


def test_trainer_errors(setup):
    from neus2_amd.capi import N2Error
    from neus2_amd.training import Trainer, default_config
    tr, *_ = setup
    with pytest.raises(N2Error, match="n_rays"):
        tr.step(n_rays=10 ** 6)
    with pytest.raises(N2Error, match="n_inference"):
        tr.step(n_rays=8, n_inference=12)
    with pytest.raises(N2Error):
        Trainer(default_config(target_batch_size=100))
    t2 = Trainer(default_config(target_batch_size=256, max_rays_per_batch=64, max_samples=1024))
    with pytest.raises(N2Error, match="set_scene"):
        t2.step(n_rays=8, n_inference=1024)


def test_samples_generated_ahead_give_the_same_steps():
    """Generating the next step's samples on the trainer's own stream changes nothing but timing, also when a
    step is called with other arguments than the ones the generation ran ahead with."""
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    cams = scene.cameras_on_sphere(6, 64)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield()
    T = 2048
    d_cams, d_rgba, d_bits = pack_cameras(cams), dev(rgba), dev(bits)
    # (n_rays, seed): consecutive seeds hit the generation that ran ahead, the others miss it
    plan = [(200, 0), (200, 1), (200, 2), (260, 3), (260, 4), (260, 9), (260, 10), (120, 11)]
    runs = []
    for ahead in (False, True):
        tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=512, max_samples=16 * T, prefetch_samples=ahead))
        tr.set_scene(d_cams, len(cams), d_rgba, d_bits)
        tr.initialize_params(seed=5, sdf_mlp_weights=None)
        log = []
        for n_rays, seed in plan:
            tr.step(n_rays=n_rays, n_inference=16 * T, seed=seed)
            log.append(tr.read_counters())
        runs.append((log, host(tr.master).copy()))
        del tr
    (log_a, m_a), (log_b, m_b) = runs
    # bit for bit: every sum of a step is formed in an order that does not depend on how the GPU schedules the work
    assert log_a == log_b and all(a["rays"] > 0 for a in log_a)
    np.testing.assert_array_equal(m_a, m_b)


def test_a_step_is_bit_reproducible_at_the_benchmark_batch():
    """Two trainers run the same steps at the 2^18 batch (the encoding's coarsest levels then split their buckets over
    several workgroups, whose partial sums meet in a fixed order): gradients, counters, loss and parameters agree bit for
    bit after every step, with the sample generation running ahead in one of them."""
    import bench
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    T = 1 << 18
    cams, rgba, bits = bench.build_scene()
    d_cams, d_rgba, d_bits = pack_cameras(cams), dev(rgba), dev(bits)
    n_inf = 280000 // 128 * 128
    runs = []
    for ahead in (True, False):
        tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=1 << 16, max_samples=16 * T, prefetch_samples=ahead))
        tr.set_scene(d_cams, len(cams), d_rgba, d_bits)
        tr.initialize_params(seed=1337, sdf_mlp_weights=None)
        seen = []
        for step in range(3):
            tr.step(n_rays=5000, n_inference=n_inf, seed=40 + step)
            seen.append((tr.read_counters(), tr.grads.clone()))
        runs.append((seen, tr.master.clone()))
        del tr
    (seen_a, m_a), (seen_b, m_b) = runs
    for (ca, ga), (cb, gb) in zip(seen_a, seen_b):
        assert ca == cb and ca["compacted"] > T // 2
        assert torch.equal(ga, gb)
        assert ga.float().abs().sum() > 0
    assert torch.equal(m_a, m_b)


def test_progressive_level_mask_follows_the_step_count(oracle):
    """With the progressive keys set, every step tells the encoding how many steps were taken before it: the levels
    not yet switched on receive exactly zero gradient, the others do receive some."""
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    cams = scene.cameras_on_sphere(8, 96)
    T = 4096
    tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=16 * T, background=(1.0, 1.0, 1.0)))
    tr.set_scene(pack_cameras(cams), len(cams), dev(scene.render_sphere_images(cams)), dev(scene.sphere_bitfield()))
    tr.initialize_params(seed=5, sdf_mlp_weights=None)
    enc = tr.encoding()
    enc.set_progressive(0.25, 0.125, 2)          # 4 levels, two more every 2 steps
    _, _, entries, offset = enc.level_table()
    g0 = tr.offsets[2]
    for step in range(5):
        tr.step(n_rays=300, n_inference=16 * T, seed=step)
        want = oracle.progressive_levels(16, 0.25, 0.125, 2, step)
        assert enc.active_levels() == want == 4 + 2 * (step // 2)
        g = host(tr.grads)[g0:g0 + 2 * int(offset[-1])]
        assert np.abs(g[:2 * int(offset[want])]).max() > 0
        assert (g[2 * int(offset[want]):] == 0).all()
    enc.set_progressive(1.0, 0.0, 0)
    assert enc.active_levels() == 16


def test_selected_activations_give_the_same_steps_as_a_second_forward():
    """The step can evaluate the field again on the compacted batch (as the reference does) or select the activations
    its first evaluation saved: parameters, optimiser state and counters agree bit for bit after several steps, also
    when the batch is padded by roll-over and when rays are cut by the batch limit."""
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    cams = scene.cameras_on_sphere(6, 64)
    d_cams, d_rgba, d_bits = pack_cameras(cams), dev(scene.render_sphere_images(cams)), dev(scene.sphere_bitfield())
    T = 4096
    plan = [(60, 0), (60, 1), (200, 2), (200, 3), (33, 4)]  # few rays: roll-over padding; many: the batch limit cuts rays
    runs = []
    for recompute in (True, False):
        tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=512, max_samples=16 * T, recompute_training_forward=recompute))
        tr.set_scene(d_cams, len(cams), d_rgba, d_bits)
        tr.initialize_params(seed=5, sdf_mlp_weights=None)
        seen = []
        for n_rays, seed in plan:
            tr.step(n_rays=n_rays, n_inference=16 * T, seed=seed)
            seen.append((tr.read_counters(), tr.grads.clone()))
        runs.append((seen, tr.master.clone()))
    (a, ma), (b, mb) = runs
    kinds = set()
    for (ca, ga), (cb, gb) in zip(a, b):
        assert ca == cb
        assert torch.equal(ga, gb)
        kinds.add("padded" if ca["compacted"] < T else "cut" if ca["compacted"] > T else "exact")
    assert {"padded", "cut"} <= kinds
    assert torch.equal(ma, mb)


def test_step_without_samples_changes_nothing(setup):
    """No ray finds an occupied cell: the step generates no sample and must not apply the previous step's gradients
    again (the reference stops training on an empty batch, src/testbed_nerf.cu:3536-3542)."""
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    _, cams, rgba, bits, T = setup
    tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=16 * T))
    empty = torch.zeros(bits.size, dtype=torch.uint8, device="cuda")
    full = dev(bits)
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), full)
    tr.initialize_params(seed=5, sdf_mlp_weights=None)
    tr.step(n_rays=300, n_inference=16 * T, seed=3)          # an ordinary step first: gradients and moments exist
    assert tr.read_counters()["compacted"] > 0
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), empty)
    master, params = tr.master.clone(), tr.params.clone()
    st = tr.optimizer_state()
    m1 = tr._view(st.first_moments, tr.n_params, torch.float32).clone()
    tr.step(n_rays=300, n_inference=16 * T, seed=4)
    c = tr.read_counters()
    assert c["samples"] == 0 and c["compacted"] == 0
    assert torch.equal(tr.master, master) and torch.equal(tr.params, params)
    assert torch.equal(tr._view(st.first_moments, tr.n_params, torch.float32), m1)


def test_depth_chunks_give_the_same_steps(oracle):
    """On a trained field most rays pass the compositor's transmittance cut long before their last marched sample.  The
    step can evaluate the field in rounds of a few samples per ray, dropping the rays that are past the cut between
    rounds: parameters, gradients and counters are bit-identical to the plain step's (which evaluates every marched sample),
    a fraction of the samples is evaluated, and a chunked step passes the stage-by-stage check against the oracle."""
    from oracle.field import Field
    from oracle.step import verify_step
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import OccupancyGrid, Trainer, default_config
    cams = scene.cameras_on_sphere(32, 128)
    rgba = scene.render_sphere_images(cams)
    d_cams, d_rgba = pack_cameras(cams), dev(rgba)
    T = 1 << 14
    W = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))

    def make(bitfield=None):
        tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=1 << 13, max_samples=1 << 19, background=(1.0, 1.0, 1.0)))
        tr.auto_depth_chunks = False
        tr.set_scene(d_cams, len(cams), d_rgba, bitfield if bitfield is not None else dev(scene.sphere_bitfield()))
        return tr
    # a trained state: the loop the reference drives (occupancy updates on their cadence, ray budget feedback)
    a = make()
    a.attach_occupancy(OccupancyGrid(1, seed=1337, max_chunk=1 << 19))
    a.initialize_params(seed=1337, sdf_mlp_weights=W)
    for it in range(500):
        a.training_prep()
        a.step()
        if it % 16 == 15 or it < 16:
            c, ok = a.update_budget()
            assert ok, c
    master = host(a.master).copy()
    bits = a.occupancy.bitfield.clone()
    n_rays, n_inf = a.budget.rays_per_batch, a.budget.n_inference()
    assert c["samples"] > 1.3 * c["compacted"], c   # rays do end early in this state (after a hundred to two hundred samples)
    runs = []
    # the last run changes the setting between steps, while the next step's samples are already being generated (a plain
    # step's generation also writes the positions as rows, one in rounds does not: a step takes what its samples come with)
    for chunks in ((0, 0), (96, 3), (16, 8), (1, 2), "switched"):
        tr = make(bits)
        tr.set_parameters(master)
        if chunks != "switched":
            tr.set_depth_chunks(*chunks)
        seen = []
        for step in range(4):
            if chunks == "switched":
                tr.set_depth_chunks(*[(16, 8), (0, 0), (96, 3), (0, 0)][step])
            params16 = host(tr.params).copy()
            tr.step(n_rays=n_rays, n_inference=n_inf, seed=100 + step)
            cs = tr.read_counters()
            view = tr.last_step(cs["rays"], cs["samples"], n_inf)
            seen.append((cs, tr.grads.clone()))
            if chunks != "switched" and chunks[1]:
                done = int(view["evaluated_counts"].sum().item())
                assert min(cs["compacted"], T) <= done <= cs["samples"]
                if chunks == (96, 3):
                    assert done < 0.95 * cs["samples"], (done, cs)
                if step == 1 and chunks == (96, 3):
                    gpu = {k: host(v) for k, v in view.items()}
                    res = verify_step(Field(fp16=True), params16, oc_cams(oracle, cams), rgba, host(bits), n_rays, n_rays, 101, n_inf, T, cs, gpu,
                                      host(tr.grads), background=(1.0, 1.0, 1.0), evaluated=gpu["evaluated_samples"])
                    assert res["compacted"] == cs["compacted"]
        runs.append((seen, tr.master.clone()))
        del tr
    (ref_seen, ref_master) = runs[0]
    for seen, m in runs[1:]:
        for (ca, ga), (cb, gb) in zip(ref_seen, seen):
            assert ca == cb and ca["compacted"] > 0
            assert torch.equal(ga, gb)
        assert torch.equal(ref_master, m)
