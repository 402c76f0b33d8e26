"""Snapshot save / load through the C ABI: the file decodes with an independent MessagePack implementation to the
device contents, and a trainer restored from it continues exactly like the one that wrote it."""
import os

import numpy as np
import pytest
import torch

from gpu_util import dev, host
from neus2_amd import scene
from test_snapshot_format import CONFIG, reference_style_file

msgpack = pytest.importorskip("msgpack")
pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CELLS = 128 ** 3


def make_trainer(ema=0.95):
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import OccupancyGrid, Trainer, default_config
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    tr = Trainer(default_config(target_batch_size=4096, max_rays_per_batch=2048, max_samples=1 << 17, ema_decay=ema))
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(scene.sphere_bitfield()))
    tr.initialize_params(seed=5, sdf_mlp_weights=np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")))
    tr.attach_occupancy(OccupancyGrid(1, seed=11, max_chunk=1 << 17))
    return tr


def run_steps(tr, n):
    log = []
    for _ in range(n):
        tr.training_prep()
        tr.step(n_rays=256, n_inference=1 << 17)
        c, _ = tr.update_budget()
        log.append((c["rays"], c["samples"], c["compacted"], c["loss"]))
    return log


def test_file_contents_and_exact_resume(tmp_path):
    from neus2_amd.snapshot import load_snapshot, save_snapshot, snapshot_info
    tr = make_trainer()
    run_steps(tr, 3)
    path = tmp_path / "step3.msgpack"
    save_snapshot(path, tr, tr.occupancy, config=CONFIG, include_optimizer_state=True, loss=0.25)
    # ---- the file, read by another implementation ----
    doc = msgpack.unpackb(path.read_bytes(), raw=False, strict_map_key=False)
    assert {k: doc[k] for k in CONFIG} == CONFIG
    snap = doc["snapshot"]
    assert snap["n_params"] == tr.n_params and snap["params_type"] == "__half" and snap["density_grid_size"] == 128
    np.testing.assert_array_equal(np.frombuffer(snap["params_binary"], np.float16), tr.params.cpu().numpy())
    np.testing.assert_array_equal(np.frombuffer(snap["density_grid_binary"], np.float16), tr.occupancy.density_grid.cpu().numpy().astype(np.float16))
    assert snap["training_step"] == 3 and snap["loss"] == 0.25 and snap["nerf"]["aabb_scale"] == 1
    assert snap["nerf"]["rgb"]["rays_per_batch"] == tr.budget.rays_per_batch
    assert snap["nerf"]["rgb"]["measured_batch_size_before_compaction"] == tr.budget.measured_before_compaction
    adam = snap["optimizer"]["nested"]["nested"]
    st = tr.optimizer_state()
    assert adam["current_step"] == 3 and abs(adam["base_learning_rate"] - 1e-3) < 1e-9
    np.testing.assert_array_equal(np.frombuffer(adam["first_moments_binary"], np.float32), tr._view(st.first_moments, tr.n_params, torch.float32).cpu().numpy())
    # the trainer keeps 16-bit counters for the default betas; the file holds the reference's 32-bit form
    assert st.param_steps_bits == 16
    np.testing.assert_array_equal(np.frombuffer(adam["param_steps_binary"], np.uint32),
                                  tr._view(st.param_steps, tr.n_params, torch.int16).cpu().numpy().view(np.uint16).astype(np.uint32))
    np.testing.assert_array_equal(np.frombuffer(snap["optimizer"]["ema_weights_binary"], np.float32), tr.ema_weights.cpu().numpy())
    info = snapshot_info(path)
    assert info.n_params == tr.n_params and info.training_step == 3 and info.has_optimizer_state and info.has_ema_weights
    assert info.density_grid_cells == CELLS and info.optimizer_steps == 3
    # ---- resume: a fresh trainer restored from the file continues bit for bit like the original ----
    tr2 = make_trainer()
    load_snapshot(path, tr2, tr2.occupancy)
    np.testing.assert_array_equal(host(tr2.params), host(tr.params))
    np.testing.assert_array_equal(host(tr2.master), host(tr.params))  # fp16 file: the master restarts from the rounded weights
    np.testing.assert_array_equal(host(tr2.occupancy.density_grid), tr.occupancy.density_grid.cpu().numpy().astype(np.float16).astype(np.float32))
    np.testing.assert_array_equal(host(tr2.inference_params), host(tr.inference_params))
    assert tr2.step_index == 3 and tr2.optimizer_state().optimizer_steps == 3
    # the original continues from the same rounded state so that both see identical inputs
    load_snapshot(path, tr, tr.occupancy)
    v, v2 = tr.occupancy.view(), tr2.occupancy.view()
    from neus2_amd import capi
    import ctypes as C
    capi.check(capi.lib().n2_occupancy_set_state(tr2.occupancy._h, C.c_uint32(v.ema_step), C.c_uint64(v.rng_state), C.c_uint64(v.rng_inc)))
    np.testing.assert_array_equal(host(tr2.occupancy.bitfield), host(tr.occupancy.bitfield))
    assert run_steps(tr, 2) == run_steps(tr2, 2)
    np.testing.assert_array_equal(host(tr2.master), host(tr.master))
    np.testing.assert_array_equal(host(tr2.ema_weights), host(tr.ema_weights))


def test_loads_files_of_another_writer_and_checks_shapes(tmp_path):
    """A file in the reference's layout written by the msgpack package (fp32 parameters, as newer tiny-cuda-nn stores them)."""
    from neus2_amd import capi
    from neus2_amd.snapshot import load_snapshot
    tr = make_trainer(ema=0.0)
    n = tr.n_params
    rng = np.random.default_rng(1)
    w = (rng.standard_normal(n) * 0.01).astype(np.float32)
    grid = rng.random(CELLS).astype(np.float16)
    doc = reference_style_file()
    doc["snapshot"].update(n_params=n, params_type="float", params_binary=w.tobytes(), density_grid_binary=grid.tobytes())
    p = tmp_path / "other.msgpack"
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    info = load_snapshot(p, tr, tr.occupancy)
    assert info.params_are_fp32 == 1 and not info.has_optimizer_state
    np.testing.assert_array_equal(host(tr.master), w)
    np.testing.assert_array_equal(host(tr.params), w.astype(np.float16).astype(np.float32))
    np.testing.assert_array_equal(host(tr.occupancy.density_grid), grid.astype(np.float32))
    # mean and bitfield were rebuilt from the loaded grid (update_density_grid_mean_and_bitfield)
    mean = float(host(tr.occupancy.mean)[0])
    assert abs(mean - grid.astype(np.float64).mean()) < 1e-4
    bits = np.unpackbits(host(tr.occupancy.bitfield)[:CELLS // 8], bitorder="little").astype(bool)
    np.testing.assert_array_equal(bits, grid.astype(np.float32) > np.float32(min(0.1, mean)))
    assert tr.step_index == 1234 and tr.budget.rays_per_batch == 4096
    # wrong parameter count / cascade count: the reference's errors, not a fault
    doc["snapshot"].update(n_params=24, params_binary=w[:24].tobytes())
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    with pytest.raises(capi.N2Error, match="parameters"):
        load_snapshot(p, tr, tr.occupancy)
    doc["snapshot"].update(n_params=n, params_binary=w.tobytes(), density_grid_binary=grid[:CELLS // 2].tobytes())
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    with pytest.raises(capi.N2Error, match="cascades"):
        load_snapshot(p, tr, tr.occupancy)


def test_step_counters_of_a_long_run_load_into_the_narrow_counters(tmp_path):
    """The trainer keeps 16-bit per-parameter step counters for the default betas (past 4096 steps the bias correction is
    exactly 1, so the count no longer matters); a file of another writer holds 32-bit counts, some beyond 65535: they load
    as min(count, 65535), a step goes on from there, and the file written afterwards holds the 32-bit form again."""
    from neus2_amd.snapshot import load_snapshot, save_snapshot
    tr = make_trainer(ema=0.0)
    n = tr.n_params
    rng = np.random.default_rng(3)
    steps = rng.integers(0, 200000, n).astype(np.uint32)
    steps[:4] = (0, 65534, 65535, 70000)
    doc = reference_style_file(with_optimizer=True)
    adam = doc["snapshot"]["optimizer"]["nested"]["nested"]
    adam.update(first_moments_binary=np.zeros(n, np.float32).tobytes(), second_moments_binary=np.ones(n, np.float32).tobytes(),
                param_steps_binary=steps.tobytes())
    del doc["snapshot"]["optimizer"]["ema_weights_binary"]
    doc["snapshot"].update(n_params=n, params_type="__half", params_binary=host(tr.params).astype(np.float16).tobytes(),
                           density_grid_binary=np.full(CELLS, 1.0, np.float16).tobytes())
    p = tmp_path / "long_run.msgpack"
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    info = load_snapshot(p, tr, tr.occupancy)
    assert info.has_optimizer_state
    st = tr.optimizer_state()
    assert st.param_steps_bits == 16
    got = tr._view(st.param_steps, n, torch.int16).cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(got, np.minimum(steps, 65535).astype(np.uint16))
    tr.step(n_rays=256, n_inference=1 << 17)
    after = tr._view(st.param_steps, n, torch.int16).cpu().numpy().view(np.uint16).astype(np.uint32)
    assert ((after == np.minimum(steps, 65535)) | (after == np.minimum(steps + 1, 65535))).all()
    assert (after != np.minimum(steps, 65535)).any()
    assert np.isfinite(host(tr.master)).all()
    out = tmp_path / "after.msgpack"
    save_snapshot(out, tr, tr.occupancy, config=CONFIG, include_optimizer_state=True)
    saved = msgpack.unpackb(out.read_bytes(), raw=False, strict_map_key=False)["snapshot"]["optimizer"]["nested"]  # no Ema level
    np.testing.assert_array_equal(np.frombuffer(saved["param_steps_binary"], np.uint32), after)


def test_params_only_resume_restores_level_mask_and_restarts_ema(tmp_path):
    """A snapshot without optimizer state still carries the training step: the progressive level mask of a trainer
    restored from it is that step's (not the first step's), the occupancy update that precedes the next step already sees
    it, and the Ema average starts again from the loaded parameters."""
    from neus2_amd.snapshot import load_snapshot, save_snapshot
    tr = make_trainer(ema=0.9)
    tr.encoding().set_progressive(0.25, 0.125, 2)  # 4 levels, two more every 2 steps
    run_steps(tr, 5)
    path = tmp_path / "params_only.msgpack"
    save_snapshot(path, tr, tr.occupancy, config=CONFIG, include_optimizer_state=False)
    tr2 = make_trainer(ema=0.9)
    enc = tr2.encoding()
    enc.set_progressive(0.25, 0.125, 2)
    assert enc.active_levels() == 4                      # step 0
    info = load_snapshot(path, tr2, tr2.occupancy)
    assert info.training_step == 5 and not info.has_optimizer_state
    assert enc.active_levels() == 4 + 2 * (5 // 2)       # restored from the file's training step
    torch.testing.assert_close(tr2.params, tr.params, rtol=0, atol=0)
    # the inference parameters are the loaded ones, not the fresh trainer's initial average
    torch.testing.assert_close(tr2.inference_params, tr2.params, rtol=0, atol=0)
    # the first Ema step after the restart reproduces the working weights (bias-corrected average of one sample)
    tr2.training_prep()
    assert enc.active_levels() == 8                      # the occupancy update of step 5 ran under step 5's mask
    tr2.step(n_rays=256, n_inference=1 << 17)
    torch.testing.assert_close(tr2.ema_weights, tr2.params.float(), rtol=1e-6, atol=1e-9)
    assert enc.active_levels() == 8
    tr2.training_prep()
    assert enc.active_levels() == 4 + 2 * (6 // 2)       # step 6


def test_ema_round_trip_with_optimizer_state(tmp_path):
    """With the Ema wrapper on and the optimizer state in the file, working and averaged weights both come back and the
    moving average continues from the saved step count."""
    from neus2_amd.snapshot import load_snapshot, save_snapshot
    tr = make_trainer(ema=0.9)
    run_steps(tr, 3)
    path = tmp_path / "ema.msgpack"
    save_snapshot(path, tr, tr.occupancy, config=CONFIG, include_optimizer_state=True)
    tr2 = make_trainer(ema=0.9)
    info = load_snapshot(path, tr2, tr2.occupancy)
    assert info.has_optimizer_state and info.has_ema_weights
    torch.testing.assert_close(tr2.params, tr.params, rtol=0, atol=0)
    torch.testing.assert_close(tr2.ema_weights, tr.ema_weights, rtol=0, atol=0)
    torch.testing.assert_close(tr2.inference_params, tr.inference_params, rtol=0, atol=0)
    assert not torch.equal(tr.inference_params, tr.params)   # the average is not the working copy
    # the average continues with the saved step count: one more step on identical inputs moves both trainers' averages alike
    load_snapshot(path, tr, tr.occupancy)
    for t in (tr, tr2):
        t.step(n_rays=256, n_inference=1 << 17, seed=99)
    torch.testing.assert_close(tr2.ema_weights, tr.ema_weights, rtol=0, atol=0)
    torch.testing.assert_close(tr2.inference_params, tr.inference_params, rtol=0, atol=0)
