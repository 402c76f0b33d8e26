"""Occupancy-grid update on the GPU against the oracle (src/testbed_nerf.cu:3286-3391), through the C ABI."""
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, dev, host, q16
from neus2_amd import scene

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CELLS = 128 ** 3


@pytest.fixture(scope="module")
def trainer():
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield()
    T = 4096
    tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=1 << 18))
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(bits))
    # geometric-init SDF net (a sphere of radius ~0.1 minus the bias), small random grid
    tr.initialize_params(seed=5, sdf_mlp_weights=np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")))
    return tr


def oracle_density_fn(oracle, params16):
    from oracle.field import Field
    f = Field(fp16=True)
    return lambda xyz: f.density(params16, xyz)[0]


def compare_update(oracle, occ, ref, info, thresh_tol=1e-4):
    pos, idx = occ.last_samples()
    # sample positions and cells: bit-exact
    np.testing.assert_array_equal(host(idx).astype(np.uint32), info["indices"])
    np.testing.assert_array_equal(host(pos), info["positions"])
    # densities (fp16 field output) splatted by maximum: the stated tolerance of the field
    tmp = host(occ.density_grid_tmp)
    assert_close(tmp, info["tmp"], rtol=RTOL, what="splatted maxima", outlier_frac=1e-4)
    grid = host(occ.density_grid)
    assert_close(grid, ref.grid, rtol=RTOL, what="density grid", outlier_frac=1e-4)
    mean = float(host(occ.mean)[0])
    assert abs(mean - ref.mean) <= 2 * RTOL * ref.mean + 1e-12, (mean, ref.mean)
    # the bitfield of the GPU's own grid and mean is exact; against the oracle's it may differ in cells at the threshold
    want = oracle.grid_to_bitfield(grid, occ.n_cascades, mean)
    np.testing.assert_array_equal(host(occ.bitfield), want)
    thresh = min(0.1, ref.mean)
    undecided = np.abs(ref.grid - thresh) <= 4 * RTOL * thresh + thresh_tol * thresh
    got_bits = np.unpackbits(host(occ.bitfield)[:occ.n_cascades * CELLS // 8], bitorder="little").astype(bool)
    ref_bits = np.unpackbits(ref.bitfield[:occ.n_cascades * CELLS // 8], bitorder="little").astype(bool)
    assert not ((got_bits != ref_bits) & ~undecided).any()


def test_update_matches_oracle(oracle, trainer):
    from neus2_amd.training import OccupancyGrid
    params16 = host(trainer.params)
    dens = oracle_density_fn(oracle, params16)
    occ = OccupancyGrid(1, seed=1337, max_chunk=1 << 18)
    ref = oracle.OccupancyGrid(1, seed=1337)
    # first update: uniform samples only (a partial sweep keeps the oracle's field evaluation short)
    n0 = 300_001  # not a multiple of 8, and more than one chunk
    occ.update(trainer._field, n0, 0)
    info = ref.update(dens, 0.95, n0, 0)
    v = occ.view()
    assert v.n_samples == n0 and v.ema_step == 1 and (int(v.rng_state), int(v.rng_inc)) == (int(ref.rng.s[0]), int(ref.rng.s[1]))
    compare_update(oracle, occ, ref, info)
    assert 0 < ref.mean and ref.bitfield[:CELLS // 8].any()
    # second update: uniform + occupied-cell samples on top of the decayed first one
    occ.update(trainer._field, 100_000, 150_000)
    info = ref.update(dens, 0.95, 100_000, 150_000)
    assert occ.view().ema_step == 2
    compare_update(oracle, occ, ref, info)
    # occupied-cell samples really come from cells above the threshold of the first update
    assert (info["tmp"] > 0).sum() > 0


def test_two_cascades_and_mips(oracle, trainer):
    from neus2_amd.training import OccupancyGrid
    params16 = host(trainer.params)
    dens = oracle_density_fn(oracle, params16)
    occ = OccupancyGrid(2, seed=7, max_chunk=1 << 18)
    ref = oracle.OccupancyGrid(2, seed=7)
    # positions of the second cascade leave the unit cube; the field clamps them, the oracle must see the same points
    occ.update(trainer._field, 120_000, 0)
    info = ref.update(lambda xyz: dens(np.clip(xyz, 0.0, 1.0)), 0.95, 120_000, 0)
    pos, idx = occ.last_samples()
    np.testing.assert_array_equal(host(idx).astype(np.uint32), info["indices"])
    np.testing.assert_array_equal(host(pos), info["positions"])
    assert (info["indices"] >= CELLS).any() and (info["indices"] < CELLS).any()
    grid, mean = host(occ.density_grid), float(host(occ.mean)[0])
    np.testing.assert_array_equal(host(occ.bitfield), oracle.grid_to_bitfield(grid, 2, mean))
    inside = (info["positions"] >= 0).all(1) & (info["positions"] <= 1).all(1)
    cells_in = info["indices"][inside]
    assert_close(host(occ.density_grid_tmp)[cells_in], info["tmp"][cells_in], rtol=RTOL, what="maxima inside the unit cube", outlier_frac=1e-3)


def test_reset_and_restore_state(oracle, trainer):
    from neus2_amd import capi
    from neus2_amd.training import OccupancyGrid
    import ctypes as C
    occ = OccupancyGrid(1, seed=3, max_chunk=1 << 18)
    occ.update(trainer._field, 50_000, 0)
    v1 = occ.view()
    g1, b1 = host(occ.density_grid).copy(), host(occ.bitfield).copy()
    occ.reset()
    assert occ.view().ema_step == 0 and not host(occ.density_grid).any() and not host(occ.bitfield).any()
    # same generator state and step, same field -> same update
    capi.check(capi.lib().n2_occupancy_set_state(occ._h, C.c_uint32(0), C.c_uint64(oracle.Pcg32(3).s[0]), C.c_uint64(oracle.Pcg32(3).s[1])))
    occ.update(trainer._field, 50_000, 0)
    np.testing.assert_array_equal(host(occ.density_grid), g1)
    np.testing.assert_array_equal(host(occ.bitfield), b1)
    assert occ.view().rng_state == v1.rng_state
    # too many samples for the workspace: error, not a fault
    with pytest.raises(capi.N2Error):
        occ.update(trainer._field, CELLS, 1)


def test_training_with_live_occupancy_grid(trainer):
    """The trainer marches through a bitfield that training_prep rebuilds from its own field; sample generation
    running ahead must not see a half-written bitfield: results are the same with and without it."""
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import OccupancyGrid, Trainer, default_config
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    w48 = np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy"))
    results = []
    for prefetch in (True, False):
        T = 4096
        tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=1 << 18, prefetch_samples=prefetch))
        tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(scene.sphere_bitfield()))
        tr.initialize_params(seed=5, sdf_mlp_weights=w48)
        # bias so that the initial sphere (radius ~0.1 from the weights) has some density everywhere near it
        tr.attach_occupancy(OccupancyGrid(1, seed=11, max_chunk=1 << 18))
        log = []
        for step in range(6):
            plan = tr.training_prep()
            assert plan == (CELLS, 0)
            tr.step(n_rays=256, n_inference=1 << 18)
            c = tr.read_counters()
            log.append((c["rays"], c["samples"], c["compacted"], c["loss"]))
        assert all(np.isfinite(l[3]) for l in log) and log[-1][1] > 0
        results.append((log, host(tr.grads).copy(), host(tr.occupancy.bitfield).copy()))
    assert results[0][0] == results[1][0]
    np.testing.assert_array_equal(results[0][1], results[1][1])
    np.testing.assert_array_equal(results[0][2], results[1][2])


def test_a_step_after_an_update_with_larger_chunks_matches_the_oracle(oracle):
    """The occupancy update evaluates the field in chunks that are larger than the training step's inference batch; its
    gather uses the SDF net's input rows as scratch at the chunk's pitch, which falls on the rows the training layout
    keeps as zero padding.  A step behind such an update (same inference batch as the step before it) is checked stage by
    stage: the weight-gradient kernels read the padding rows against non-zero weight columns."""
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import OccupancyGrid, Trainer, default_config
    from oracle.field import Field
    from oracle.step import verify_step
    from test_oracle_sampler import oc_cams
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield()
    T, n_inf, chunk = 4096, 1 << 15, 1 << 18
    tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=chunk, background=(1.0, 1.0, 1.0)))
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(bits))
    tr.initialize_params(seed=9, sdf_mlp_weights=None)   # Xavier: the padding columns of W_0 are not zero
    occ = OccupancyGrid(1, seed=21, max_chunk=chunk)
    n_rays = 300
    tr.step(n_rays=n_rays, n_inference=n_inf, seed=1)
    assert n_inf < chunk < 16 * n_inf
    occ.update(tr._field, 2 * chunk, 0)
    params16 = host(tr.params).copy()
    tr.step(n_rays=n_rays, n_inference=n_inf, seed=2)
    c = tr.read_counters()
    gpu = {k: host(v) for k, v in tr.last_step(c["rays"], c["samples"], n_inf).items()}
    res = verify_step(Field(fp16=True), params16, oc_cams(oracle, cams), rgba, bits, n_rays, n_rays, 2, n_inf, T, c, gpu, host(tr.grads),
                      background=(1.0, 1.0, 1.0))
    assert res["compacted"] > T // 2, res
