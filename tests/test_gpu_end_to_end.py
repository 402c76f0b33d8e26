"""The whole loop the way the reference drives it: occupancy-grid updates on its cadence, training steps with
Ema(ExponentialDecay(Adam)), the ray budget feedback, then the SDF lattice and marching cubes.  A sphere of radius 0.3
seen by 32 cameras must come out of a network initialised as a sphere of radius ~0.1."""
import os

import numpy as np
import pytest
import torch

from neus2_amd import scene

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_training_recovers_the_sphere():
    from neus2_amd.mesh import density_on_grid, marching_cubes
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import ExponentialDecay, OccupancyGrid, Trainer, default_config
    cams = scene.cameras_on_sphere(32, 128)
    rgba = scene.render_sphere_images(cams)
    tr = Trainer(default_config(target_batch_size=1 << 16, max_rays_per_batch=1 << 14, max_samples=1 << 21, ema_decay=0.95))
    occ = OccupancyGrid(1, seed=1337, max_chunk=1 << 21)
    tr.set_scene(pack_cameras(cams), len(cams), torch.from_numpy(rgba).cuda(), occ.bitfield)
    tr.attach_occupancy(occ)
    tr.initialize_params(seed=1337, sdf_mlp_weights=np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")))
    tr.lr_schedule = ExponentialDecay()

    def mean_radius():
        v, t, _ = marching_cubes(density_on_grid(tr._field, (96, 96, 96)), 0.0)
        return float((v - 0.5).norm(dim=1).mean()), int(t.shape[0])

    r0, _ = mean_radius()
    assert 0.07 < r0 < 0.16  # the geometric initialisation
    losses, occupied = [], []
    for step in range(500):
        plan = tr.training_prep()
        assert (plan is not None) == (step % min(max(step // 16, 1), 16) == 0)
        tr.step()
        if step % 16 == 15 or step < 16:
            c, ok = tr.update_budget()
            assert ok and np.isfinite(c["loss"])
            losses.append(c["loss"] / max(c["rays"], 1))
            occupied.append(float(np.unpackbits(occ.bitfield[:128 ** 3 // 8].cpu().numpy()).mean()))
    r1, n_tris = mean_radius()
    assert 0.24 < r1 < 0.33 and n_tris > 10000, (r0, r1, n_tris)
    assert np.mean(losses[-4:]) < 0.5 * np.mean(losses[2:6]), losses
    # the occupancy grid first opens up (densities spread while the surface moves), then closes in on the shell
    assert max(occupied) > 1.5 * occupied[-1] and 0.05 < occupied[-1] < 0.4, occupied
    assert tr.optimizer_state().optimizer_steps == 500 and tr.ema_weights is not None
