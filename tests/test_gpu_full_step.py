"""The training step at the benchmark's shape (BASELINE configuration 4: 64 cameras at 512 x 512, 2^18-sample batch,
capacity 16 x 2^18, sample generation running ahead), checked stage by stage against the oracle
(Testbed::train_nerf_step, src/testbed_nerf.cu:3717-3987)."""
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, dev, host
from test_oracle_sampler import oc_cams

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("loss_scale", [8192.0, 128.0])
def test_two_steps_at_the_benchmark_shape(oracle, loss_scale):
    """loss_scale 128 is the reference's (testbed.h:237).  With about 5000 rays per step it puts the colour gradients of a
    sample near 2.5e-6, i.e. into the SUBNORMAL range of fp16 (steps of 6e-8), which is the precision of the matrices the
    fully fused networks pass the hidden layers' gradients through.  The trainer therefore gives the colour net's backward
    an exponent (n2_colour_gradient_exponent) under which those matrices hold 2^k times the values: every figure is held to
    the stated tolerance at both loss scales."""
    import bench
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    from oracle.field import Field
    from oracle.step import verify_step
    T = 1 << 18
    cams, rgba, bits = bench.build_scene()
    cfg = default_config(target_batch_size=T, max_rays_per_batch=1 << 16, max_samples=16 * T, prefetch_samples=True)
    cfg.loss_scale = loss_scale
    tr = Trainer(cfg)
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(bits))
    # Xavier weights in the SDF net too: with the geometric initialisation its encoding columns are zero and the grid's
    # first-order gradient would vanish
    tr.initialize_params(seed=1337, sdf_mlp_weights=None)
    of = Field(fp16=True)
    ocams = oc_cams(oracle, cams)
    n_rays, seed = 5000, 40          # about 2^18 marched samples: the batch is nearly full and is rolled over
    n_inf = 280000 // 128 * 128
    results = []
    for step in range(2):            # the second step's samples were generated ahead, beside the first step's kernels
        params16 = host(tr.params).copy()
        tr.step(n_rays=n_rays, n_inference=n_inf, seed=seed + step)
        c = tr.read_counters()
        gpu = {k: host(v) for k, v in tr.last_step(c["rays"], c["samples"], n_inf).items()}
        res = verify_step(of, params16, ocams, rgba, bits, n_rays, step * n_rays, seed + step, n_inf, T, c, gpu, host(tr.grads),
                          background=(1.0, 1.0, 1.0), loss_scale=loss_scale, rtol=RTOL)
        results.append(res)
        assert res["samples"] <= n_inf and 0.8 * T < res["compacted"] <= n_inf, res
    assert results[0]["samples"] != results[1]["samples"]   # two different sets of rays


def test_many_rays_whose_batch_is_filled_up(oracle):
    """From 8192 rays on, the compositor places the rays in the batch with the prefix sums of a scan kernel instead of sums
    inside its backward kernel; here such a step keeps fewer samples than the batch holds, so the batch is also filled up by
    roll-over with those offsets.  Every stage against the oracle, as above."""
    import bench
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    from oracle.field import Field
    from oracle.step import verify_step
    T = 1 << 19
    cams, rgba, bits = bench.build_scene()
    cfg = default_config(target_batch_size=T, max_rays_per_batch=1 << 14, max_samples=T, prefetch_samples=True)
    cfg.loss_scale = 8192.0
    tr = Trainer(cfg)
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(bits))
    tr.initialize_params(seed=1338, sdf_mlp_weights=None)
    n_rays, seed, n_inf = 8500, 7, T
    params16 = host(tr.params).copy()
    tr.step(n_rays=n_rays, n_inference=n_inf, seed=seed)
    c = tr.read_counters()
    assert n_rays >= 8192 and c["rays"] > 0 and 0 < c["compacted"] < T, c  # the scan kernel goes by the rays asked for
    gpu = {k: host(v) for k, v in tr.last_step(c["rays"], c["samples"], n_inf).items()}
    res = verify_step(Field(fp16=True), params16, oc_cams(oracle, cams), rgba, bits, n_rays, 0, seed, n_inf, T, c, gpu, host(tr.grads),
                      background=(1.0, 1.0, 1.0), loss_scale=8192.0, rtol=RTOL)
    assert res["compacted"] == c["compacted"]
