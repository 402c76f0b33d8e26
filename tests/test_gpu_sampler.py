"""GPU parity of the training-sample generator: bit-exact against the oracle."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host
from neus2_amd import scene
from test_oracle_sampler import oc_cams

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sc(oracle):
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield()
    return cams, rgba, bits


@pytest.mark.parametrize("n_rays,total,seed,cap", [(4096, 0, 1, 1 << 19), (1000, 7777, 5, 1 << 19), (4096, 0, 2, 20000), (1, 0, 3, 4096),
                                                  (70000, 0, 4, 1 << 19)])  # dozens of scan blocks, the budget cut in the middle
def test_sampler_bit_exact(oracle, sc, n_rays, total, seed, cap):
    from neus2_amd.tcnn_api import generate_training_samples, pack_cameras
    cams, rgba, bits = sc
    bg = (0.25, 0.5, 0.75)
    ref = oracle.generate_training_samples(n_rays, total, seed, oc_cams(oracle, cams), rgba, bg, bits, cap)
    got = generate_training_samples(n_rays, total, seed, pack_cameras(cams), len(cams), dev(rgba), bg, dev(bits), cap)
    k = ref["ray_counter"]
    assert int(host(got["ray_counter"])[0]) == k
    assert int(host(got["sample_counter"])[0]) == ref["sample_counter"]
    assert np.array_equal(host(got["ray_indices"]).view(np.uint32)[:k], ref["ray_indices"][:k])
    assert np.array_equal(host(got["numsteps"]).view(np.uint32)[:k], ref["numsteps"][:k])
    assert np.array_equal(host(got["rgb_target"])[:k], ref["rgb_target"][:k])
    n_samples = int(ref["numsteps"][:k, 0].sum()) if k else 0
    # positions, dt and directions: identical bits
    assert np.array_equal(host(got["coords"])[:n_samples].view(np.uint32), ref["coords"][:n_samples].view(np.uint32))
    if cap == 20000:
        assert ref["sample_counter"] > cap  # the budget path is exercised


def test_sampler_full_and_empty_bitfield(oracle, sc):
    from neus2_amd.tcnn_api import generate_training_samples, pack_cameras
    cams, rgba, _ = sc
    for fill in (0, 255):
        bits = np.full(128 ** 3 // 8, fill, np.uint8)
        ref = oracle.generate_training_samples(512, 0, 9, oc_cams(oracle, cams), rgba, (0, 0, 0), bits, 1 << 20)
        got = generate_training_samples(512, 0, 9, pack_cameras(cams), len(cams), dev(rgba), (0, 0, 0), dev(bits), 1 << 20)
        assert int(host(got["ray_counter"])[0]) == ref["ray_counter"]
        assert int(host(got["sample_counter"])[0]) == ref["sample_counter"]
        n = ref["sample_counter"]
        assert np.array_equal(host(got["coords"])[:n], ref["coords"][:n])
    r0 = generate_training_samples(0, 0, 9, pack_cameras(cams), len(cams), dev(rgba), (0, 0, 0), dev(bits), 64)
    assert int(host(r0["ray_counter"])[0]) == 0
