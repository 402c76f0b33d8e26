"""GPU parity of the Adam step against the oracle."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, q16

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,n_matrix", [(12288 + 40000 + 4, 12288), (1003, 0), (1003, 1003), (7, 3)])
def test_adam_steps_match_oracle(oracle, n, n_matrix):
    from neus2_amd.tcnn_api import Adam
    rng = np.random.default_rng(n)
    w0 = rng.standard_normal(n).astype(np.float32)
    w, m1, m2, steps = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint32)
    d_master = dev(w0.copy())
    d_params = d_master.half()  # the trainer's invariant: fp16 copy == round(master)
    opt = Adam(d_master, n_matrix)
    for it in range(4):
        g = q16(rng.standard_normal(n) * 128)
        g[rng.random(n) < 0.7] = 0  # sparse gradients, as the hash table sees them
        oracle.adam_step(w, g, m1, m2, steps, n_matrix_params=n_matrix)
        opt.step(d_params, dev(g, torch.float16))
        np.testing.assert_allclose(host(opt.master), w, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(host(opt.m1), m1, rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(host(opt.m2), m2, rtol=1e-5, atol=1e-7)
        assert np.array_equal(host(opt.steps).view(np.uint32), steps)
        np.testing.assert_array_equal(host(d_params), q16(host(opt.master)))
    # non-matrix parameters whose gradient was zero every time never moved
    never = steps == 0
    np.testing.assert_array_equal(host(opt.master)[never], w0[never])


def test_adam_errors():
    from neus2_amd.tcnn_api import Adam, N2Error
    m = torch.zeros(16, device="cuda")
    opt = Adam(m, 8)
    with pytest.raises(N2Error):
        opt.step(torch.zeros(8, dtype=torch.float16, device="cuda"), torch.zeros(16, dtype=torch.float16, device="cuda"))
    with pytest.raises(N2Error, match="loss_scale"):
        opt.step(torch.zeros(16, dtype=torch.float16, device="cuda"), torch.zeros(16, dtype=torch.float16, device="cuda"), 0.0)


@pytest.mark.parametrize("n", [4096 + 3, 5])
def test_ema_steps_match_oracle(oracle, n):
    """The Ema wrapper's kernel (bias-corrected moving average of the fp16 weights) against the oracle."""
    import ctypes as C
    from neus2_amd import capi
    rng = np.random.default_rng(n)
    tmp = np.zeros(n, np.float32)
    d_tmp = dev(tmp.copy())
    d_ema = torch.zeros(n, dtype=torch.float16, device="cuda")
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for t in range(1, 8):
        w = q16(rng.standard_normal(n))
        want = oracle.ema_step(w, tmp, t, 0.95)
        capi.check(capi.lib().n2_ema_step(s, C.c_uint32(n), C.c_float(0.95), C.c_uint32(t), capi.ptr(dev(w, torch.float16)), capi.ptr(d_tmp),
                                          capi.ptr(d_ema)), "n2_ema_step")
        np.testing.assert_allclose(host(d_tmp), tmp, rtol=2e-6, atol=2e-7)  # fma contraction on one side only
        assert (np.abs(host(d_ema) - want) <= 2.0 ** -10 * np.abs(want) + 1e-7).all()
    with pytest.raises(capi.N2Error):
        capi.check(capi.lib().n2_ema_step(s, C.c_uint32(n), C.c_float(1.5), C.c_uint32(1), capi.ptr(d_ema), capi.ptr(d_tmp), capi.ptr(d_ema)))
    with pytest.raises(capi.N2Error):
        capi.check(capi.lib().n2_ema_step(s, C.c_uint32(n), C.c_float(0.95), C.c_uint32(0), capi.ptr(d_ema), capi.ptr(d_tmp), capi.ptr(d_ema)))


def test_trainer_with_ema_and_decaying_learning_rate(oracle):
    """Ema(ExponentialDecay(Adam)) as configs/nerf/base.json nests them: the inference copy follows the oracle's moving
    average of the working weights, and the schedule lowers the step size of later steps."""
    from neus2_amd import scene
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import ExponentialDecay, Trainer, default_config
    cams = scene.cameras_on_sphere(8, 96)
    rgba = scene.render_sphere_images(cams)
    T = 4096
    tr = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=1 << 17, ema_decay=0.95))
    tr.set_scene(pack_cameras(cams), len(cams), dev(rgba), dev(scene.sphere_bitfield()))
    tr.initialize_params(seed=5)
    tr.lr_schedule = ExponentialDecay(1e-3, decay_start=2, decay_interval=2, decay_base=0.5)
    assert tr.ema_weights is not None and not host(tr.ema_weights).any()
    tmp = np.zeros(tr.n_params, np.float32)
    lrs, moved = [], []
    for t in range(1, 6):
        before = host(tr.master).copy()
        tr.step(n_rays=256, n_inference=1 << 17)
        want = oracle.ema_step(host(tr.params), tmp, t, 0.95)
        np.testing.assert_allclose(host(tr.ema_weights), tmp, rtol=2e-6, atol=2e-7)
        assert (np.abs(host(tr.inference_params) - want) <= 2.0 ** -10 * np.abs(want) + 1e-7).all()
        s = tr.optimizer_state()
        assert s.optimizer_steps == t
        lrs.append(s.learning_rate)
        moved.append(np.abs(host(tr.master) - before)[:4096].max())  # SDF MLP weights: every one moves by about lr
    np.testing.assert_allclose(lrs, [1e-3, 5e-4, 5e-4, 2.5e-4, 2.5e-4], rtol=1e-6)
    # Adam's first steps move each weight by about the learning rate: steps taken at half the rate are about half as long
    assert 0.3 < moved[2] / moved[0] < 0.75 and 0.1 < moved[4] / moved[0] < 0.4
    # without the wrapper the inference parameters are the working copy
    tr2 = Trainer(default_config(target_batch_size=T, max_rays_per_batch=2048, max_samples=1 << 17))
    assert tr2.ema_weights is None and tr2.inference_params.data_ptr() == tr2.params.data_ptr()
