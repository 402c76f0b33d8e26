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
