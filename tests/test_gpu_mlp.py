"""GPU parity of the fully fused MLP kernels against the CPU oracle, through the C ABI."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, assert_grad_close, dev, host, q16, rel_l2

pytestmark = pytest.mark.gpu
# A hidden pre-activation within fp32 summation-order error of zero can land on
# either side of the ReLU; allow that for at most one entry in 10^4.
FLIP = 1e-4
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def make(oracle, in_w, n_hidden, seed, scale=0.3):
    from neus2_amd.tcnn_api import FullyFusedMLP
    om = oracle.Mlp(in_w, 64, n_hidden, 16)
    gm = FullyFusedMLP(in_w, n_hidden)
    assert gm.n_params() == om.n_params
    rng = np.random.default_rng(seed)
    W = q16(rng.standard_normal(om.n_params) * scale)
    dW = dev(W, torch.float16)
    dG = torch.zeros_like(dW)
    gm.set_params(dW, dG)
    return om, gm, W, dW, dG, rng


SHAPES = [(48, 1), (48, 2), (32, 1), (16, 1), (64, 2), (64, 1), (32, 2), (16, 2)]


@pytest.mark.parametrize("in_w,n_hidden", SHAPES)
@pytest.mark.parametrize("n", [8, 64, 200, 4096 + 72])
def test_forward(oracle, in_w, n_hidden, n):
    from neus2_amd.tcnn_api import LAYOUT_AOS, LAYOUT_SOA
    om, gm, W, *_ , rng = make(oracle, in_w, n_hidden, 1)
    x = q16(rng.standard_normal((in_w, n)))
    ref_y, ref_h = om.forward(W, x, round_hidden=True)
    y, hid = gm.forward(dev(x, torch.float16), LAYOUT_SOA, want_hidden=True)
    assert_close(host(y), ref_y, what="mlp forward SoA", outlier_frac=FLIP)
    assert_close(host(hid), ref_h.reshape(-1, n), what="hidden activations", outlier_frac=FLIP)
    y2, _ = gm.forward(dev(x, torch.float16), LAYOUT_AOS)
    assert torch.equal(y2.t().contiguous(), y)


@pytest.mark.parametrize("in_w,n_hidden", SHAPES)
@pytest.mark.parametrize("n", [8, 136, 10000])  # less than one wave's tile, a ragged second round of 128, many rounds per workgroup
def test_backward_all_modes(oracle, in_w, n_hidden, n):
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_IGNORE, GRAD_OVERWRITE, LAYOUT_AOS, LAYOUT_SOA
    om, gm, W, dW, dG, rng = make(oracle, in_w, n_hidden, 2)
    x = q16(rng.standard_normal((in_w, n)))
    dy = q16(rng.standard_normal((16, n)))
    _, h = om.forward(W, x, round_hidden=True)
    ref_dx, ref_dW = om.backward(W, x, h, dy)
    dx_, ddy = dev(x, torch.float16), dev(dy, torch.float16)
    dG.fill_(3.0)
    dx = gm.backward(dx_, ddy, LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE)
    assert_close(host(dx), ref_dx, what="dL_dinput", outlier_frac=FLIP)
    # fp32 accumulation over the batch, one rounding to fp16 at the end
    assert_grad_close(host(dG), ref_dW, what="weight gradients")
    # AoS gradient layout gives the same result
    dG.zero_()
    dx2 = gm.backward(dx_, ddy.t().contiguous(), LAYOUT_AOS, want_input_grad=True, mode=GRAD_OVERWRITE)
    assert torch.equal(dx, dx2)
    assert_grad_close(host(dG), ref_dW, what="weight gradients (AoS dL_dy)")
    # Ignore: gradient buffer untouched
    before = dG.clone()
    dx3 = gm.backward(dx_, ddy, LAYOUT_SOA, want_input_grad=True, mode=GRAD_IGNORE)
    assert torch.equal(before, dG) and torch.equal(dx3, dx)
    # Accumulate, without input gradient
    none = gm.backward(dx_, ddy, LAYOUT_SOA, want_input_grad=False, mode=GRAD_ACCUMULATE)
    assert none is None
    assert_grad_close(host(dG), 2 * ref_dW, what="accumulated weight gradients")


@pytest.mark.parametrize("in_w,n_hidden", [(48, 2), (48, 1), (32, 2)])
def test_output_gradients_in_the_subnormal_range(oracle, in_w, n_hidden):
    """Output gradients of 2e-6 (what a loss scale of 128 over 5000 rays gives the colour rows): the hidden layers' gradients
    are fp16 matrices inside the kernel and would be rounded in steps of 6e-8.  With the exponent set, the kernel works on
    2^k times the values and the results are held to the same bounds as gradients of order one; exponent 0 reproduces the
    plain call bit for bit on gradients that lose nothing."""
    from neus2_amd import capi
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, LAYOUT_SOA
    om, gm, W, dW, dG, rng = make(oracle, in_w, n_hidden, 12)
    n = 20000
    x = q16(rng.standard_normal((in_w, n)))
    dy = np.zeros((16, n), np.float32)
    dy[:3] = q16(rng.standard_normal((3, n)) * 2e-6)     # subnormal fp16 values, as the compositor stores them
    assert 0 < np.abs(dy[:3]).max() < 6.1e-5
    _, h = om.forward(W, x, round_hidden=True)
    ref_dx, ref_dW = om.backward(W, x, h, dy)
    dx_, ddy = dev(x, torch.float16), dev(dy, torch.float16)
    k = capi.lib().n2_colour_gradient_exponent(C.c_float(128.0), C.c_uint32(5000))
    assert k == 9                                        # 128 / 5000 * 2^9 = 13.1 <= 16 < 26.2
    gm.set_output_gradient_exponent(k)
    gm.backward(dx_, ddy, LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE)
    assert_grad_close(host(dG), ref_dW, what="weight gradients of subnormal output gradients")
    # without it the same call misses the bound (which is what the exponent is for)
    gm.set_output_gradient_exponent(0)
    gm.backward(dx_, ddy, LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE)
    assert rel_l2(host(dG), ref_dW) > RTOL
    # gradients of order one: the exponent changes nothing but the last bit of sums whose rounding it moves
    dy1 = q16(rng.standard_normal((16, n)))
    ref_dx1, ref_dW1 = om.backward(W, x, h, dy1)
    for kk in (0, 3):
        gm.set_output_gradient_exponent(kk)
        dx = gm.backward(dx_, dev(dy1, torch.float16), LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE)
        assert_close(host(dx), ref_dx1, what=f"dL_dinput, exponent {kk}", outlier_frac=FLIP)
        assert_grad_close(host(dG), ref_dW1, what=f"weight gradients, exponent {kk}")
    gm.set_output_gradient_exponent(0)
    with pytest.raises(capi.N2Error):
        gm.set_output_gradient_exponent(15)


def test_colour_gradient_exponent_rule():
    """Largest k with loss_scale / n_rays * 2^k <= 16, clamped to [0, 14]."""
    from neus2_amd import capi
    f = lambda ls, n: capi.lib().n2_colour_gradient_exponent(C.c_float(ls), C.c_uint32(n))
    assert f(128.0, 5000) == 9 and f(128.0, 50000) == 12 and f(8192.0, 5000) == 3 and f(128.0, 8) == 0 and f(128.0, 1) == 0
    assert f(1.0, 1 << 20) == 14 and f(0.0, 10) == 0 and f(128.0, 0) == 0
    for ls, n in ((128.0, 4992), (100.0, 777), (3.0, 65536)):
        k = f(ls, n)
        assert ls / n * 2.0 ** k <= 16.0 and (k == 14 or ls / n * 2.0 ** (k + 1) > 16.0)


@pytest.mark.parametrize("in_w", [48, 32, 16, 64])
def test_backward_backward_input(oracle, in_w):
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_IGNORE, GRAD_OVERWRITE
    om, gm, W, dW, dG, rng = make(oracle, in_w, 1, 3)
    n = 8192 + 40
    x = q16(rng.standard_normal((in_w, n)))
    v = q16(rng.standard_normal((in_w, n)))
    g = q16(rng.standard_normal((16, n)))
    _, h = om.forward(W, x, round_hidden=True)
    ref_dW, ref_out = om.backward_backward_input(W, h, v, g)
    out = gm.backward_backward_input(dev(x, torch.float16), dev(v, torch.float16), dev(g, torch.float16),
                                     want_dL_ddLdoutput=True, mode=GRAD_OVERWRITE)
    assert_close(host(out), ref_out, what="dL_ddLdoutput", outlier_frac=FLIP)
    assert_grad_close(host(dG), ref_dW, what="second-order weight gradients")
    # the reference's call: g = e_0, Accumulate on top of first-order gradients, no outputs
    e0 = np.zeros((16, n), np.float32)
    e0[0] = 1
    ref2, _ = om.backward_backward_input(W, h, v, e0)
    base = q16(rng.standard_normal(om.n_params))
    dG.copy_(dev(base, torch.float16))
    none = gm.backward_backward_input(dev(x, torch.float16), dev(v, torch.float16), dev(e0, torch.float16),
                                      want_dL_ddLdoutput=False, mode=GRAD_ACCUMULATE)
    assert none is None
    assert_grad_close(host(dG), base + ref2, what="accumulated second-order gradients")
    before = dG.clone()
    gm.backward_backward_input(dev(x, torch.float16), dev(v, torch.float16), dev(e0, torch.float16), mode=GRAD_IGNORE)
    assert torch.equal(before, dG)


def test_geometric_init_sphere_on_gpu(oracle):
    """The reference's utils/mlp_weights.txt through the GPU path: identical to the oracle's sphere."""
    from neus2_amd.tcnn_api import GRAD_IGNORE, FullyFusedMLP
    W = q16(np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")))
    om = oracle.Mlp(48, 64, 1, 16)
    gm = FullyFusedMLP(48, 1)
    gm.set_params(dev(W, torch.float16), None)
    rng = np.random.default_rng(0)
    n = 1 << 14
    x = np.zeros((48, n), np.float32)
    x[:3] = q16(rng.random((3, n)) - 0.5)
    ref_y, h = om.forward(W, x, round_hidden=True)
    y, _ = gm.forward(dev(x, torch.float16))
    assert_close(host(y), ref_y, what="sdf of the geometric init")
    e0 = np.zeros((16, n), np.float32)
    e0[0] = 1
    ref_dx, _ = om.backward(W, x, h, e0, want_dW=False)
    dx = gm.backward(dev(x, torch.float16), dev(e0, torch.float16), want_input_grad=True, mode=GRAD_IGNORE)
    assert_close(host(dx), ref_dx, what="normals of the geometric init")


def test_mlp_errors(oracle):
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, FullyFusedMLP, N2Error
    with pytest.raises(N2Error, match="in_width"):
        FullyFusedMLP(40, 1)
    with pytest.raises(N2Error, match="n_hidden_layers"):
        FullyFusedMLP(48, 3)
    m = FullyFusedMLP(48, 2)
    x = torch.zeros((48, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(N2Error, match="set_params"):
        m.forward(x)
    m.set_params(torch.zeros(m.n_params(), dtype=torch.float16, device="cuda"), None)
    with pytest.raises(N2Error, match="multiple of 8"):
        m.forward(torch.zeros((48, 12), dtype=torch.float16, device="cuda"))
    with pytest.raises(N2Error, match="gradient buffer"):
        m.backward(x, torch.zeros((16, 64), dtype=torch.float16, device="cuda"), mode=GRAD_OVERWRITE)
    with pytest.raises(N2Error, match="one hidden layer"):
        m.set_params(torch.zeros(m.n_params(), dtype=torch.float16, device="cuda"),
                     torch.zeros(m.n_params(), dtype=torch.float16, device="cuda"))
        m.backward_backward_input(x, x, torch.zeros((16, 64), dtype=torch.float16, device="cuda"))
    y, _ = m.forward(torch.zeros((48, 0), dtype=torch.float16, device="cuda"))
    assert y.shape == (16, 0)


@pytest.mark.parametrize("in_w,n_hidden", [(48, 1), (48, 2), (32, 1), (64, 2)])
@pytest.mark.parametrize("n", [8, 200, 4096 + 72])
def test_forward_and_input_gradient_equals_the_two_calls(oracle, in_w, n_hidden, n):
    """The fused pass writes exactly what forward and input_gradient write separately (same arithmetic, one read of x)."""
    from neus2_amd.tcnn_api import LAYOUT_AOS, LAYOUT_SOA
    om, gm, W, *_, rng = make(oracle, in_w, n_hidden, 7)
    x = dev(q16(rng.standard_normal((in_w, n))), torch.float16)
    for dim in (0, 5):
        y_ref, _ = gm.forward(x, LAYOUT_SOA)
        d_ref = gm.input_gradient(x, dim)
        y, d = gm.forward_and_input_gradient(x, dim, LAYOUT_SOA)
        assert torch.equal(y, y_ref) and torch.equal(d, d_ref)
        y2, d2 = gm.forward_and_input_gradient(x, dim, LAYOUT_AOS)
        assert torch.equal(y2.t().contiguous(), y_ref) and torch.equal(d2, d_ref)


def test_deferred_reduction_sums_pending_passes_in_one_launch(oracle):
    """backward(OVERWRITE) + second-order pass(ACCUMULATE) with the reduction deferred: the gradients appear only after
    reduce_deferred, equal the oracle's sum, and two networks reduce in one call."""
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE, LAYOUT_SOA, N2Error
    om, gm, W, dW, dG, rng = make(oracle, 48, 1, 11)
    om2, gm2, W2, dW2, dG2, _ = make(oracle, 32, 2, 12)
    n = 8192 + 40
    x = q16(rng.standard_normal((48, n)))
    v = q16(rng.standard_normal((48, n)))
    g = q16(rng.standard_normal((16, n)) * 0.1)
    x2 = q16(rng.standard_normal((32, n)))
    g2 = q16(rng.standard_normal((16, n)) * 0.1)
    _, h = om.forward(W, x, round_hidden=True)
    ref1 = om.backward(W, x, h, g)[1]
    e0 = np.zeros((16, n), np.float32)
    e0[0] = 1
    ref2, _ = om.backward_backward_input(W, h, v, e0)
    _, h2 = om2.forward(W2, x2, round_hidden=True)
    ref3 = om2.backward(W2, x2, h2, g2)[1]
    gm.set_deferred_reduction(True)
    gm2.set_deferred_reduction(True)
    dG.fill_(7.0)
    dG2.fill_(7.0)
    gm.backward(dev(x, torch.float16), dev(g, torch.float16), LAYOUT_SOA, want_input_grad=False, mode=GRAD_OVERWRITE)
    gm.backward_backward_input(dev(x, torch.float16), dev(v, torch.float16), None, mode=GRAD_ACCUMULATE)
    gm2.backward(dev(x2, torch.float16), dev(g2, torch.float16), LAYOUT_SOA, want_input_grad=False, mode=GRAD_OVERWRITE)
    torch.cuda.synchronize()
    assert (dG == 7.0).all() and (dG2 == 7.0).all()      # nothing folded yet
    with pytest.raises(N2Error):                          # OVERWRITE cannot follow a pending pass
        gm.backward(dev(x, torch.float16), dev(g, torch.float16), LAYOUT_SOA, want_input_grad=False, mode=GRAD_OVERWRITE)
    with pytest.raises(N2Error):                          # nor can the switch be flipped with passes pending
        gm.set_deferred_reduction(False)
    gm.reduce_deferred(gm2)
    assert_grad_close(host(dG), ref1 + ref2, what="deferred first + second order weight gradients")
    assert_grad_close(host(dG2), ref3, what="deferred gradients of the second network")
    # nothing pending: a second reduce is a no-op, and ACCUMULATE as first pending pass adds to the buffer
    before = dG.clone()
    gm.reduce_deferred()
    assert torch.equal(before, dG)
    gm.backward(dev(x, torch.float16), dev(g, torch.float16), LAYOUT_SOA, want_input_grad=False, mode=GRAD_ACCUMULATE)
    gm.reduce_deferred()
    assert_grad_close(host(dG), 2 * ref1 + ref2, what="accumulate through a deferred reduction")
    gm.set_deferred_reduction(False)


@pytest.mark.parametrize("layout", ["soa", "aos"])
def test_backward_rows_equals_backward_of_the_zero_padded_gradient(oracle, layout):
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, LAYOUT_AOS, LAYOUT_SOA
    om, gm, W, dW, dG, rng = make(oracle, 48, 2, 21)
    n = 4096 + 136
    x = dev(q16(rng.standard_normal((48, n))), torch.float16)
    dy = q16(rng.standard_normal((16, n)))
    padded = dy.copy()
    padded[3:] = 0
    lay = LAYOUT_AOS if layout == "aos" else LAYOUT_SOA
    shape = (lambda a: np.ascontiguousarray(a.T)) if layout == "aos" else (lambda a: a)
    dx_ref = gm.backward(x, dev(shape(padded), torch.float16), lay, mode=GRAD_OVERWRITE)
    g_ref = dG.clone()
    dG.fill_(2.0)
    dx = gm.backward_rows(x, dev(shape(dy), torch.float16), 3, lay, mode=GRAD_OVERWRITE)
    assert torch.equal(dx, dx_ref) and torch.equal(dG, g_ref)


@pytest.mark.parametrize("in_w", [48, 32, 16, 64])
@pytest.mark.parametrize("unit", [True, False])
def test_backward_and_second_order_equals_the_two_calls(oracle, in_w, unit):
    """The SDF net's first-order backward and its second-order pass (nerf_network.h:402 and :560-571) in one launch:
    the input gradient is that of backward, the weight gradients are the sum of both passes, against the oracle and
    against the two separate calls."""
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE, LAYOUT_AOS, LAYOUT_SOA
    om, gm, W, dW, dG, rng = make(oracle, in_w, 1, 31)
    n = 8192 + 72
    x = q16(rng.standard_normal((in_w, n)))
    dy = q16(rng.standard_normal((16, n)))
    v = q16(rng.standard_normal((in_w, n)))
    g = np.zeros((16, n), np.float32)
    if unit:
        g[0] = 1
    else:
        g[:] = q16(rng.standard_normal((16, n)))
    _, h = om.forward(W, x, round_hidden=True)
    ref_dx, ref1 = om.backward(W, x, h, dy)
    ref2, _ = om.backward_backward_input(W, h, v, g)
    dx_, ddy, dv = dev(x, torch.float16), dev(dy, torch.float16), dev(v, torch.float16)
    dg = None if unit else dev(g, torch.float16)
    # the two calls
    dx_two = gm.backward(dx_, ddy, LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE)
    gm.backward_backward_input(dx_, dv, dg, mode=GRAD_ACCUMULATE)
    two = host(dG)
    # one launch
    dG.fill_(5.0)
    dx_one = gm.backward_and_second_order(dx_, ddy, dv, dg, mode=GRAD_OVERWRITE)
    one = host(dG)
    assert torch.equal(dx_one, dx_two)
    assert_close(host(dx_one), ref_dx, what="dL_dinput", outlier_frac=FLIP)
    assert_grad_close(one, ref1 + ref2, what="first + second order weight gradients")
    assert rel_l2(one, two) < 1e-3  # the same sums in another order, each rounded to fp16 once
    # AoS first-order gradient, Accumulate on top of what is there
    base = q16(rng.standard_normal(om.n_params))
    dG.copy_(dev(base, torch.float16))
    dx_aos = gm.backward_and_second_order(dx_, ddy.t().contiguous(), dv, dg, dL_layout=LAYOUT_AOS, mode=GRAD_ACCUMULATE)
    assert torch.equal(dx_aos, dx_one)
    assert_grad_close(host(dG), base + ref1 + ref2, what="accumulated first + second order weight gradients")


def test_backward_and_second_order_errors(oracle):
    from neus2_amd.tcnn_api import GRAD_IGNORE, FullyFusedMLP, N2Error
    om, gm, W, dW, dG, rng = make(oracle, 48, 1, 32)
    x = dev(q16(rng.standard_normal((48, 256))), torch.float16)
    dy = dev(q16(rng.standard_normal((16, 256))), torch.float16)
    with pytest.raises(N2Error, match="OVERWRITE or ACCUMULATE"):
        gm.backward_and_second_order(x, dy, x, mode=GRAD_IGNORE)
    om2, gm2, *_ = make(oracle, 48, 2, 33)
    with pytest.raises(N2Error, match="one hidden layer"):
        gm2.backward_and_second_order(x, dy, x)
