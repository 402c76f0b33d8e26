"""CPU oracle of the SDF network with its eikonal second-order path (grid + 48-64-16 MLP without the colour branch):

    loss = mean |sdf| + w_ek * mean (|grad sdf| - 1)^2

composed from the oracle's grid and MLP functions the way NerfNetwork composes them (nerf_network.h:184-234 forward and
normals, :402-429 first-order backward, :534-571 second-order backward).

TEST INFRASTRUCTURE ONLY (see oracle/neus2_oracle.cpp): imported by tests/ and by bench.py's cpu_baseline leg.  Pinned
through its pieces (tests/test_oracle_grid.py, tests/test_oracle_mlp.py: torch autograd and double backward of an
independent fp64 forward).
"""
import numpy as np

from . import oracle


def q16(a):
    return oracle.round_fp16(np.asarray(a, np.float32))


def sdf_eikonal_step(P, W, x, ek_weight, loss_scale):
    og = oracle.Grid(16, 19, 16, 1.447)
    om = oracle.Mlp(48, 64, 1, 16)
    n = x.shape[1]
    enc, J = og.forward(P, x, want_dy_dx=True)
    inp = np.zeros((48, n), np.float32)
    inp[0:3] = q16(q16(x) - 0.5)
    inp[3:35] = q16(enc)
    y, h = om.forward(W, inp, round_hidden=True)
    e0 = np.zeros((16, n), np.float32)
    e0[0] = 1
    g, _ = om.backward(W, inp, h, e0, want_dW=False)
    g = q16(g)
    normal = np.einsum("rnd,rn->dn", J, g[3:35]) + g[0:3]
    sdf = q16(y[0])
    norm = np.maximum(np.linalg.norm(normal, axis=0), 1e-12)
    loss = np.abs(sdf).mean() + ek_weight * ((norm - 1) ** 2).mean()
    dL_dy = np.zeros((16, n), np.float32)
    dL_dy[0] = q16(np.sign(sdf) * (loss_scale / n))
    v = (normal * (2 * ek_weight * (norm - 1) / norm * (loss_scale / n))).astype(np.float32)
    d_inp, dW = om.backward(W, inp, h, dL_dy)
    grad, _ = og.backward(P, x, q16(d_inp)[3:35], want_dx=False)
    grad, jv, _ = og.backward_backward_input(P, x, v, g[3:35], grad=grad, want_dinput=False)
    v_in = np.zeros((48, n), np.float32)
    v_in[0:3] = q16(v)
    v_in[3:35] = q16(jv)
    dW, _ = om.backward_backward_input(W, h, v_in, e0, dW=dW)
    return dict(sdf=sdf, normal=normal, loss=loss, grid_grad=grad, mlp_grad=dW, offset=og.offset)
