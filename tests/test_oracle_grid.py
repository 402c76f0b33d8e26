"""Pins the oracle's hash-grid functions without the (absent) tcnn source."""
import numpy as np
import pytest
import torch
from scipy import ndimage

from torch_ref import grid_forward as t_grid_forward

RES = [16, 24, 34, 49, 71, 102, 147, 213, 308, 445, 644, 932, 1349, 1951, 2823, 4085]
ENTRIES = [4096, 13824, 39304, 117656, 357912] + [524288] * 11


@pytest.fixture(scope="module")
def grid(oracle):
    return oracle.Grid(16, 19, 16, 1.447)


def test_level_table_matches_published(grid):
    assert grid.resolution.tolist() == RES
    assert grid.entries.tolist() == ENTRIES
    assert int(grid.offset[-1]) == 6299960
    assert grid.n_params == 12599920
    assert abs(grid.scale[0] - 15.0) < 1e-4 and abs(grid.scale[15] - 4083.5872) < 0.05
    np.testing.assert_array_equal(np.diff(grid.offset.astype(np.int64)), ENTRIES)


def test_small_table_geometry(oracle):
    g = oracle.Grid(4, 10, 4, 2.0)  # scales 3,7,15,31 -> res 4,8,16,32
    assert g.resolution.tolist() == [4, 8, 16, 32]
    assert g.entries.tolist() == [64, 512, 1024, 1024]


def _np_index(grid, l, gx, gy, gz):
    """uint32 closed form, vectorised in numpy."""
    r, n = np.uint32(grid.resolution[l]), np.uint32(grid.entries[l])
    dense = int(grid.resolution[l]) ** 3 <= int(grid.entries[l])
    with np.errstate(over="ignore"):
        if dense:
            i = gx + gy * r + gz * r * r
        else:
            i = gx ^ (gy * np.uint32(2654435761)) ^ (gz * np.uint32(805459861))
    return i % n


def test_indices_closed_form_and_invariants(grid):
    rng = np.random.default_rng(0)
    n = 4096
    xyz = rng.random((3, n), dtype=np.float32)
    idx, w = grid.indices(xyz)
    assert idx.dtype == np.uint32
    for l in range(16):
        pos = xyz.astype(np.float32) * grid.scale[l] + np.float32(0.5)
        # fused and unfused products may differ by one ulp only right at a cell
        # boundary; compare on points that are clear of it
        cell = np.floor(pos.astype(np.float64) if False else pos).astype(np.uint32)
        frac = pos - np.floor(pos)
        ok = (np.abs(frac - 0.5) < 0.499).all(0)
        assert ok.mean() > 0.99
        for k in range(8):
            gx = cell[0] + np.uint32(k & 1)
            gy = cell[1] + np.uint32((k >> 1) & 1)
            gz = cell[2] + np.uint32((k >> 2) & 1)
            ref = _np_index(grid, l, gx, gy, gz)
            np.testing.assert_array_equal(idx[l, k][ok], ref[ok])
        assert (idx[l] < grid.entries[l]).all()
        assert ((w[l] >= 0) & (w[l] < 1)).all()
    # dense levels: corner k differs from corner 0 by the dense strides
    for l in range(5):
        r = int(grid.resolution[l])
        inside = (idx[l, 0].astype(np.int64) + 1 + r + r * r) < int(grid.entries[l])
        for k in range(8):
            d = (k & 1) + ((k >> 1) & 1) * r + ((k >> 2) & 1) * r * r
            np.testing.assert_array_equal(idx[l, k][inside].astype(np.int64), idx[l, 0][inside].astype(np.int64) + d)


def test_hash_known_answers(grid):
    # hand-computed uint32 values of x ^ y*2654435761 ^ z*805459861 mod 2^19
    l = 10  # scale ~642.88, hashed
    s = float(grid.scale[l])
    for cell in [(1, 1, 1), (3, 5, 7), (100, 200, 300), (641, 0, 13)]:
        xyz = np.array([[(c + 0.25 - 0.5) / s] for c in cell], np.float32)
        idx, _ = grid.indices(xyz)
        x, y, z = cell
        want = (x ^ ((y * 2654435761) & 0xFFFFFFFF) ^ ((z * 805459861) & 0xFFFFFFFF)) % (1 << 19)
        assert int(idx[l, 0, 0]) == want, cell
        want7 = ((x + 1) ^ (((y + 1) * 2654435761) & 0xFFFFFFFF) ^ (((z + 1) * 805459861) & 0xFFFFFFFF)) % (1 << 19)
        assert int(idx[l, 7, 0]) == want7, cell


def test_forward_matches_scipy_map_coordinates_on_dense_levels(grid):
    rng = np.random.default_rng(1)
    n = 2000
    xyz = (rng.random((3, n)) * 0.9).astype(np.float32)
    params = rng.uniform(-1, 1, grid.n_params).astype(np.float32)
    y = grid.forward(params, xyz)
    for l in range(5):
        r, off = int(grid.resolution[l]), int(grid.offset[l])
        vol = params[off * 2:(off + r ** 3) * 2].reshape(r, r, r, 2)  # [z][y][x][f]
        pos = xyz.astype(np.float64) * float(grid.scale[l]) + 0.5
        for f in range(2):
            ref = ndimage.map_coordinates(vol[..., f].astype(np.float64), [pos[2], pos[1], pos[0]], order=1)
            np.testing.assert_allclose(y[2 * l + f], ref, rtol=0, atol=3e-5 * max(1.0, float(grid.scale[l]) / 16))


def test_forward_vertex_and_partition_of_unity(grid):
    # constant params -> output equals the constant (weights sum to one), every level
    xyz = np.random.default_rng(2).random((3, 512), dtype=np.float32)
    y = grid.forward(np.full(grid.n_params, 0.75, np.float32), xyz)
    np.testing.assert_allclose(y, 0.75, atol=1e-6)
    # a point on a vertex returns that vertex's features
    rng = np.random.default_rng(3)
    params = rng.uniform(-1, 1, grid.n_params).astype(np.float32)
    for l in (0, 3, 7, 15):
        s = float(grid.scale[l])
        cell = np.array([[3], [5], [2]])
        xyz = ((cell - 0.5) / s).astype(np.float32)
        idx, w = grid.indices(xyz)
        y = grid.forward(params, xyz)
        near = int(np.argmax([np.prod([w[l, d, 0] if (k >> d) & 1 else 1 - w[l, d, 0] for d in range(3)]) for k in range(8)]))
        e = int(grid.offset[l]) + int(idx[l, near, 0])
        np.testing.assert_allclose(y[2 * l:2 * l + 2, 0], params[2 * e:2 * e + 2], atol=2e-3)


def _small(oracle):
    # 6 levels: 3 dense + 3 hashed at T=2^12, small enough for fp64 autograd
    return oracle.Grid(6, 12, 4, 1.6)


def test_backward_matches_autograd(oracle):
    g = _small(oracle)
    rng = np.random.default_rng(4)
    n = 300
    xyz = rng.random((3, n)).astype(np.float32)
    params = rng.uniform(-1, 1, g.n_params).astype(np.float32)
    dy = rng.standard_normal((g.n_out, n)).astype(np.float32)
    idx, _ = g.indices(xyz)
    tp = torch.tensor(params, dtype=torch.float64, requires_grad=True)
    tx = torch.tensor(xyz, dtype=torch.float64, requires_grad=True)
    ty = t_grid_forward(tp, tx, g.scale, g.offset, idx)
    y, J = g.forward(params, xyz, want_dy_dx=True)
    np.testing.assert_allclose(y, ty.detach().numpy(), atol=1e-5)
    (ty * torch.tensor(dy, dtype=torch.float64)).sum().backward()
    grad, dx = g.backward(params, xyz, dy)
    np.testing.assert_allclose(grad, tp.grad.numpy(), atol=2e-5)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-4, atol=1e-3)
    # dy_dx against autograd, one output row at a time on a few rows
    for k in (0, 5, 11):
        tx2 = torch.tensor(xyz, dtype=torch.float64, requires_grad=True)
        t_grid_forward(tp.detach(), tx2, g.scale, g.offset, idx)[k].sum().backward()
        np.testing.assert_allclose(J[k].T, tx2.grad.numpy(), rtol=1e-4, atol=1e-3)


def test_backward_backward_input_matches_double_backward(oracle):
    g = _small(oracle)
    rng = np.random.default_rng(5)
    n = 200
    xyz = rng.random((3, n)).astype(np.float32)
    params = rng.uniform(-1, 1, g.n_params).astype(np.float32)
    gg = rng.standard_normal((g.n_out, n)).astype(np.float32)
    v = rng.standard_normal((3, n)).astype(np.float32)
    idx, _ = g.indices(xyz)
    tp = torch.tensor(params, dtype=torch.float64, requires_grad=True)
    tx = torch.tensor(xyz, dtype=torch.float64, requires_grad=True)
    tg = torch.tensor(gg, dtype=torch.float64, requires_grad=True)
    ty = t_grid_forward(tp, tx, g.scale, g.offset, idx)
    (q,) = torch.autograd.grad(ty, tx, tg, create_graph=True)  # first backward: dL_dx
    s = (q * torch.tensor(v, dtype=torch.float64)).sum()
    dp, dg, dxx = torch.autograd.grad(s, [tp, tg, tx])
    grad, out, din = g.backward_backward_input(params, xyz, v, gg)
    sc = float(g.scale.max())
    np.testing.assert_allclose(grad, dp.numpy(), rtol=1e-4, atol=1e-4 * sc)
    np.testing.assert_allclose(out, dg.numpy(), rtol=1e-4, atol=1e-4 * sc)
    np.testing.assert_allclose(din, dxx.numpy(), rtol=1e-3, atol=1e-3 * sc * sc)
    # accumulate semantics: passing an existing gradient adds to it
    base = rng.standard_normal(g.n_params).astype(np.float32)
    grad2, _, _ = g.backward_backward_input(params, xyz, v, gg, grad=base.copy(), want_dinput=False)
    np.testing.assert_allclose(grad2, base + grad, rtol=1e-5, atol=1e-4)


def test_second_derivative_diagonal_vanishes(oracle):
    # trilinear interpolation is linear in each coordinate: with v = e_a and the
    # output restricted to dinput[a] the result must be exactly zero
    g = _small(oracle)
    rng = np.random.default_rng(6)
    n = 64
    xyz = rng.random((3, n)).astype(np.float32)
    params = rng.uniform(-1, 1, g.n_params).astype(np.float32)
    gg = rng.standard_normal((g.n_out, n)).astype(np.float32)
    for a in range(3):
        v = np.zeros((3, n), np.float32)
        v[a] = 1
        _, _, din = g.backward_backward_input(params, xyz, v, gg)
        assert np.all(din[a] == 0)
