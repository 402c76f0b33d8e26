"""Marching cubes and the SDF lattice on the GPU against the oracle, through the C ABI."""
import os

import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, dev, host, q16
from oracle import marching_cubes as omc
from test_oracle_marching_cubes import check_closed_oriented, sphere_lattice

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_case_table_equals_the_oracles():
    from neus2_amd.mesh import case_table
    np.testing.assert_array_equal(case_table(), omc.TRIANGLE_TABLE)


@pytest.mark.parametrize("res,kind", [((40, 48, 32), "sphere"), ((17, 9, 33), "noise"), ((2, 2, 2), "noise"), ((64, 64, 64), "two"),
                                      ((100, 24, 10), "noise"), ((130, 9, 7), "noise"), ((96, 80, 72), "sphere")])  # rows that end inside a wave's 64 points
def test_mesh_matches_oracle(res, kind):
    from neus2_amd.mesh import marching_cubes
    rng = np.random.default_rng(res[0])
    if kind == "sphere":
        f, thresh = sphere_lattice(res), 0.0
    elif kind == "two":  # two overlapping balls, threshold off zero
        f = np.maximum(sphere_lattice(res, (0.4, 0.5, 0.5), 0.2), sphere_lattice(res, (0.65, 0.55, 0.45), 0.15))
        thresh = 0.01
    else:  # every case of the table, ambiguous faces included
        f, thresh = rng.standard_normal((res[2], res[1], res[0])).astype(np.float32), 0.1
    lo, hi = (-0.5, 0.0, 0.25), (1.5, 1.0, 0.75)
    want_v, want_t = omc.marching_cubes(f, res, thresh, lo, hi)
    v, t, n = marching_cubes(dev(f), thresh, lo, hi)
    assert v.shape == (len(want_v), 3) and t.shape == (len(want_t), 3)
    np.testing.assert_array_equal(host(v), want_v)                      # bit-exact vertex positions, same numbering
    np.testing.assert_array_equal(host(t).view(np.uint32), want_t)      # same triangles in the same order
    want_n = omc.vertex_normals(want_v, want_t)
    np.testing.assert_allclose(host(n), want_n, rtol=1e-4, atol=1e-6 * max(1.0, float(np.abs(want_n).max())))
    if kind in ("sphere", "two"):
        assert check_closed_oriented(host(v), host(t).astype(np.int64)) == 2


def test_empty_lattice_and_errors():
    from neus2_amd import capi
    from neus2_amd.mesh import marching_cubes
    v, t, n = marching_cubes(torch.full((8, 8, 8), -1.0, device="cuda"), 0.0)
    assert v.shape == (0, 3) and t.shape == (0, 3)
    with pytest.raises(capi.N2Error):
        marching_cubes(torch.zeros((1, 8, 8), device="cuda"), 0.0)
    with pytest.raises(capi.N2Error):
        marching_cubes(torch.zeros((8, 8, 8), device="cuda", dtype=torch.float16), 0.0)


def test_sdf_lattice_and_mesh_of_the_initial_sphere(oracle, tmp_path):
    """get_density_on_grid + marching cubes on the geometric-init network: the zero level set of its SDF is a sphere of
    radius ~0.1 around the cube centre (sdf ~ |x - 0.5| - 0.1)."""
    from neus2_amd.mesh import density_on_grid, marching_cubes, marching_cubes_resolution, save_mesh
    from neus2_amd.training import Trainer, default_config
    from oracle.field import Field
    tr = Trainer(default_config(target_batch_size=4096, max_rays_per_batch=256, max_samples=1 << 16))
    tr.initialize_params(seed=5, sdf_mlp_weights=np.load(os.path.join(GOLD, "sdf_mlp_weights_48.npy")))
    assert marching_cubes_resolution(40) == (48, 48, 48) and marching_cubes_resolution(64, (0, 0, 0), (1, 0.5, 0.25)) == (64, 32, 16)
    res = (48, 32, 48)
    lo, hi = (0.25, 0.3, 0.25), (0.75, 0.7, 0.75)
    d = density_on_grid(tr._field, res, lo, hi, chunk=1 << 14)  # several chunks, the last one partial
    # lattice positions as the reference computes them, SDF from the oracle's field
    z, y, x = np.meshgrid(np.arange(res[2], dtype=np.float32), np.arange(res[1], dtype=np.float32), np.arange(res[0], dtype=np.float32), indexing="ij")
    ext = np.asarray(hi, np.float32) - np.asarray(lo, np.float32)
    pos = np.stack([(x * np.float32(1.0 / res[0])) * ext[0] + np.float32(lo[0]), (y * np.float32(1.0 / res[1])) * ext[1] + np.float32(lo[1]),
                    (z * np.float32(1.0 / res[2])) * ext[2] + np.float32(lo[2])]).reshape(3, -1)
    want = Field(fp16=True).sdf_values(host(tr.params), pos)[0].reshape(res[2], res[1], res[0])
    assert_close(host(d), want, rtol=RTOL, what="SDF lattice", outlier_frac=1e-3)
    v, t, n = marching_cubes(d, 0.0, lo, hi)
    vv, tt = host(v), host(t).astype(np.int64)
    assert len(tt) > 500 and check_closed_oriented(vv, tt) == 2
    r = np.linalg.norm(vv - 0.5, axis=1)
    assert abs(r.mean() - 0.1) < 0.03 and r.std() < 0.04  # 64 random neurons: a lumpy sphere
    # OBJ and PLY as the reference writes them
    for ext_ in ("obj", "ply"):
        p = tmp_path / f"mesh.{ext_}"
        save_mesh(p, vv, host(n), tt)
        text = p.read_text().splitlines()
        if ext_ == "obj":
            assert sum(l.startswith("v ") for l in text) == len(vv) and sum(l.startswith("vn ") for l in text) == len(vv)
            faces = [l for l in text if l.startswith("f ")]
            assert len(faces) == len(tt)
            a, b, c = (int(tok.split("//")[0]) - 1 for tok in faces[0].split()[1:])
            assert (a, b, c) == (tt[0][2], tt[0][1], tt[0][0])  # reversed winding, 1-based
        else:
            assert text[0] == "ply" and f"element vertex {len(vv)}" in text and f"element face {len(tt)}" in text
            assert len(text) == text.index("end_header") + 1 + len(vv) + len(tt)
