"""Pins the marching-cubes oracle: the derived case table (against the reference's table when its source is present,
and by construction), and the extracted mesh by the properties a closed surface must have."""
import os
import re

import numpy as np
import pytest

from oracle import marching_cubes as mc

REF = "/root/reference/src/marching_cubes.cu"


def contour(row):
    """Directed segments on the cube's faces: triangle edges that no other triangle of the case uses backwards."""
    tris = [tuple(int(x) for x in row[k:k + 3]) for k in range(0, 15, 3) if row[k] >= 0]
    d = {(t[k], t[(k + 1) % 3]) for t in tris for k in range(3)}
    return sorted((a, b) for (a, b) in d if (b, a) not in d)


def test_table_rows_close_up_on_every_case():
    T = mc.TRIANGLE_TABLE
    assert list(T[0]) == [-1] * 16 and list(T[255]) == [-1] * 16 and list(T[1][:4]) == [0, 8, 3, -1]
    for mask in range(256):
        cut = {e for e, (a, b) in enumerate(mc.EDGES) if ((mask >> a) & 1) != ((mask >> b) & 1)}
        row = T[mask]
        used = {int(e) for e in row if e >= 0}
        assert used == cut, mask                              # exactly the cut edges carry vertices
        segs = contour(row)
        assert sorted(segs) == sorted(mc.face_segments(mask)), mask   # the triangles' boundary is the face contour
        # every boundary edge enters and leaves each cut edge once: closed loops
        assert sorted(a for a, _ in segs) == sorted(cut) and sorted(b for _, b in segs) == sorted(cut), mask


def test_neighbouring_cubes_agree_on_shared_faces():
    """The contour on a face depends only on that face's four corners, so two cubes sharing it draw the same segments
    (with opposite directions, as they see the face from opposite sides)."""
    def on_face(mask, axis, side):
        cs = {i for i in range(8) if mc.CORNERS[i][axis] == side}
        out = set()
        for a, b in mc.face_segments(mask):
            ea, eb = mc.EDGES[a], mc.EDGES[b]
            if set(ea) <= cs and set(eb) <= cs:
                # name the edges by their corner coordinates within the face, so both cubes use the same names
                key = lambda e: tuple(sorted(tuple(np.delete(mc.CORNERS[c], axis)) for c in e))
                out.add((key(ea), key(eb)))
        return out
    rng = np.random.default_rng(0)
    for axis in range(3):
        for _ in range(300):
            left, right = int(rng.integers(0, 256)), int(rng.integers(0, 256))
            # make the right cube's side-0 face equal to the left cube's side-1 face
            for i in range(8):
                if mc.CORNERS[i][axis] == 0:
                    j = [k for k in range(8) if (np.delete(mc.CORNERS[k], axis) == np.delete(mc.CORNERS[i], axis)).all() and mc.CORNERS[k][axis] == 1][0]
                    right = (right & ~(1 << i)) | (((left >> j) & 1) << i)
            a, b = on_face(left, axis, 1), on_face(right, axis, 0)
            assert a == {(y, x) for (x, y) in b}


@pytest.mark.skipif(not os.path.exists(REF), reason="reference source not present")
def test_table_has_the_reference_tables_contours():
    """Read as text, not run: for all 256 cases the reference's triangle_table has the same directed face contour and the
    same number of triangles as the derived table, i.e. the same surface; rows may differ in how polygons are cut."""
    src = open(REF).read()
    i = src.index("triangle_table[256][16]")
    body = src[i:src.index("};", i)]
    nums = [int(x) for x in re.findall(r"-?\d+", body[body.index("{"):])]
    ref = np.array(nums[:4096]).reshape(256, 16)
    for mask in range(256):
        assert contour(ref[mask]) == contour(mc.TRIANGLE_TABLE[mask]), mask
        assert (ref[mask] >= 0).sum() == (mc.TRIANGLE_TABLE[mask] >= 0).sum(), mask


def sphere_lattice(res, centre=(0.5, 0.5, 0.5), radius=0.3):
    rx, ry, rz = res
    z, y, x = np.meshgrid(np.arange(rz) / rz, np.arange(ry) / ry, np.arange(rx) / rx, indexing="ij")
    # "density" grows towards the inside, like the quantity the reference thresholds
    return (radius - np.sqrt((x - centre[0]) ** 2 + (y - centre[1]) ** 2 + (z - centre[2]) ** 2)).astype(np.float32)


def check_closed_oriented(verts, tris):
    e = np.concatenate([tris[:, [0, 1]], tris[:, [1, 2]], tris[:, [2, 0]]]).astype(np.int64)
    key = e[:, 0] * (len(verts) + 1) + e[:, 1]
    rev = e[:, 1] * (len(verts) + 1) + e[:, 0]
    assert len(np.unique(key)) == len(key)                       # no directed edge twice
    assert np.array_equal(np.sort(key), np.sort(rev))            # every edge has its opposite: closed and consistently oriented
    n_e = len(key) // 2
    return len(verts) - n_e + len(tris)                           # Euler characteristic


def test_sphere_mesh_is_a_closed_sphere():
    res = (40, 48, 32)
    f = sphere_lattice(res)
    verts, tris = mc.marching_cubes(f, res, 0.0)
    assert check_closed_oriented(verts, tris) == 2
    # vertices sit on the sphere up to the interpolation error of a distance field, O(h^2 / r)
    r = np.linalg.norm(verts.astype(np.float64) - 0.5, axis=1)
    assert np.abs(r - 0.3).max() < 2e-3
    a, b, c = (verts[tris[:, k]].astype(np.float64) for k in range(3))
    area = 0.5 * np.linalg.norm(np.cross(b - a, c - a), axis=1).sum()
    vol = np.einsum("ij,ij->i", a - 0.5, np.cross(b - 0.5, c - 0.5)).sum() / 6.0
    assert abs(area - 4 * np.pi * 0.09) / (4 * np.pi * 0.09) < 0.01
    # triangle normals point to the inside (where density > thresh), like the classic table's: signed volume negative
    assert abs(-vol - 4 / 3 * np.pi * 0.027) / (4 / 3 * np.pi * 0.027) < 0.01
    n = mc.vertex_normals(verts, tris)
    # accumulate_1ring's cross product (pb - pa) x (pa - pc) is minus the triangle normal: it points outwards here
    cosang = np.einsum("ij,ij->i", n / np.linalg.norm(n, axis=1, keepdims=True), (verts - 0.5) / r[:, None])
    assert cosang.min() > 0.9


def test_vertex_formula_and_aabb_mapping():
    res = (16, 16, 16)
    f = np.full((16, 16, 16), -1.0, np.float32)
    f[5, 6, 7] = 3.0  # one inside point: an octahedron around lattice point (7, 6, 5)
    lo, hi = (-1.0, 0.0, 2.0), (1.0, 4.0, 3.0)
    verts, tris = mc.marching_cubes(f, res, 0.0, lo, hi)
    assert len(verts) == 6 and len(tris) == 8 and check_closed_oriented(verts, tris) == 2
    scale = (np.asarray(hi, np.float32) - np.asarray(lo, np.float32)) / 16
    # an edge that ends in the inside point has f0 = -1, f1 = 3: dt = (0 - f0) / (f1 - f0) = 0.25 from its first point;
    # an edge that starts there has f0 = 3, f1 = -1: dt = 0.75
    lattice = [(6.25, 6, 5), (7.75, 6, 5), (7, 5.25, 5), (7, 6.75, 5), (7, 6, 4.25), (7, 6, 5.75)]
    want = [np.array(p, np.float32) * scale + np.asarray(lo, np.float32) for p in lattice]
    got = {tuple(np.round(v, 5)) for v in verts}
    assert got == {tuple(np.round(v, 5)) for v in want}
    # numbering: by lattice point (x fastest), then direction: the z edge below the point comes first
    np.testing.assert_allclose(verts[0], want[4], rtol=0, atol=1e-6)


def test_empty_and_full_lattices():
    res = (8, 8, 8)
    for value in (-1.0, 1.0):
        v, t = mc.marching_cubes(np.full((8, 8, 8), value, np.float32), res, 0.0)
        assert len(v) == 0 and len(t) == 0
