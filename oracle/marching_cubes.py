"""CPU oracle of the mesh extraction (TEST INFRASTRUCTURE ONLY): marching cubes over a density lattice as
marching_cubes_gpu does it (src/marching_cubes.cu:276-329 gen_vertices, :377-718 gen_faces, :794-822 driver) and the
area-weighted vertex normals of accumulate_1ring (:331-366).

Geometry conventions taken from the reference:
 * lattice value at (x, y, z) is density[x + y*rx + z*rx*ry]; a point is inside when density > thresh (:293)
 * one vertex per lattice edge whose end points differ in that test, at p0 + dt along the edge with
   dt = (thresh - f0) / (f1 - f0), then scaled by (aabb.max - aabb.min) / res and shifted by aabb.min (:281-282, 300-302)
 * cube corner bits: 1 (x,y,z), 2 (x+1,y,z), 4 (x+1,y+1,z), 8 (x,y+1,z), 16..128 the same at z+1 (:676-686)
 * cube edges 0..3 around the bottom face (x edge at y, y edge at x+1, x edge at y+1, y edge at x), 4..7 the same at
   z+1, 8..11 the z edges at corners 0..3 (:690-706)

What differs on purpose:
 * vertex and triangle ORDER: the reference hands out slots with atomicAdd (a race); here vertices are numbered by
   lattice point (x fastest), then edge direction x, y, z, and triangles by cube;
 * the case table is derived, not copied: every cube face is walked, the cut edges on it are joined into directed
   segments (an ambiguous face, with two diagonal inside corners, always separates the inside corners), the segments
   chain into closed loops and every loop is triangulated as a fan from its lowest edge.  Row 1 comes out as the
   classic (0, 8, 3).  A fixed rule per face makes neighbouring cubes agree on every shared face, so the surface is
   closed.  For all 256 cases the derived table has the same directed contour segments on every cube face, and the
   same number of triangles, as the table in the reference (tests/test_oracle_marching_cubes.py checks this against
   the reference's text when it is present): same surface, same orientation, same resolution of ambiguous faces.
   98 rows are identical triangle for triangle; the others cut the same polygons into triangles along other diagonals.
"""
import numpy as np

CORNERS = np.array([(0, 0, 0), (1, 0, 0), (1, 1, 0), (0, 1, 0), (0, 0, 1), (1, 0, 1), (1, 1, 1), (0, 1, 1)])
EDGES = [(0, 1), (1, 2), (2, 3), (3, 0), (4, 5), (5, 6), (6, 7), (7, 4), (0, 4), (1, 5), (2, 6), (3, 7)]
EDGE_OF = {frozenset(e): i for i, e in enumerate(EDGES)}


def cube_faces():
    """The 6 faces as corner cycles, counter-clockwise when seen from outside the cube."""
    faces = []
    for axis in range(3):
        for side in (0, 1):
            cs = [i for i in range(8) if CORNERS[i][axis] == side]
            centre = CORNERS[cs].mean(0)
            outward = np.zeros(3)
            outward[axis] = 1 if side else -1
            # order the four corners by angle around the outward normal
            u = np.roll(np.eye(3)[axis], 1)
            v = np.cross(outward, u)
            ang = [np.arctan2((CORNERS[c] - centre) @ v, (CORNERS[c] - centre) @ u) for c in cs]
            cyc = [c for _, c in sorted(zip(ang, cs))]
            n = np.cross(CORNERS[cyc[1]] - CORNERS[cyc[0]], CORNERS[cyc[2]] - CORNERS[cyc[1]])
            assert n @ outward > 0
            faces.append(cyc)
    return faces


FACES = cube_faces()


def face_segments(mask, separate_inside=True):
    """Directed segments (from_edge, to_edge) on every face of the cube with inside-corner bit mask ``mask``."""
    segs = []
    for cyc in FACES:
        inside = [(mask >> c) & 1 for c in cyc]
        if sum(inside) in (0, 4):
            continue
        ambiguous = inside in ([1, 0, 1, 0], [0, 1, 0, 1])
        # maximal runs of inside corners (or of outside corners on an ambiguous face resolved the other way)
        want = 1 if (separate_inside or not ambiguous) else 0
        for k in range(4):
            if inside[k] == want and inside[k - 1] != want:
                j = k
                while inside[(j + 1) % 4] == want:
                    j += 1
                before = EDGE_OF[frozenset((cyc[k - 1], cyc[k]))]
                after = EDGE_OF[frozenset((cyc[j % 4], cyc[(j + 1) % 4]))]
                # the surface normal points to the inside: the contour leaves through the edge after the inside run
                segs.append((after, before) if want == 1 else (before, after))
    return segs


def case_loops(mask):
    nxt = dict()
    for a, b in face_segments(mask):
        assert a not in nxt
        nxt[a] = b
    loops, seen = [], set()
    for e in sorted(nxt):
        if e in seen:
            continue
        loop = [e]
        seen.add(e)
        while nxt[loop[-1]] != e:
            loop.append(nxt[loop[-1]])
            seen.add(loop[-1])
        loops.append(loop)
    return loops


def build_triangle_table():
    """int8 [256][16]: up to 5 triangles as edge triples, terminated by -1."""
    table = np.full((256, 16), -1, np.int8)
    for mask in range(256):
        tris = []
        for loop in case_loops(mask):
            for k in range(1, len(loop) - 1):
                tris += [loop[0], loop[k], loop[k + 1]]
        assert len(tris) <= 15, (mask, tris)
        table[mask, :len(tris)] = tris
    return table


TRIANGLE_TABLE = build_triangle_table()


def marching_cubes(density, res, thresh, aabb_min=(0.0, 0.0, 0.0), aabb_max=(1.0, 1.0, 1.0)):
    """density: float32 [rz, ry, rx] (x fastest).  Returns (vertices float32 [V, 3], indices uint32 [T, 3])."""
    rx, ry, rz = res
    f = np.asarray(density, np.float32).reshape(rz, ry, rx)
    inside = f > np.float32(thresh)
    scale = (np.asarray(aabb_max, np.float32) - np.asarray(aabb_min, np.float32)) / np.asarray(res, np.float32)
    offset = np.asarray(aabb_min, np.float32)
    # cut flags per lattice point and direction
    cut = np.zeros((3, rz, ry, rx), bool)
    cut[0, :, :, :-1] = inside[:, :, :-1] != inside[:, :, 1:]
    cut[1, :, :-1, :] = inside[:, :-1, :] != inside[:, 1:, :]
    cut[2, :-1, :, :] = inside[:-1, :, :] != inside[1:, :, :]
    per_point = cut.sum(0).astype(np.int64).ravel()
    first = np.concatenate([[0], np.cumsum(per_point)[:-1]])  # first vertex of each lattice point
    vid = np.full((3, rz * ry * rx), -1, np.int64)
    rank = np.zeros(rz * ry * rx, np.int64)
    for a in range(3):
        c = cut[a].ravel()
        vid[a, c] = first[c] + rank[c]
        rank += c
    n_verts = int(per_point.sum())
    verts = np.zeros((n_verts, 3), np.float32)
    zz, yy, xx = np.meshgrid(np.arange(rz), np.arange(ry), np.arange(rx), indexing="ij")
    base = np.stack([xx, yy, zz], -1).astype(np.float32).reshape(-1, 3)
    fl = f.ravel()
    step = (1, rx, rx * ry)
    for a in range(3):
        sel = np.nonzero(cut[a].ravel())[0]
        f0, f1 = fl[sel], fl[sel + step[a]]
        dt = (np.float32(thresh) - f0) / (f1 - f0)
        p = base[sel].copy()
        p[:, a] = p[:, a] + dt
        verts[vid[a, sel]] = p * scale + offset
    # faces
    m = np.zeros((rz - 1, ry - 1, rx - 1), np.int64)
    for bit, (dx, dy, dz) in enumerate(CORNERS):
        m |= inside[dz:rz - 1 + dz, dy:ry - 1 + dy, dx:rx - 1 + dx].astype(np.int64) << bit
    cz, cy, cx = np.nonzero((m != 0) & (m != 255))
    idx = cx + cy * rx + cz * rx * ry
    masks = m[cz, cy, cx]
    # lattice point and direction that own each of the 12 cube edges
    own = [(0, 0), (1, 1), (rx, 0), (0, 1), (rx * ry, 0), (rx * ry + 1, 1), (rx * ry + rx, 0), (rx * ry, 1), (0, 2), (1, 2), (1 + rx, 2), (rx, 2)]
    tris = []
    for i, mask in zip(idx, masks):
        row = TRIANGLE_TABLE[mask]
        for k in range(0, 15, 3):
            if row[k] < 0:
                break
            tris.append([vid[own[e][1], i + own[e][0]] for e in row[k:k + 3]])
    indices = np.asarray(tris, np.int64).reshape(-1, 3)
    assert (indices >= 0).all()
    return verts, indices.astype(np.uint32)


def vertex_normals(verts, indices):
    """accumulate_1ring's normal part: per vertex, the sum of (pb - pa) x (pa - pc) over its triangles (not normalised)."""
    v = verts.astype(np.float32)
    pa, pb, pc = v[indices[:, 0]], v[indices[:, 1]], v[indices[:, 2]]
    n = np.cross(pb - pa, pa - pc).astype(np.float32)
    out = np.zeros((len(v), 3), np.float64)
    for k in range(3):
        np.add.at(out, indices[:, k], n)
    return out.astype(np.float32)
