"""Pins the oracle's ray marcher / training-sample generator."""
import numpy as np
import pytest

from neus2_amd import scene


def oc_cams(oracle, cams):
    out = []
    for c in cams:
        po = int(c["pixel_offset"])
        out.append(oracle.Camera((oracle.C.c_float * 12)(*c["xform"]), (oracle.C.c_float * 2)(*c["focal"]),
                                 (oracle.C.c_float * 2)(*c["principal"]), (oracle.C.c_uint32 * 2)(*c["res"]),
                                 po & 0xFFFFFFFF, po >> 32))
    return out


@pytest.fixture(scope="module")
def small_scene(oracle):
    cams = scene.cameras_on_sphere(6, 64)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield()
    return cams, rgba, bits


def test_morton_closed_form(oracle):
    assert oracle.morton3d(1, 0, 0) == 1 and oracle.morton3d(0, 1, 0) == 2 and oracle.morton3d(0, 0, 1) == 4
    assert oracle.morton3d(3, 5, 7) == int("".join(f"{(7 >> b) & 1}{(5 >> b) & 1}{(3 >> b) & 1}" for b in (2, 1, 0)), 2)
    rng = np.random.default_rng(0)
    for x, y, z in rng.integers(0, 128, (200, 3)):
        m = oracle.morton3d(int(x), int(y), int(z))
        assert m < 128 ** 3 and oracle.morton3d_invert(m) == (x, y, z)
    xs = rng.integers(0, 128, (3, 500)).astype(np.uint32)
    got = scene.morton3d(xs[0], xs[1], xs[2])
    assert all(int(got[i]) == oracle.morton3d(int(xs[0, i]), int(xs[1, i]), int(xs[2, i])) for i in range(0, 500, 7))


def test_bitfield_band(oracle):
    bits = scene.sphere_bitfield(radius=0.3, band=0.03)
    assert bits.size == 128 ** 3 // 8 * 8
    n_occ = int(np.unpackbits(bits).sum())
    shell = 4 * np.pi * 0.3 ** 2 * 0.06 * 128 ** 3
    assert abs(n_occ - shell) / shell < 0.05
    # centre cell empty, a surface cell occupied
    def occ(p):
        i = np.clip((np.asarray(p) * 128).astype(int), 0, 127)
        m = oracle.morton3d(int(i[0]), int(i[1]), int(i[2]))
        return (bits[m // 8] >> (m % 8)) & 1
    assert occ((0.5, 0.5, 0.5)) == 0 and occ((0.8, 0.5, 0.5)) == 1 and occ((0.5, 0.5, 0.2)) == 1


def test_full_and_empty_bitfield(oracle, small_scene):
    cams, rgba, _ = small_scene
    oc = oc_cams(oracle, cams)
    n = 256
    empty = np.zeros(128 ** 3 // 8, np.uint8)
    r = oracle.generate_training_samples(n, 0, 1, oc, rgba, (0, 0, 0), empty, 1 << 16)
    assert r["ray_counter"] == 0 and r["sample_counter"] == 0
    full = np.full(128 ** 3 // 8, 255, np.uint8)
    r = oracle.generate_training_samples(n, 0, 1, oc, rgba, (0, 0, 0), full, 1 << 20)
    k = r["ray_counter"]
    assert k > 0.5 * n  # a 25-degree camera at distance 2 mostly sees the unit cube
    step = oracle.MIN_STEP
    for s in range(0, k, 17):
        cnt, base = r["numsteps"][s]
        c = r["coords"][base:base + cnt]
        d = c[0, 4:7] * 2 - 1
        assert abs(np.linalg.norm(d) - 1) < 1e-5
        assert ((c[:, :3] >= 0) & (c[:, :3] <= 1)).all() and (c[:, 3] == 0).all() and (c[:, 4:7] == c[0, 4:7]).all()
        if cnt > 1:
            gaps = np.linalg.norm(np.diff(c[:, :3], axis=0), axis=1)
            np.testing.assert_allclose(gaps, step, rtol=2e-3)
        assert cnt <= 1024
        # chord through the unit cube: at most sqrt(3)/step samples
        assert cnt <= int(np.sqrt(3) / step) + 2
    # ranges are handed out in ray order and tile [0, sample_counter)
    ns = r["numsteps"][:k]
    np.testing.assert_array_equal(ns[:, 1], np.concatenate([[0], np.cumsum(ns[:, 0])[:-1]]))
    assert r["sample_counter"] == ns[:, 0].sum()
    assert (np.diff(r["ray_indices"][:k].astype(np.int64)) > 0).all()


def test_dda_skip_equals_brute_force_stepping(oracle, small_scene):
    """Skipping empty voxels must visit exactly the occupied steps a plain t += dt march would."""
    cams, rgba, bits = small_scene
    oc = oc_cams(oracle, cams)
    n = 200
    r = oracle.generate_training_samples(n, 0, 7, oc, rgba, (0, 0, 0), bits, 1 << 18)
    full = oracle.generate_training_samples(n, 0, 7, oc, rgba, (0, 0, 0), np.full(128 ** 3 // 8, 255, np.uint8), 1 << 20)
    full_by_ray = {int(full["ray_indices"][s]): s for s in range(full["ray_counter"])}

    def occupied(p):
        q = ((p.astype(np.float32) - np.float32(0.5)) * np.float32(1) + np.float32(0.5)) * np.float32(128)
        i = np.clip(q.astype(np.int32), 0, 127)
        m = scene.morton3d(i[:, 0], i[:, 1], i[:, 2])
        return ((bits[m // 8] >> (m % 8).astype(np.uint8)) & 1).astype(bool)

    assert r["ray_counter"] > 20
    for s in range(r["ray_counter"]):
        i = int(r["ray_indices"][s])
        cnt, base = r["numsteps"][s]
        fs = full_by_ray[i]
        fc, fb = full["numsteps"][fs]
        all_pos = full["coords"][fb:fb + fc, :3]
        want = all_pos[occupied(all_pos)]
        got = r["coords"][base:base + cnt, :3]
        assert got.shape == want.shape, (i, got.shape, want.shape)
        np.testing.assert_array_equal(got, want)


def test_targets_and_budget(oracle, small_scene):
    cams, rgba, bits = small_scene
    oc = oc_cams(oracle, cams)
    n = 512
    r = oracle.generate_training_samples(n, 0, 3, oc, rgba, (0.2, 0.3, 0.4), bits, 1 << 18)
    k = r["ray_counter"]
    # rays that march through the shell either see the sphere (alpha 1: pixel colour) or graze it (background)
    t = r["rgb_target"][:k]
    assert ((t >= 0) & (t <= 1.0001)).all()
    is_bg = np.all(np.abs(t - np.array([0.2, 0.3, 0.4], np.float32)) < 1e-6, axis=1)
    assert 0 < is_bg.sum() < k
    # a small budget drops every ray from the first overflow on, but the counter keeps counting
    cap = int(r["sample_counter"]) // 3
    r2 = oracle.generate_training_samples(n, 0, 3, oc, rgba, (0.2, 0.3, 0.4), bits, cap)
    assert r2["sample_counter"] == r["sample_counter"] and r2["ray_counter"] < k
    k2 = r2["ray_counter"]
    np.testing.assert_array_equal(r2["numsteps"][:k2], r["numsteps"][:k2])
    assert (r2["numsteps"][:k2].sum(1) <= cap).all()
    # n_rays_total shifts the image assignment
    r3 = oracle.generate_training_samples(n, n // 2, 3, oc, rgba, (0.2, 0.3, 0.4), bits, 1 << 18)
    assert not np.array_equal(r3["numsteps"], r["numsteps"])
