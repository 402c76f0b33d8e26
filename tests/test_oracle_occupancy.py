"""Pins the oracle's occupancy-grid update (src/testbed_nerf.cu:630-786, 3286-3391) and its PCG32."""
import numpy as np
import pytest

from neus2_amd import scene
from neus2_amd.training import density_grid_update_plan

CELLS = 128 ** 3


def test_pcg32_published_vectors(oracle):
    # first outputs of the PCG32 reference generator seeded with (42, 54), as printed by the pcg32 demo program
    r = oracle.Pcg32(42, 54)
    assert [int(x) for x in r.next_uints(6)] == [0xa15c02b7, 0x7b47f409, 0xba1d3330, 0x83d2f293, 0xbfa4784b, 0xcbed606e]


def test_pcg32_advance_equals_draws(oracle):
    for delta in (0, 1, 2, 7, 4 * 12345, 1 << 20):
        a, b = oracle.Pcg32(1337), oracle.Pcg32(1337)
        a.next_uints(delta) if delta else None
        b.advance(delta)
        assert int(a.s[0]) == int(b.s[0])
        assert np.array_equal(a.next_uints(4), b.next_uints(4))
    # the skip used between launches: 2^32 is two jumps of 2^31
    a, b = oracle.Pcg32(5), oracle.Pcg32(5)
    a.advance(1 << 31)
    a.advance(1 << 31)
    b.advance(1 << 32)
    assert int(a.s[0]) == int(b.s[0])


def test_pcg32_float_is_mantissa_trick(oracle):
    a, b = oracle.Pcg32(9), oracle.Pcg32(9)
    u = a.next_uints(1000)
    f = b.next_floats(1000)
    want = ((u >> 9) | np.uint32(0x3f800000)).view(np.float32) - np.float32(1.0)
    assert np.array_equal(f, want) and f.min() >= 0.0 and f.max() < 1.0


def morton_invert_np(m):
    def compact(x):
        x = x & 0x49249249
        x = (x | (x >> 2)) & 0xc30c30c3
        x = (x | (x >> 4)) & 0x0f00f00f
        x = (x | (x >> 8)) & 0xff0000ff
        x = (x | (x >> 16)) & 0x0000ffff
        return x
    m = m.astype(np.uint64)
    return np.stack([compact(m), compact(m >> 1), compact(m >> 2)], -1).astype(np.int64)


def test_uniform_samples_cover_every_cell_once(oracle):
    grid = np.zeros(CELLS, np.float32)
    for step in (0, 3):
        pos, idx = oracle.generate_grid_samples(CELLS, oracle.Pcg32(1337), step, grid, 1, -0.01)
        # (i + step * n) * odd + c modulo a power of two is a bijection of the cells
        assert np.array_equal(np.sort(idx), np.arange(CELLS, dtype=np.uint32))
        i = np.arange(CELLS, dtype=np.uint64)
        want = ((i + step * CELLS) * 56924617 + 96925573) % (1 << 32) % CELLS
        assert np.array_equal(idx.astype(np.uint64), want)
        # every position lies inside its own cell (morton order); c + u may round up to the cell's far face
        cell = morton_invert_np(idx)
        off = pos.astype(np.float64) * 128 - cell
        assert off.min() >= 0.0 and off.max() <= 1.0
        assert (np.floor(pos.astype(np.float64) * 128).astype(np.int64) != cell).mean() < 1e-5


def test_sample_positions_use_draws_1_to_3(oracle):
    grid = np.zeros(CELLS, np.float32)
    n = 1000
    pos, idx = oracle.generate_grid_samples(n, oracle.Pcg32(77), 0, grid, 1, -0.01)
    cell = morton_invert_np(idx).astype(np.float32)
    for i in (0, 1, 17, 999):
        u = oracle.Pcg32(77).next_floats(4, skip=4 * i)  # draw 0 picks the cascade
        want = (cell[i] + u[1:4]) / np.float32(128) - np.float32(0.5)
        want = want * np.float32(1.0) + np.float32(0.5)
        assert np.array_equal(pos[i], want.astype(np.float32))


def test_cascades_scale_positions(oracle):
    nc = 3
    grid = np.zeros(nc * CELLS, np.float32)
    n = 4096
    pos, idx = oracle.generate_grid_samples(n, oracle.Pcg32(3), 1, grid, nc, -0.01)
    level = idx // CELLS
    u0 = np.array([oracle.Pcg32(3).next_floats(1, skip=4 * i)[0] for i in range(0, n, 64)])
    assert np.array_equal(level[::64], (u0 * nc).astype(np.uint32) % nc)
    assert set(np.unique(level)) == {0, 1, 2}
    cell = morton_invert_np(idx % CELLS)
    # undo the cascade's scaling about the cube centre: the point falls into its cell of the unit grid
    unit = (pos.astype(np.float64) - 0.5) / (2.0 ** level)[:, None] + 0.5
    assert np.abs(unit * 128 - cell - 0.5).max() <= 0.5 + 1e-4


def test_nonuniform_samples_prefer_occupied_cells(oracle):
    rng = np.random.default_rng(0)
    grid = np.where(rng.random(CELLS) < 0.3, 1.0, 0.0).astype(np.float32)
    n = 20000
    _, idx = oracle.generate_grid_samples(n, oracle.Pcg32(1), 2, grid, 1, 0.1)
    i = np.arange(n, dtype=np.uint64)
    want = np.zeros(n, np.uint64)
    done = np.zeros(n, bool)
    for j in range(10):
        cand = ((i + 2 * n) * 56924617 + j * 19349663 + 96925573) % (1 << 32) % CELLS
        take = ~done
        want[take] = cand[take]
        done |= grid[cand] > 0.1
    assert np.array_equal(idx.astype(np.uint64), want)
    # ten tries at 30% occupancy: all but ~0.7^10 of the samples land in occupied cells
    assert (grid[idx] > 0.1).mean() > 0.95


def test_splat_and_decayed_maximum(oracle):
    rng = np.random.default_rng(1)
    n_cells = 4096
    idx = rng.integers(0, n_cells, 20000).astype(np.uint32)
    dens = rng.random(20000).astype(np.float32) * 50
    tmp = np.zeros(n_cells, np.float32)
    oracle.splat_grid_max(idx, dens, tmp)
    want = np.zeros(n_cells, np.float32)
    np.maximum.at(want, idx, dens)
    assert np.array_equal(tmp, want)
    grid = (rng.random(n_cells).astype(np.float32) * 40 - 5).astype(np.float32)  # some cells negative
    before = grid.copy()
    oracle.ema_grid(grid, tmp, 0.95)
    want = np.where(before < 0, before, np.maximum(before * np.float32(0.95), tmp))
    assert np.array_equal(grid, want)


def bitfield_cells(bits_level):
    """128^3 booleans indexed [x, y, z] from one level of the morton bitfield."""
    flat = np.unpackbits(bits_level, bitorder="little").astype(bool)
    c = morton_invert_np(np.arange(CELLS, dtype=np.uint64))
    vol = np.zeros((128, 128, 128), bool)
    vol[c[:, 0], c[:, 1], c[:, 2]] = flat
    return vol


def test_bitfield_threshold_and_mip_pooling(oracle):
    rng = np.random.default_rng(2)
    grid = np.zeros(CELLS, np.float32)
    hot = rng.integers(0, CELLS, 3000)
    grid[hot] = rng.random(3000).astype(np.float32) * 2
    mean = oracle.grid_mean(grid)
    assert abs(mean - np.maximum(grid, 0).astype(np.float64).mean()) < 1e-9 + 1e-6 * mean
    bits = oracle.grid_to_bitfield(grid, 1, mean)
    assert bits.size == 8 * CELLS // 8
    thresh = min(0.1, mean)
    lvl0 = bits[:CELLS // 8]
    assert np.array_equal(np.unpackbits(lvl0, bitorder="little").astype(bool), grid > np.float32(thresh))
    prev = bitfield_cells(lvl0)
    for level in range(1, 8):
        cur = bitfield_cells(bits[level * CELLS // 8:(level + 1) * CELLS // 8])
        # a cell of the next level covers 2^3 cells of the previous one and sits in the central 64^3 block
        pooled = prev.reshape(64, 2, 64, 2, 64, 2).any(axis=(1, 3, 5))
        want = np.zeros((128, 128, 128), bool)
        want[32:96, 32:96, 32:96] = pooled
        assert np.array_equal(cur, want), level
        prev = cur
    # with two cascades the second level also keeps its own cells
    grid2 = np.concatenate([grid, np.zeros(CELLS, np.float32)])
    grid2[CELLS + 5] = 1.0
    bits2 = oracle.grid_to_bitfield(grid2, 2, mean)
    lvl1 = bitfield_cells(bits2[CELLS // 8:2 * CELLS // 8])
    c5 = morton_invert_np(np.array([5], np.uint64))[0]
    assert lvl1[c5[0], c5[1], c5[2]] and lvl1[32:96, 32:96, 32:96].sum() >= 1


def test_analytic_density_reproduces_the_sphere_shell(oracle):
    """An update driven by an analytic density (large inside a shell around the sphere) yields the bitfield the
    benchmark scene is built with."""
    occ = oracle.OccupancyGrid(1, seed=1337)

    def density(xyz):
        d = np.abs(np.linalg.norm(xyz - 0.5, axis=0) - 0.3)
        return np.where(d <= 0.03, 1.0, 0.0).astype(np.float32)

    occ.update(density, 0.95, CELLS, 0)
    shell = np.unpackbits(scene.sphere_bitfield(radius=0.3, band=0.03)[:CELLS // 8], bitorder="little").astype(bool)
    got = np.unpackbits(occ.bitfield[:CELLS // 8], bitorder="little").astype(bool)
    # the update samples a random point per cell, the scene helper tests cell centres: they differ only on the rim
    assert (got != shell).mean() < 0.02 and abs(int(got.sum()) - int(shell.sum())) < 0.1 * shell.sum()
    assert occ.ema_step == 1 and 0 < occ.mean < 0.1


def test_update_cadence():
    # every step for the first 32, then every step // 16 steps up to every 16th; full coverage before step 256
    assert all(density_grid_update_plan(s) == (CELLS, 0) for s in range(32))
    assert density_grid_update_plan(32) == (CELLS, 0) and density_grid_update_plan(33) is None
    assert density_grid_update_plan(48) == (CELLS, 0) and density_grid_update_plan(50) is None and density_grid_update_plan(51) == (CELLS, 0)
    assert density_grid_update_plan(256) == (CELLS // 4, CELLS // 4) and density_grid_update_plan(257) is None
    assert density_grid_update_plan(272, n_cascades=2) == (CELLS // 2, CELLS // 2)
    assert sum(density_grid_update_plan(s) is not None for s in range(1024, 2048)) == 64
