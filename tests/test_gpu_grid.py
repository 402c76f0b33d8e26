"""GPU parity of the hash-grid kernels against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from gpu_util import RTOL, assert_close, dev, host, q16, rel_l2

pytestmark = pytest.mark.gpu

CFG = dict(n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447)


@pytest.fixture(scope="module")
def setup(oracle):
    from neus2_amd.tcnn_api import GridEncoding
    og = oracle.Grid(CFG["n_levels"], CFG["log2_hashmap_size"], CFG["base_resolution"], CFG["per_level_scale"])
    gg = GridEncoding(**CFG)
    assert gg.n_params() == og.n_params
    rng = np.random.default_rng(0)
    params = q16(rng.uniform(-1, 1, og.n_params))
    d_params = dev(params, torch.float16)
    d_grads = torch.zeros_like(d_params)
    gg.set_params(d_params, d_grads)
    return og, gg, params, d_params, d_grads


def test_config1_indices_bit_exact(setup):
    """The benchmark's plumbing configuration: 2^14 points U[0,1)^3, seed 0: every corner index of every level identical."""
    og, gg, *_ = setup
    xyz = np.random.default_rng(0).random((3, 1 << 14), dtype=np.float32)
    ref, _ = og.indices(xyz)
    got = host(gg.corner_indices(dev(xyz))).view(np.uint32)
    assert np.array_equal(got, ref)


def test_indices_bit_exact_edge_positions(setup):
    og, gg, *_ = setup
    edge = np.array([0.0, 1.0, np.nextafter(np.float32(1), np.float32(0)), 0.5, 1e-8, 0.25, 0.999999, 1.0 / 3], np.float32)
    xyz = np.stack(np.meshgrid(edge, edge, edge, indexing="ij")).reshape(3, -1).astype(np.float32)
    # plus vertices of several levels, where floor() sits on a knife edge
    extra = [((np.arange(40, dtype=np.float32) - 0.5) / s) for s in og.scale[[0, 3, 9, 15]]]
    e = np.clip(np.concatenate(extra), 0, 1).astype(np.float32)
    xyz = np.concatenate([xyz, np.stack([e, e[::-1], e])], axis=1)
    ref, _ = og.indices(xyz)
    got = host(gg.corner_indices(dev(xyz))).view(np.uint32)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("n", [1, 255, 256, 257, 5000])
def test_forward_values_and_ragged_sizes(setup, n):
    og, gg, params, *_ = setup
    xyz = np.random.default_rng(n).random((3, n), dtype=np.float32)
    ref, ref_j = og.forward(params, xyz, want_dy_dx=True)
    out, dy_dx = gg.forward(dev(xyz), prepare_input_gradients=True)
    assert_close(host(out), ref, what="grid forward")
    # dy_dx is fp32 on both sides; differences of fp16 table values times scale
    assert_close(host(dy_dx), ref_j, rtol=1e-4, what="dy_dx")
    out2, none = gg.forward(dev(xyz))
    # the two instantiations may round a tie differently: at most one fp16 ulp apart
    assert none is None
    assert_close(host(out2), host(out), rtol=1e-3, what="forward without dy_dx")


def test_forward_accepts_nerf_coordinate_rows(setup):
    """7 floats per point (xyz, dt, dir), the column-major batch the reference feeds (nerf.h:76-102)."""
    og, gg, params, *_ = setup
    n = 3000
    rng = np.random.default_rng(7)
    coords = rng.random((n, 7), dtype=np.float32)
    out_rows, _ = gg.forward(dev(coords))
    out_soa, _ = gg.forward(dev(np.ascontiguousarray(coords[:, :3].T)))
    assert torch.equal(out_rows, out_soa)


def test_forward_empty_batch(setup):
    _, gg, *_ = setup
    out, _ = gg.forward(torch.zeros((3, 0), dtype=torch.float32, device="cuda"))
    assert out.shape == (32, 0)


def test_forward_small_uniform_params_config1(setup, oracle):
    """Config 1's parameter distribution U(-1e-4, 1e-4), seed 0."""
    og, gg, _, d_params, d_grads = setup
    rng = np.random.default_rng(0)
    p = q16(rng.uniform(-1e-4, 1e-4, og.n_params))
    from neus2_amd.tcnn_api import GridEncoding
    g2 = GridEncoding(**CFG)
    dp = dev(p, torch.float16)
    g2.set_params(dp, None)
    xyz = rng.random((3, 1 << 14), dtype=np.float32)
    out, _ = g2.forward(dev(xyz))
    # fp16 subnormal spacing (6e-8) dominates at this magnitude: absolute floor of one subnormal ulp
    ref = og.forward(p, xyz)
    assert np.abs(host(out) - ref).max() <= 6e-8 + RTOL * np.abs(ref).max()


def test_backward_param_scatter_and_input_grad(setup):
    og, gg, params, d_params, d_grads = setup
    n = 1 << 14
    rng = np.random.default_rng(11)
    xyz = rng.random((3, n), dtype=np.float32)
    dy = q16(rng.standard_normal((32, n)))
    ref_grad, ref_dx = og.backward(params, xyz, dy)
    d_xyz = dev(xyz)
    _, ctx = gg.forward(d_xyz, prepare_input_gradients=True)
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_IGNORE, GRAD_OVERWRITE
    d_grads.fill_(7.0)  # Overwrite must discard this
    dx = gg.backward(ctx, d_xyz, dev(dy, torch.float16), want_input_grad=True, mode=GRAD_OVERWRITE)
    got = host(d_grads)
    assert_close(host(dx), ref_dx, rtol=1e-4, what="dL_dx")
    # fp16 atomics round after every addition: the error of an entry that received
    # k contributions grows like sqrt(k) half-ulps, so coarse levels get a wider band
    for l in range(16):
        a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
        k = 8.0 * n / max(1, int(og.entries[l]))
        tol = RTOL * max(1.0, np.sqrt(k))
        assert rel_l2(got[a:b], ref_grad[a:b]) < tol, (l, rel_l2(got[a:b], ref_grad[a:b]), tol)
    # Accumulate adds a second copy; Ignore leaves the buffer alone
    gg.backward(ctx, d_xyz, dev(dy, torch.float16), mode=GRAD_ACCUMULATE)
    got2 = host(d_grads)
    assert rel_l2(got2, 2 * ref_grad) < 2e-2
    before = d_grads.clone()
    dx2 = gg.backward(ctx, d_xyz, dev(dy, torch.float16), want_input_grad=True, mode=GRAD_IGNORE)
    assert torch.equal(before, d_grads) and torch.equal(dx, dx2)


def test_backward_backward_input(setup):
    og, gg, params, d_params, d_grads = setup
    n = 1 << 13
    rng = np.random.default_rng(13)
    xyz = rng.random((3, n), dtype=np.float32)
    g = q16(rng.standard_normal((32, n)) * 0.1)
    v = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    ref_grad, ref_out, ref_din = og.backward_backward_input(params, xyz, v, g)
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_IGNORE, GRAD_OVERWRITE
    d_xyz, d_v, d_g = dev(xyz), dev(v), dev(g, torch.float16)
    out, din = gg.backward_backward_input(d_xyz, d_v, d_g, want_dL_ddLdy=True, want_dL_dx=True, mode=GRAD_OVERWRITE)
    assert_close(host(out), ref_out, what="dL_ddLdy")
    assert_close(host(din), ref_din, rtol=1e-3, what="second-order dL_dx")
    got = host(d_grads)
    for l in range(16):
        a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
        k = 8.0 * n / max(1, int(og.entries[l]))
        tol = RTOL * max(1.0, np.sqrt(k))
        assert rel_l2(got[a:b], ref_grad[a:b]) < tol, (l, rel_l2(got[a:b], ref_grad[a:b]), tol)
    # the reference's call: Accumulate on top of the first-order gradients, outputs optional
    base = q16(rng.standard_normal(og.n_params) * 1e-3)
    d_grads.copy_(dev(base, torch.float16))
    out2, none = gg.backward_backward_input(d_xyz, d_v, d_g, want_dL_ddLdy=True, want_dL_dx=False, mode=GRAD_ACCUMULATE)
    # (a different kernel serves calls that also ask for the second-order dL_dx: same values up to fp16 rounding)
    assert none is None
    assert_close(host(out2), ref_out, what="dL_ddLdy without dL_dx")
    assert rel_l2(host(d_grads), base + ref_grad) < 1e-2
    before = d_grads.clone()
    gg.backward_backward_input(d_xyz, d_v, d_g, mode=GRAD_IGNORE)
    assert torch.equal(before, d_grads)


@pytest.mark.parametrize("cfg", [(6, 12, 4, 1.6), (5, 4, 2, 1.5), (8, 14, 4, 2.0), (14, 19, 16, 1.4472692012786865)])
def test_other_table_shapes(oracle, cfg):
    """Small tables exercise the true-modulo index paths; 14 levels is the reference's shipped config."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, GridEncoding
    og = oracle.Grid(*cfg)
    gg = GridEncoding(n_levels=cfg[0], log2_hashmap_size=cfg[1], base_resolution=cfg[2], per_level_scale=cfg[3])
    rng = np.random.default_rng(17)
    params = q16(rng.uniform(-1, 1, og.n_params))
    dp = dev(params, torch.float16)
    dg = torch.zeros_like(dp)
    gg.set_params(dp, dg)
    n = 2049
    xyz = rng.random((3, n), dtype=np.float32)
    ref_idx, _ = og.indices(xyz)
    assert np.array_equal(host(gg.corner_indices(dev(xyz))).view(np.uint32), ref_idx)
    out, ctx = gg.forward(dev(xyz), prepare_input_gradients=True)
    assert_close(host(out), og.forward(params, xyz), what="forward")
    dy = q16(rng.standard_normal((og.n_out, n)))
    ref_grad, ref_dx = og.backward(params, xyz, dy)
    dx = gg.backward(ctx, dev(xyz), dev(dy, torch.float16), want_input_grad=True, mode=GRAD_OVERWRITE)
    assert_close(host(dx), ref_dx, rtol=1e-4, what="dL_dx")
    assert rel_l2(host(dg), ref_grad) < 2e-2


@pytest.mark.parametrize("cfg", [(6, 12, 4, 1.6), (5, 4, 2, 1.5), (8, 14, 4, 2.0), (14, 19, 16, 1.4472692012786865),
                                 (16, 19, 32, 1.4472692012786865), (4, 21, 512, 1.9)])
def test_sorted_scatter_other_table_shapes(oracle, cfg):
    """The bucketed scatter on other tables: one bucket per level (2^12 entries), four buckets (2^14: no multiple of the
    8 XCDs), tiny tables with a true modulo, the 14-level config, hashed levels whose resolution exceeds the 12 index bits
    a pair record relies on (base 32: 5646 and 8170 cells, one record per corner there), and a table too large for the
    bucket plan (2^21 entries: falls back to the atomic scatter)."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, GridEncoding
    og = oracle.Grid(*cfg)
    gg = GridEncoding(n_levels=cfg[0], log2_hashmap_size=cfg[1], base_resolution=cfg[2], per_level_scale=cfg[3])
    rng = np.random.default_rng(23)
    params = q16(rng.uniform(-1, 1, og.n_params))
    dp = dev(params, torch.float16)
    dg = torch.zeros_like(dp)
    gg.set_params(dp, dg)
    n = 3 * 4096 + 13 * 8
    assert gg.reserve_scatter_workspace(1 << 14) == (cfg[1] <= 19)
    xyz = rng.random((3, n), dtype=np.float32)
    dy = q16(rng.standard_normal((og.n_out, n)))
    g2 = q16(rng.standard_normal((og.n_out, n)) * 0.1)
    v = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    ref1, _ = og.backward(params, xyz, dy, want_dx=False)
    ref, _, _ = og.backward_backward_input(params, xyz, v, g2, grad=ref1.copy(), want_dinput=False)
    dg.fill_(7.0)
    gg.backward_fused(dev(xyz), dev(dy, torch.float16), dev(v), dev(g2, torch.float16), want_dL_ddLdy=False, mode=GRAD_OVERWRITE)
    got = host(dg)
    for l in range(cfg[0]):
        a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
        k = 8.0 * n / max(1, int(og.entries[l]))
        tol = RTOL * (1.0 if cfg[1] <= 19 else max(1.0, np.sqrt(k)))  # the atomic fallback adds in fp16
        assert rel_l2(got[a:b], ref[a:b]) < tol, (l, rel_l2(got[a:b], ref[a:b]), tol)


def test_sorted_scatter_split_buckets(oracle):
    """A small table under a large batch: every level has fewer buckets than the batch needs workgroups, so buckets are
    split over several workgroups whose fp32 images a combine launch adds in a fixed order (both record kinds: the dense
    levels' single records and the hashed levels' pair records).  Against the oracle, accumulate mode included, and two
    runs give the same bits."""
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE, GridEncoding
    cfg = (6, 12, 4, 1.6)
    og = oracle.Grid(*cfg)
    gg = GridEncoding(n_levels=cfg[0], log2_hashmap_size=cfg[1], base_resolution=cfg[2], per_level_scale=cfg[3])
    rng = np.random.default_rng(29)
    params = q16(rng.uniform(-1, 1, og.n_params))
    dp = dev(params, torch.float16)
    dg = torch.zeros_like(dp)
    gg.set_params(dp, dg)
    n = 40 * 1024 + 77  # 8 n / 65536 = 5 workgroups per bucket
    assert gg.reserve_scatter_workspace(n)
    xyz = rng.random((3, n), dtype=np.float32)
    dy = q16(rng.standard_normal((og.n_out, n)) * 0.05)
    g2 = q16(rng.standard_normal((og.n_out, n)) * 0.01)
    v = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    ref1, _ = og.backward(params, xyz, dy, want_dx=False)
    ref, _, _ = og.backward_backward_input(params, xyz, v, g2, grad=ref1.copy(), want_dinput=False)
    d_xyz, d_dy, d_v, d_g2 = dev(xyz), dev(dy, torch.float16), dev(v), dev(g2, torch.float16)

    def check(got, want, what):
        for l in range(cfg[0]):
            a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
            assert rel_l2(got[a:b], want[a:b]) < RTOL, (what, l, rel_l2(got[a:b], want[a:b]))

    dg.fill_(7.0)
    gg.backward_fused(d_xyz, d_dy, d_v, d_g2, want_dL_ddLdy=False, mode=GRAD_OVERWRITE)
    first = dg.clone()
    check(host(dg), ref, "overwrite")
    gg.backward_fused(d_xyz, d_dy, d_v, d_g2, want_dL_ddLdy=False, mode=GRAD_ACCUMULATE)
    check(host(dg), 2 * ref, "accumulate")
    dg.fill_(-3.0)
    gg.backward_fused(d_xyz, d_dy, d_v, d_g2, want_dL_ddLdy=False, mode=GRAD_OVERWRITE)
    assert torch.equal(dg, first)


def test_errors_are_reported_not_launched():
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, GridEncoding, N2Error
    gg = GridEncoding(**CFG)
    x = torch.rand((3, 16), device="cuda")
    with pytest.raises(N2Error, match="set_params"):
        gg.forward(x)
    p = torch.zeros(gg.n_params(), dtype=torch.float16, device="cuda")
    gg.set_params(p, None)
    out, ctx = gg.forward(x, prepare_input_gradients=True)
    with pytest.raises(N2Error, match="gradient buffer"):
        gg.backward(ctx, x, torch.zeros((32, 16), dtype=torch.float16, device="cuda"), mode=GRAD_OVERWRITE)
    with pytest.raises(N2Error):
        gg.forward(x.double())


@pytest.mark.parametrize("n", [1 << 13, 1001])
def test_backward_fused_equals_first_plus_second_order(setup, n):
    """One scatter pass == backward(Overwrite) followed by backward_backward_input(Accumulate)."""
    og, gg, params, d_params, d_grads = setup
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE
    rng = np.random.default_rng(21)
    xyz = rng.random((3, n), dtype=np.float32)
    dy = q16(rng.standard_normal((32, n)))
    g2 = q16(rng.standard_normal((32, n)) * 0.1)
    v = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    ref1, _ = og.backward(params, xyz, dy, want_dx=False)
    ref, ref_out, _ = og.backward_backward_input(params, xyz, v, g2, grad=ref1.copy(), want_dinput=False)
    d_grads.fill_(3.0)
    out = gg.backward_fused(dev(xyz), dev(dy, torch.float16), dev(v), dev(g2, torch.float16), mode=GRAD_OVERWRITE)
    assert_close(host(out), ref_out, what="fused dL_ddLdy")
    got = host(d_grads)
    for l in range(16):
        a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
        k = 8.0 * n / max(1, int(og.entries[l]))
        tol = RTOL * max(1.0, np.sqrt(k))
        assert rel_l2(got[a:b], ref[a:b]) < tol, (l, rel_l2(got[a:b], ref[a:b]), tol)
    none = gg.backward_fused(dev(xyz), dev(dy, torch.float16), dev(v), dev(g2, torch.float16), want_dL_ddLdy=False,
                             mode=GRAD_ACCUMULATE)
    assert none is None and rel_l2(host(d_grads), 2 * ref) < 2e-2


@pytest.mark.parametrize("kind", ["uniform", "clustered", "rays"])
def test_sorted_scatter_path(oracle, kind):
    """With a scatter workspace, batches go through the run-length kernel (coarsest levels) and the
    LDS counting sort (the others): fp32 / exact accumulation, tighter agreement with the fp32 oracle than the
    atomic path, on uniform points, on points packed into a few cells (the contention case) and on points in ray
    order (consecutive samples share cells on the coarse levels, so runs are merged before they are written)."""
    from neus2_amd.tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE, GridEncoding
    og = oracle.Grid(CFG["n_levels"], CFG["log2_hashmap_size"], CFG["base_resolution"], CFG["per_level_scale"])
    gg = GridEncoding(**CFG)
    rng = np.random.default_rng(31)
    params = q16(rng.uniform(-1, 1, og.n_params))
    dp = dev(params, torch.float16)
    dg = torch.zeros_like(dp)
    gg.set_params(dp, dg)
    n = 3 * 4096 + 520  # not a multiple of the 1024-point tile
    assert gg.reserve_scatter_workspace(1 << 15)
    if kind == "uniform":
        xyz = rng.random((3, n), dtype=np.float32)
    elif kind == "clustered":
        xyz = (0.4 + 0.02 * rng.random((3, n))).astype(np.float32)
    else:
        per_ray = 97  # not a divisor of the 32-sample runs a lane walks
        n_rays = (n + per_ray - 1) // per_ray
        o = 0.3 + 0.4 * rng.random((n_rays, 1, 3))
        d = rng.standard_normal((n_rays, 1, 3))
        d /= np.linalg.norm(d, axis=-1, keepdims=True)
        k = np.arange(per_ray).reshape(1, per_ray, 1) - per_ray // 2
        xyz = np.clip(o + d * k * (np.sqrt(3.0) / 1024), 0, 1).reshape(-1, 3)[:n].T.astype(np.float32).copy()
    dy = q16(rng.standard_normal((32, n)))
    g2 = q16(rng.standard_normal((32, n)) * 0.1)
    v = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    ref1, _ = og.backward(params, xyz, dy, want_dx=False)
    ref, ref_out, _ = og.backward_backward_input(params, xyz, v, g2, grad=ref1.copy(), want_dinput=False)
    d_xyz, d_dy, d_v, d_g2 = dev(xyz), dev(dy, torch.float16), dev(v), dev(g2, torch.float16)

    def check(got, want, what):
        for l in range(16):
            a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
            # every contribution is rounded to fp16 once, sums are fp32, one final rounding
            assert rel_l2(got[a:b], want[a:b]) < RTOL, (what, l, rel_l2(got[a:b], want[a:b]))

    dg.fill_(9.0)
    gg.backward(None, d_xyz, d_dy, mode=GRAD_OVERWRITE)
    check(host(dg), ref1, "first order")
    dg.fill_(9.0)
    out = gg.backward_fused(d_xyz, d_dy, d_v, d_g2, mode=GRAD_OVERWRITE)
    assert_close(host(out), ref_out, what="fused dL_ddLdy")
    check(host(dg), ref, "fused")
    gg.backward_fused(d_xyz, d_dy, d_v, d_g2, want_dL_ddLdy=False, mode=GRAD_ACCUMULATE)
    check(host(dg), 2 * ref, "fused accumulate")
    # second-order only, accumulated on top
    _, ref2, _ = None, None, None
    base = host(dg).copy()
    ref_bbi, _, _ = og.backward_backward_input(params, xyz, v, g2, want_dinput=False)
    gg.backward_backward_input(d_xyz, d_v, d_g2, mode=GRAD_ACCUMULATE)
    check(host(dg), base + ref_bbi, "second order accumulate")
    # untouched entries stay exactly zero after Overwrite
    gg.backward(None, d_xyz, d_dy, mode=GRAD_OVERWRITE)
    got = host(dg)
    assert (got[ref1 == 0] == 0).all()


def test_sorted_scatter_pair_records_edge_cells(oracle):
    """Hashed levels sort one record per pair of x-neighbour corners; the second corner's place in the bucket is the
    first one's xor 2^(t+1) - 1, t = trailing one bits of the cell's x.  Cells whose x ends in 0 .. 11 one bits (the
    longest carries a 12-bit index can take), the first and the last cell of every level, against the oracle; and points
    outside the unit cube that carry a zero gradient change nothing."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, GridEncoding
    og = oracle.Grid(CFG["n_levels"], CFG["log2_hashmap_size"], CFG["base_resolution"], CFG["per_level_scale"])
    gg = GridEncoding(**CFG)
    rng = np.random.default_rng(41)
    params = q16(rng.uniform(-1, 1, og.n_params))
    dp = dev(params, torch.float16)
    dg = torch.zeros_like(dp)
    gg.set_params(dp, dg)
    n = 2 * 4096 + 264
    assert gg.reserve_scatter_workspace(1 << 14)
    xyz = rng.random((3, n), dtype=np.float32)
    # x coordinates in the middle of cells 2^k - 1 (k = 0 .. 11), 0 and res - 2 of the finest levels
    j = 0
    for level in (15, 14, 11, 8, 5):
        scale = float(og.scale[level])
        res = int(og.resolution[level])
        for cell in [0, res - 2] + [(1 << k) - 1 for k in range(13) if (1 << k) - 1 <= res - 2]:
            for rep in range(4):
                xyz[0, j] = np.float32((cell + 0.1 + 0.2 * rep) / scale)
                j += 1
    assert j < 4096
    dy = q16(rng.standard_normal((32, n)))
    stray = slice(n - 200, n)
    xyz[:, stray] = rng.uniform(-3, 4, (3, 200)).astype(np.float32)
    xyz[0, n - 200:n - 100] = rng.uniform(1.001, 40, 100).astype(np.float32)  # cells beyond the 12 index bits
    dy[:, stray] = 0
    inside = slice(0, n - 200)
    ref, _ = og.backward(params, np.ascontiguousarray(xyz[:, inside]), np.ascontiguousarray(dy[:, inside]), want_dx=False)
    dg.fill_(9.0)
    gg.backward(None, dev(xyz), dev(dy, torch.float16), mode=GRAD_OVERWRITE)
    got = host(dg)
    for l in range(16):
        a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
        assert rel_l2(got[a:b], ref[a:b]) < RTOL, (l, rel_l2(got[a:b], ref[a:b]))
    assert (got[ref == 0] == 0).all()


def _level_tols(og, n):
    return [RTOL * max(1.0, np.sqrt(8.0 * n / max(1, int(og.entries[l])))) for l in range(og.n_levels)]


@pytest.mark.parametrize("kind", ["global", "per_point", "progressive"])
@pytest.mark.parametrize("bucketed", [False, True])
def test_level_mask(setup, oracle, kind, bucketed):
    """Switched-off levels: zero features and dy_dx, no gradient, zero dL_ddLdy rows; everything else as unmasked.
    Expected values = the oracle on inputs whose switched-off (level, point) rows are zeroed."""
    from neus2_amd.tcnn_api import GRAD_OVERWRITE
    og, gg, params, d_params, d_grads = setup
    n = 3 * 4096 + 40 if bucketed else 3000
    rng = np.random.default_rng(77)
    xyz = rng.random((3, n), dtype=np.float32)
    dy = q16(rng.standard_normal((32, n)))
    g2 = q16(rng.standard_normal((32, n)) * 0.1)
    v = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    keep = None
    try:
        if bucketed:
            assert gg.reserve_scatter_workspace(1 << 14)
        if kind == "global":
            gg.set_max_level(0.5)
            assert gg.active_levels() == 9
            off = oracle.level_mask(16, n, 0.5)
        elif kind == "per_point":
            frac = (rng.random(n) * 2).astype(np.float32)  # the reference draws random_val * 2 per ray
            keep = dev(frac)
            gg.set_max_level_gpu(keep)
            off = oracle.level_mask(16, n, frac)
            assert 0.2 < off.mean() < 0.4
        else:
            gg.set_progressive(0.2, 0.02, 100)
            gg.set_training_step(1234)
            want = oracle.progressive_levels(16, 0.2, 0.02, 100, 1234)
            assert gg.active_levels() == want == 7
            off = oracle.level_mask(16, n, 1.0, valid_levels=want)
        off_rows = np.repeat(off, 2, axis=0)
        ref_y, ref_j = og.forward(params, xyz, want_dy_dx=True)
        ref_y[off_rows] = 0
        ref_j[off_rows] = 0
        d_xyz = dev(xyz)
        y, ctx = gg.forward(d_xyz, prepare_input_gradients=True)
        assert_close(host(y), ref_y, what="masked grid output")
        assert_close(host(ctx), ref_j, rtol=1e-4, what="masked dy_dx")
        assert (host(y)[off_rows] == 0).all() and (host(ctx)[off_rows] == 0).all()
        dy_m, g2_m = dy.copy(), g2.copy()
        dy_m[off_rows] = 0
        g2_m[off_rows] = 0
        ref1, ref_dx = og.backward(params, xyz, dy_m)
        ref, ref_out, _ = og.backward_backward_input(params, xyz, v, g2_m, grad=ref1.copy(), want_dinput=False)
        ref_out[off_rows] = 0
        d_grads.fill_(5.0)
        dx = gg.backward(ctx, d_xyz, dev(dy, torch.float16), want_input_grad=True, mode=GRAD_OVERWRITE)
        assert_close(host(dx), ref_dx, rtol=1e-4, what="masked dL_dx")
        got1 = host(d_grads)
        d_grads.fill_(5.0)
        out = gg.backward_fused(d_xyz, dev(dy, torch.float16), dev(v), dev(g2, torch.float16), mode=GRAD_OVERWRITE)
        got = host(d_grads)
        assert_close(host(out), ref_out, what="masked dL_ddLdy")
        assert (host(out)[off_rows] == 0).all()
        for l, tol in enumerate(_level_tols(og, n)):
            a, b = int(og.offset[l]) * 2, int(og.offset[l + 1]) * 2
            for g, r, what in ((got1, ref1, "first order"), (got, ref, "fused")):
                if np.abs(r[a:b]).max() == 0:
                    assert (g[a:b] == 0).all(), (what, l)  # a level nobody uses: Overwrite leaves zeros
                else:
                    assert rel_l2(g[a:b], r[a:b]) < tol, (what, l, rel_l2(g[a:b], r[a:b]), tol)
        # the second-order kernel that also returns dL_dx
        out2, din = gg.backward_backward_input(d_xyz, dev(v), dev(g2, torch.float16), want_dL_ddLdy=True, want_dL_dx=True,
                                               mode=GRAD_OVERWRITE)
        _, _, ref_din = og.backward_backward_input(params, xyz, v, g2_m)
        assert_close(host(out2), ref_out, what="masked dL_ddLdy (dL_dx variant)")
        assert_close(host(din), ref_din, rtol=1e-3, what="masked second-order dL_dx")
    finally:
        gg.set_max_level(1.0)
        gg.set_max_level_gpu(None)
        gg.set_progressive(1.0, 0.0, 0)
        if bucketed:
            from neus2_amd import capi
            import ctypes as C
            capi.lib().n2_grid_set_workspace(gg._h, None, C.c_uint64(0), C.c_uint32(0))
    assert gg.active_levels() == 16


def test_lattice_order_forward(setup):
    """The one-lane-per-point forward that n2_grid_set_point_order selects for lattice-ordered inference: same values as
    the oracle (and as the default kernel up to fp32 summation order), also with a level mask and ragged sizes."""
    og, gg, params, d_params, d_grads = setup
    r = 40
    z, y, x = np.meshgrid(np.arange(r), np.arange(r), np.arange(r), indexing="ij")
    xyz = (np.stack([x, y, z]).reshape(3, -1)[:, :r ** 3 - 13] / np.float32(r)).astype(np.float32)
    ref = og.forward(params, xyz)
    try:
        gg.set_point_order(True)
        y1, _ = gg.forward(dev(xyz))
        assert_close(host(y1), ref, what="lattice-order forward")
        gg.set_max_level(0.25)
        y2, _ = gg.forward(dev(xyz))
        ref2 = ref.copy()
        ref2[10:] = 0  # limit 4: levels 0..4 stay
        assert_close(host(y2), ref2, what="lattice-order forward, masked")
        assert (host(y2)[10:] == 0).all()
    finally:
        gg.set_point_order(False)
        gg.set_max_level(1.0)
    y0, _ = gg.forward(dev(xyz))
    assert rel_l2(host(y1), host(y0)) < 1e-3
