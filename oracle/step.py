"""CPU oracle of one whole training step (TEST INFRASTRUCTURE ONLY): the sequence of
Testbed::train_nerf_step + Trainer::optimizer_step (src/testbed_nerf.cu:3717-3987, 3498)
assembled from the oracle's pieces.  Used by tests, by ``__graft_entry__.smoke`` as the
checker and by ``bench.py`` as the timed CPU baseline."""
import numpy as np

from . import oracle as orc
from .field import Field


class StepState:
    def __init__(self, field: Field, master):
        self.field = field
        self.master = np.ascontiguousarray(master, np.float32).copy()
        n = self.master.size
        self.m1 = np.zeros(n, np.float32)
        self.m2 = np.zeros(n, np.float32)
        self.steps = np.zeros(n, np.uint32)
        self.n_rays_total = 0

    def params16(self):
        return orc.round_fp16(self.master)


def training_step(state: StepState, cameras, rgba, bitfield, n_rays, n_inference, seed, target_batch_size,
                  background=(1.0, 1.0, 1.0), ek_loss_weight=0.01, loss_scale=128.0, adam=None):
    """Returns dict(rays, samples, compacted, loss, grad)."""
    f = state.field
    p16 = state.params16()
    s = orc.generate_training_samples(n_rays, state.n_rays_total, seed, cameras, rgba, background, bitfield, n_inference)
    state.n_rays_total += n_rays
    k = s["ray_counter"]
    S = int(s["numsteps"][:k, 0].sum()) if k else 0
    T = target_batch_size
    if S == 0:
        return dict(rays=k, samples=s["sample_counter"], compacted=0, loss=0.0, grad=None)
    out, _ = f.forward(p16, s["coords"][:S])
    comp = orc.composite_loss(s["numsteps"][:k], orc.round_fp16(out.T.copy()), s["coords"][:S], s["rgb_target"][:k], T,
                              n_rays_norm=n_rays, loss_scale=loss_scale, ek_loss_weight=ek_loss_weight,
                              background=background)
    n_in = min(comp["counter"], T)
    dloss = orc.fill_rollover(orc.round_fp16(comp["dloss"]), n_in, rescale=True)
    coords_c = orc.fill_rollover(comp["coords"].copy(), n_in)
    _, ctx = f.forward(p16, coords_c)
    grad = f.backward(p16, ctx, orc.round_fp16(dloss).T.copy(), ek_batch_size=T)
    grad16 = orc.round_fp16(grad)
    kw = adam or {}
    orc.adam_step(state.master, grad16, state.m1, state.m2, state.steps, n_matrix_params=f.n_matrix_params,
                  loss_scale=loss_scale, **kw)
    return dict(rays=k, samples=s["sample_counter"], compacted=comp["counter"], loss=float(comp["loss"].sum()), grad=grad16)


def _rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _band(got, ref, rtol, what, scale=None, outlier_frac=0.0, atol=0.0):
    """|got - ref| <= rtol * (|ref| + scale) + atol, scale defaulting to the RMS of ref; outlier_frac of the entries may lie outside."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    if scale is None:
        scale = float(np.sqrt(np.mean(ref ** 2))) if ref.size else 0.0
    bad = np.abs(got - ref) > rtol * (np.abs(ref) + scale) + atol
    assert bad.sum() <= outlier_frac * bad.size, f"{what}: {int(bad.sum())} of {bad.size} outside rtol {rtol} (rel_l2 {_rel_l2(got, ref):.3g})"


def verify_step(field: Field, params16, cameras, rgba, bitfield, n_rays, n_rays_total, seed, n_inference, target_batch_size, counters,
                gpu, grads, background=(1.0, 1.0, 1.0), ek_loss_weight=0.01, loss_scale=128.0, rtol=2e-3, evaluated=None):
    """Checks one GPU training step stage by stage, every stage against the oracle run on the GPU's own input to that
    stage, so that a wiring error (a wrong batch size in the eikonal term, a mis-scaled roll-over, loss_scale / n_rays)
    shows at the stage where it happens and nothing is blurred by the one-sample differences that the 1e-4
    transmittance cut-off can cause between two compositors.
      counters  dict(rays, samples, compacted, loss) read from the trainer
      gpu       numpy arrays of the step's device buffers (Trainer.last_step): coords, numsteps, rgb_target,
                ray_indices, network_output, coords_compacted, dloss_doutput, source_index
      grads     the fp16 gradient vector the step left (as float32)
      evaluated marched samples the GPU evaluated the field on when it ran the forward pass in depth chunks (the others lie
                behind their rays' cuts and hold no output); None: all of them
    Returns a dict of the figures it checked."""
    f, T = field, target_batch_size
    # 1. sample generation: bit-exact
    s = orc.generate_training_samples(n_rays, n_rays_total, seed, cameras, rgba, background, bitfield, n_inference)
    k, S = s["ray_counter"], s["sample_counter"]
    assert (counters["rays"], counters["samples"]) == (k, S), (counters, k, S)
    S = int(s["numsteps"][:k, 0].sum())
    assert np.array_equal(gpu["coords"][:S].view(np.uint32), s["coords"][:S].view(np.uint32)), "sample coordinates differ"
    assert np.array_equal(gpu["rgb_target"][:k].view(np.uint32), s["rgb_target"][:k].view(np.uint32)), "ray targets differ"
    assert np.array_equal(gpu["ray_indices"][:k].astype(np.int64), s["ray_indices"][:k].astype(np.int64)), "ray order differs"
    # 2. field forward over every marched sample
    out_ref, _ = f.forward(params16, s["coords"][:S])
    out_gpu = gpu["network_output"][:S].astype(np.float32)
    if evaluated is not None:
        # what was not evaluated must lie behind the cut: the oracle's compositor is given its own values there, and stops
        # at another sample than the GPU's if the GPU evaluated too little
        skipped = np.ones(S, bool)
        skipped[np.asarray(evaluated, np.int64)] = False
        assert len(np.unique(evaluated)) == len(evaluated) and not skipped.all()
        out_gpu[skipped] = orc.round_fp16(out_ref.T[skipped])
    for name, rows in (("rgb", slice(0, 3)), ("sdf", slice(3, 4)), ("normal", slice(4, 7)), ("variance", slice(7, 8)), ("dir", slice(8, 11))):
        _band(out_gpu[:, rows].T, out_ref[rows], rtol, f"field output {name}", outlier_frac=2e-4)
    # 3. compositing, loss, gradients and compaction, on the GPU's own network output
    comp = orc.composite_loss(s["numsteps"][:k], out_gpu, s["coords"][:S], s["rgb_target"][:k], T, n_rays_norm=n_rays,
                              loss_scale=loss_scale, ek_loss_weight=ek_loss_weight, background=background)
    rn, gn = comp["numsteps"], gpu["numsteps"][:k].view(np.uint32)
    n_in = min(int(counters["compacted"]), T)
    same = rn[:, 0] == gn[:, 0]
    assert (~same).sum() <= max(1, k // 1000), f"{int((~same).sum())} rays end at another sample than the oracle's"
    if same.all():
        assert np.array_equal(rn, gn) and counters["compacted"] == comp["counter"]
        m = min(comp["counter"], T)
        assert np.array_equal(gpu["coords_compacted"][:m].view(np.uint32), comp["coords"][:m].view(np.uint32)), "compacted coordinates differ"
    rows_g, rows_r = [], []
    for i in np.nonzero(same)[0]:
        n, bg, br = int(rn[i, 0]), int(gn[i, 1]), int(rn[i, 1])
        if n == 0 or bg + n > n_in:  # the ray that the batch cuts short is compared below through its prefix
            n = max(0, min(n, n_in - bg))
        if n:
            rows_g.append(gpu["dloss_doutput"][bg:bg + n].astype(np.float32))
            rows_r.append(comp["dloss"][br:br + n])
            assert np.array_equal(gpu["source_index"][bg:bg + n].astype(np.int64), int(s["numsteps"][i, 1]) + np.arange(n)), "source index differs"
    G, R = np.concatenate(rows_g), np.concatenate(rows_r)
    for name, sl in (("rgb", slice(0, 3)), ("sdf", slice(3, 4)), ("eikonal", slice(4, 7)), ("variance", slice(7, 8)), ("normal", slice(8, 11))):
        # the gradients are stored as fp16 and, divided by thousands of rays, reach its subnormal range: one step of 2^-24 is allowed
        _band(G[:, sl], R[:, sl], 2 * rtol, f"dloss {name}", scale=float(np.abs(R[:, sl]).mean()), outlier_frac=1e-4, atol=6e-8)
    loss_ref = float(comp["loss"][same].sum())
    assert abs(counters["loss"] - float(comp["loss"].sum())) <= 2 * rtol * abs(loss_ref) + 1e-7 + float(np.abs(comp["loss"][~same]).sum()) * 2, (counters["loss"], loss_ref)
    # 4. roll-over to exactly T samples: wrapped coordinates, wrapped and rescaled gradients
    if 0 < n_in < T:
        idx = np.arange(n_in, T)
        assert np.array_equal(gpu["coords_compacted"][idx].view(np.uint32), gpu["coords_compacted"][idx % n_in].view(np.uint32)), "roll-over of the coordinates"
        want = gpu["dloss_doutput"][idx % n_in].astype(np.float32) * np.float32(n_in) / np.float32(T)
        # bit for bit: the copies are formed from the stored fp16 values with one fp32 product and one correctly rounded division
        assert np.array_equal(gpu["dloss_doutput"][idx].astype(np.float32), orc.round_fp16(want)), "roll-over of the gradients"
        assert np.array_equal(gpu["source_index"][idx], gpu["source_index"][idx % n_in]), "roll-over of the source index"
    # 5. backward of the GPU's own batch
    _, ctx = f.forward(params16, gpu["coords_compacted"])
    ref = f.backward(params16, ctx, gpu["dloss_doutput"].astype(np.float32).T.copy(), ek_batch_size=T)
    res = {}
    for name, a, b in (("sdf mlp", f.off_sdf, f.off_rgb), ("rgb mlp", f.off_rgb, f.off_grid), ("grid", f.off_grid, f.off_var)):
        r = _rel_l2(grads[a:b], ref[a:b])
        res[name] = r
        bound = 2 * rtol
        assert r <= bound, f"{name} gradient: rel_l2 {r:.3g} > {bound}"
    dv = abs(float(grads[f.off_var]) - float(ref[f.off_var]))
    res["variance"] = dv
    # one fp16 rounding of the sum, fp32 accumulation of the terms
    assert dv <= 2 * rtol * abs(float(ref[f.off_var])) + 1e-5 * float(np.abs(gpu["dloss_doutput"][:, 7].astype(np.float64)).sum()) + 1e-6, (grads[f.off_var], ref[f.off_var])
    res.update(rays=k, samples=S, compacted=int(counters["compacted"]), rays_off_by_one=int((~same).sum()))
    return res
