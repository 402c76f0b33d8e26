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
