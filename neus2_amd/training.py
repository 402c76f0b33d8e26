"""Host side of the training loop: the trainer object over the C ABI, parameter
initialisation and the ray-count feedback of the reference's train_nerf
(src/testbed_nerf.cu:3393-3498).  torch supplies device memory and the stream."""
import ctypes as C
import math

import numpy as np
import torch

from . import capi
from .capi import N2Error, check, ptr

BATCH_SIZE_GRANULARITY = 128  # tcnn::batch_size_granularity, src/testbed_nerf.cu:3429, 3768


def next_multiple(x, m):
    return (int(x) + m - 1) // m * m


def default_config(target_batch_size=1 << 18, max_rays_per_batch=1 << 16, max_samples=None, n_levels=16,
                   log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447, ek_loss_weight=0.01,
                   background=(1.0, 1.0, 1.0), learning_rate=1e-3, prefetch_samples=True, ema_decay=0.0,
                   recompute_training_forward=False):
    """configs/nerf/base.json, with the level count and growth factor of the benchmark configurations (16 levels, 1.447)."""
    if max_samples is None:
        max_samples = 16 * target_batch_size  # src/testbed_nerf.cu:3719
    cfg = capi.TrainerConfig()
    cfg.field = capi.FieldConfig(n_levels, 2, log2_hashmap_size, base_resolution, per_level_scale, 1, 2, -0.1)
    cfg.adam = capi.AdamConfig(learning_rate, 0.9, 0.99, 1e-15, 1e-6)
    cfg.composite = capi.CompositeConfig(128.0, ek_loss_weight, 1.0, (C.c_float * 3)(*background), 1)
    cfg.target_batch_size = target_batch_size
    cfg.max_rays_per_batch = max_rays_per_batch
    cfg.max_samples = max_samples
    cfg.loss_scale = 128.0
    cfg.prefetch_samples = 1 if prefetch_samples else 0
    cfg.ema_decay = ema_decay  # configs/nerf/base.json:5-7 wraps Adam in Ema(0.95); 0 leaves plain Adam
    # False: the compacted batch re-uses the activations of the step's first field evaluation (bit-identical gradients)
    cfg.recompute_training_forward = 1 if recompute_training_forward else 0
    return cfg


class ExponentialDecay:
    """tcnn's ExponentialDecay wrapper with the settings of configs/nerf/base.json:8-12: after nested step t, the
    learning rate is multiplied by decay_base whenever t >= decay_start and (t - decay_start) % decay_interval == 0."""

    def __init__(self, base_learning_rate=1e-3, decay_start=20000, decay_interval=10000, decay_base=0.33):
        self.learning_rate = float(np.float32(base_learning_rate))
        self.decay_start, self.decay_interval, self.decay_base = decay_start, decay_interval, decay_base

    def after_step(self, steps_done):
        """Returns the learning rate of the next step; ``steps_done`` counts the nested steps including the last one."""
        if steps_done >= self.decay_start and (steps_done - self.decay_start) % self.decay_interval == 0:
            self.learning_rate = float(np.float32(self.learning_rate) * np.float32(self.decay_base))
        return self.learning_rate


def initial_parameters(offsets, sdf_in_width, seed=1337, sdf_mlp_weights=None):
    """NerfNetwork::initialize_params (nerf_network.h:805-876): Xavier-uniform MLPs, the SDF MLP overwritten with
    the geometric-init weights when given (utils/mlp_weights*.txt), grid U(-1e-4, 1e-4), variance 0.3.
    The reference draws from tcnn's pcg32, which is not reproducible here: numpy's generator stands in."""
    off_sdf, off_rgb, off_grid, off_var, n = offsets
    rng = np.random.default_rng(seed)
    p = np.zeros(n, np.float32)

    def xavier(rows, cols):
        s = math.sqrt(6.0 / (rows + cols))
        return rng.uniform(-s, s, rows * cols).astype(np.float32)

    p[off_sdf:off_rgb] = np.concatenate([xavier(64, sdf_in_width), xavier(16, 64)])
    if sdf_mlp_weights is not None:
        w = np.asarray(sdf_mlp_weights, np.float32)
        if w.size != off_rgb - off_sdf:
            raise N2Error(f"SDF MLP weight file has {w.size} values, the network needs {off_rgb - off_sdf}")
        p[off_sdf:off_rgb] = w
    p[off_rgb:off_grid] = np.concatenate([xavier(64, 48), xavier(64, 64), xavier(16, 64)])
    p[off_grid:off_var] = rng.uniform(-1e-4, 1e-4, off_var - off_grid).astype(np.float32)
    p[off_var:] = 0.3
    return p


class RayBudget:
    """Feedback that keeps the compacted batch near the target (src/testbed_nerf.cu:3406-3429, 3751-3756):
    after reading the counters, rays_per_batch is rescaled by target / measured compacted samples, and the
    next steps' inference window is the measured number of marched samples rounded up to 128."""

    def __init__(self, target_batch_size, max_rays, max_samples, rays_per_batch=1 << 12):
        self.target, self.max_rays, self.max_samples = target_batch_size, max_rays, max_samples
        self.rays_per_batch = min(rays_per_batch, max_rays)
        self.measured_before_compaction = 0
        self.measured = 0  # counters_rgb.measured_batch_size: samples the rays kept after compaction

    def n_inference(self):
        if self.measured_before_compaction == 0:
            return self.max_samples
        return next_multiple(min(self.measured_before_compaction, self.max_samples), BATCH_SIZE_GRANULARITY)

    def update(self, rays, samples, compacted):
        if compacted == 0 or samples == 0:
            return False  # the reference warns and stops training (src/testbed_nerf.cu:3536-3542)
        self.measured_before_compaction = min(int(samples), self.max_samples)
        self.measured = int(compacted)
        r = next_multiple(self.rays_per_batch * self.target / compacted, BATCH_SIZE_GRANULARITY)
        self.rays_per_batch = int(min(max(r, BATCH_SIZE_GRANULARITY), self.max_rays))
        return True


GRID_CELLS = 128 ** 3  # NERF_GRIDSIZE()^3, nerf.h:24-26


def density_grid_update_plan(training_step, n_cascades=1):
    """Which occupancy update Testbed::train runs before step ``training_step`` (src/testbed.cu:2658-2674 and
    training_prep_nerf, src/testbed_nerf.cu:3989-4002): None when the step is skipped, else
    (n_uniform, n_nonuniform).  The update runs every clamp(step / 16, 1, 16) steps; the first 256 steps
    sample every cell once, later ones a quarter of the cells uniformly and a quarter among occupied cells."""
    skip = min(max(training_step // 16, 1), 16)
    if training_step % skip != 0:
        return None
    n = GRID_CELLS * n_cascades
    return (n, 0) if training_step < 256 else (n // 4, n // 4)


class OccupancyGrid:
    """The density grid and its bitfield (Testbed::Nerf::density_grid / density_grid_bitfield), updated through
    the C ABI from a field's density."""

    def __init__(self, n_cascades=1, seed=1337, max_chunk=1 << 21, device="cuda"):
        L = capi.lib()
        self._h = C.c_void_p()
        check(L.n2_occupancy_create(C.c_uint32(n_cascades), C.c_uint64(seed), C.byref(self._h)), "n2_occupancy_create")
        self.n_cascades = n_cascades
        self.max_samples = GRID_CELLS * n_cascades
        nbytes = int(L.n2_occupancy_workspace_bytes(self._h, C.c_uint32(self.max_samples), C.c_uint32(max_chunk)))
        if nbytes == 0:
            raise N2Error("n2_occupancy_workspace_bytes: " + L.n2_last_error().decode())
        self._ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        check(L.n2_occupancy_set_workspace(self._h, ptr(self._ws), C.c_uint64(nbytes), C.c_uint32(self.max_samples),
                                           C.c_uint32(max_chunk)), "n2_occupancy_set_workspace")
        self.reset()

    def __del__(self):
        try:
            if getattr(self, "_h", None) is not None and self._h.value:
                capi.lib().n2_occupancy_destroy(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass

    @staticmethod
    def _stream():
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def reset(self):
        check(capi.lib().n2_occupancy_reset(self._h, self._stream()), "n2_occupancy_reset")

    def update(self, field_handle, n_uniform, n_nonuniform, decay=0.95):
        """decay: Testbed::Nerf::Training::density_grid_decay (testbed.h:635)."""
        check(capi.lib().n2_occupancy_update(self._h, field_handle, self._stream(), C.c_float(decay), C.c_uint32(n_uniform),
                                             C.c_uint32(n_nonuniform)), "n2_occupancy_update")

    def update_bitfield(self):
        check(capi.lib().n2_occupancy_update_bitfield(self._h, self._stream()), "n2_occupancy_update_bitfield")

    def view(self):
        v = capi.OccupancyBuffers()
        check(capi.lib().n2_occupancy_view(self._h, C.byref(v)), "n2_occupancy_view")
        return v

    def _tensor(self, address, nbytes, dtype):
        off = address - self._ws.data_ptr()
        return self._ws[off:off + nbytes].view(dtype)

    @property
    def density_grid(self):
        return self._tensor(self.view().density_grid, 4 * GRID_CELLS * self.n_cascades, torch.float32)

    @property
    def density_grid_tmp(self):
        return self._tensor(self.view().density_grid_tmp, 4 * GRID_CELLS * self.n_cascades, torch.float32)

    @property
    def bitfield(self):
        """uint8 [8 * 128^3 / 8]; the first 128^3 / 8 bytes are what the sample generator reads."""
        return self._tensor(self.view().bitfield, GRID_CELLS, torch.uint8)

    @property
    def mean(self):
        return self._tensor(self.view().mean, 4, torch.float32)

    def last_samples(self):
        """Positions [n, 3] and cells [n] of the last update's samples, in the reference's order (the uniform group, then
        the others; the library keeps a group of 2^k samples in the order that walks the cells in sequence)."""
        v = self.view()
        pos = self._tensor(v.positions, 12 * v.n_samples, torch.float32).view(-1, 3)
        idx = self._tensor(v.indices, 4 * v.n_samples, torch.int32)
        slot = torch.arange(v.n_samples, dtype=torch.int64, device=pos.device)
        for first, n in ((0, v.n_uniform), (v.n_uniform, v.n_samples - v.n_uniform)):
            if n >= 2 and n & (n - 1) == 0:  # sample i sits in slot i * 56924617 mod n of its group
                i = torch.arange(n, dtype=torch.int64, device=pos.device)
                slot[first:first + n] = first + (i * 56924617) % n
        return pos[slot], idx[slot]


class Trainer:
    def __init__(self, cfg=None, device="cuda"):
        self.cfg = cfg if cfg is not None else default_config()
        L = capi.lib()
        nbytes = int(L.n2_trainer_workspace_bytes(C.byref(self.cfg)))
        if nbytes == 0:
            raise N2Error("invalid trainer configuration: " + L.n2_last_error().decode())
        self.workspace_bytes = nbytes
        self._ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        self._h = C.c_void_p()
        check(L.n2_trainer_create(C.byref(self.cfg), ptr(self._ws), C.c_uint64(nbytes), C.byref(self._h)), "n2_trainer_create")
        m, p, g, n = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_uint32()
        check(L.n2_trainer_buffers(self._h, C.byref(m), C.byref(p), C.byref(g), C.byref(n)), "n2_trainer_buffers")
        self.n_params = int(n.value)
        base = self._ws.data_ptr()
        self.master = self._ws[m.value - base:m.value - base + 4 * self.n_params].view(torch.float32)
        self.params = self._ws[p.value - base:p.value - base + 2 * self.n_params].view(torch.float16)
        self.grads = self._ws[g.value - base:g.value - base + 2 * self.n_params].view(torch.float16)
        self._field = C.c_void_p(L.n2_trainer_field(self._h))
        o = (C.c_uint32 * 5)()
        check(L.n2_field_param_offsets(self._field, o), "n2_field_param_offsets")
        self.offsets = list(o)
        self.sdf_in_width = (3 + 2 * self.cfg.field.n_levels + 15) // 16 * 16
        self._scene = None
        self.budget = RayBudget(self.cfg.target_batch_size, self.cfg.max_rays_per_batch, self.cfg.max_samples)
        self.step_index = 0
        self.lr_schedule = None  # an ExponentialDecay, when the optimizer configuration nests one
        # update_budget switches the forward pass in depth chunks on and off by the measured ratio of marched to kept samples
        self.auto_depth_chunks = True
        self.depth_chunks = (0, 0)

    def __del__(self):
        try:
            if getattr(self, "_h", None) is not None and self._h.value:
                capi.lib().n2_trainer_destroy(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass

    def _stream(self):
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def encoding(self):
        """The field's grid encoding (m_nerf_network->encoding(), src/testbed.cu:2643-2646): set_progressive /
        set_max_level live there; every step tells it the number of steps taken so far."""
        from .tcnn_api import GridEncoding
        return GridEncoding._borrowed(capi.lib().n2_field_encoding(self._field), self)

    def set_depth_chunks(self, chunk_size, n_rounds):
        """n2_trainer_set_depth_chunks: the field over the marched samples in rounds of ``chunk_size`` samples per ray, rays
        past the compositor's cut dropping out between rounds (n_rounds < 2: off).  Results are bit-identical either way."""
        check(capi.lib().n2_trainer_set_depth_chunks(self._h, C.c_uint32(chunk_size), C.c_uint32(n_rounds)), "n2_trainer_set_depth_chunks")
        self.depth_chunks = (chunk_size, n_rounds) if n_rounds >= 2 else (0, 0)

    def set_parameters(self, master_np):
        self.master.copy_(torch.from_numpy(np.ascontiguousarray(master_np, np.float32)).to(self.master.device))
        check(capi.lib().n2_trainer_sync_params(self._h, self._stream()), "n2_trainer_sync_params")

    def initialize_params(self, seed=1337, sdf_mlp_weights=None):
        self.set_parameters(initial_parameters(self.offsets, self.sdf_in_width, seed, sdf_mlp_weights))

    def set_scene(self, cameras, n_images, rgba, bitfield):
        """cameras: device byte tensor (tcnn_api.pack_cameras); rgba fp32 [pixels, 4]; bitfield uint8."""
        self._scene = (cameras, rgba, bitfield)  # keep alive
        self._n_images = n_images
        check(capi.lib().n2_trainer_set_scene(self._h, ptr(cameras), C.c_uint32(n_images), ptr(rgba), ptr(bitfield)),
              "n2_trainer_set_scene")

    def attach_occupancy(self, occupancy):
        """From now on the rays march through ``occupancy``'s bitfield, which training_prep keeps up to date
        (the reference's own density grid instead of a bitfield supplied with the scene)."""
        if self._scene is None:
            raise N2Error("attach_occupancy: call set_scene first")
        self.occupancy = occupancy
        cameras, rgba, _ = self._scene
        n_images = self._n_images
        self.set_scene(cameras, n_images, rgba, occupancy.bitfield)

    def training_prep(self):
        """Testbed::train's occupancy-grid cadence for the step about to run (src/testbed.cu:2658-2674).
        Returns the (n_uniform, n_nonuniform) update that ran, or None."""
        occ = getattr(self, "occupancy", None)
        if occ is None:
            return None
        # the encoding's level mask is that of the step about to run (src/testbed.cu:2641-2647)
        check(capi.lib().n2_trainer_set_training_step(self._h, C.c_uint32(self.step_index)), "n2_trainer_set_training_step")
        plan = density_grid_update_plan(self.step_index, occ.n_cascades)
        if plan is None:
            return None
        # a sample generation running ahead reads the bitfield that is about to change
        check(capi.lib().n2_trainer_invalidate_prefetch(self._h), "n2_trainer_invalidate_prefetch")
        if self.step_index == 0:
            occ.reset()
        occ.update(self._field, plan[0], plan[1])
        return plan

    def step(self, n_rays=None, n_inference=None, seed=None):
        n_rays = self.budget.rays_per_batch if n_rays is None else n_rays
        n_inference = self.budget.n_inference() if n_inference is None else n_inference
        seed = self.step_index if seed is None else seed
        check(capi.lib().n2_trainer_set_training_step(self._h, C.c_uint32(self.step_index)), "n2_trainer_set_training_step")
        check(capi.lib().n2_trainer_step(self._h, self._stream(), C.c_uint32(n_rays), C.c_uint32(n_inference),
                                         C.c_uint32(seed)), "n2_trainer_step")
        self.step_index += 1
        if self.lr_schedule is not None:
            before = self.lr_schedule.learning_rate
            lr = self.lr_schedule.after_step(self.optimizer_state().optimizer_steps)
            if lr != before:
                check(capi.lib().n2_trainer_set_learning_rate(self._h, C.c_float(lr)), "n2_trainer_set_learning_rate")

    def optimizer_state(self):
        s = capi.TrainerOptimizerBuffers()
        check(capi.lib().n2_trainer_optimizer_state(self._h, C.byref(s)), "n2_trainer_optimizer_state")
        return s

    def _view(self, address, count, dtype):
        off = address - self._ws.data_ptr()
        return self._ws[off:off + count * torch.empty(0, dtype=dtype).element_size()].view(dtype)

    @property
    def inference_params(self):
        """fp16 parameters to render / extract with: the Ema copy when the wrapper is on, else the working copy."""
        return self._view(self.optimizer_state().inference_params, self.n_params, torch.float16)

    @property
    def ema_weights(self):
        s = self.optimizer_state()
        return None if not s.ema_weights else self._view(s.ema_weights, self.n_params, torch.float32)

    def last_step(self, n_rays, n_samples, n_inference):
        """Tensors (views into the workspace) of the last step's buffers: see n2_trainer_step_view.  n_rays / n_samples:
        the step's live rays and marched samples (read_counters), n_inference: the forward batch it was called with."""
        v = capi.TrainerStepView()
        check(capi.lib().n2_trainer_last_step_view(self._h, C.byref(v)), "n2_trainer_last_step_view")
        T = self.cfg.target_batch_size
        source_index = self._view(v.source_index, T, torch.int32)
        extra = {}
        if v.evaluated_samples:
            # a step in depth chunks: the index names places in the list of evaluated samples
            counts = self._view(v.evaluated_counts, 8, torch.int32)
            evaluated = self._view(v.evaluated_samples, self.cfg.max_samples, torch.int32)[:int(counts.sum().item())]
            source_index = evaluated[source_index.long()]
            extra = dict(evaluated_samples=evaluated, evaluated_counts=counts)
        return dict(**extra, coords=self._view(v.coords, n_samples * 7, torch.float32).view(-1, 7),
                    numsteps=self._view(v.numsteps, n_rays * 2, torch.int32).view(-1, 2),
                    rgb_target=self._view(v.rgb_target, n_rays * 3, torch.float32).view(-1, 3),
                    ray_indices=self._view(v.ray_indices, n_rays, torch.int32),
                    network_output=self._view(v.network_output, n_inference * 16, torch.float16).view(-1, 16),
                    coords_compacted=self._view(v.coords_compacted, T * 7, torch.float32).view(-1, 7),
                    dloss_doutput=self._view(v.dloss_doutput, T * 16, torch.float16).view(-1, 16),
                    source_index=source_index)

    def read_counters(self):
        r, s, c, l = C.c_uint32(), C.c_uint32(), C.c_uint32(), C.c_float()
        check(capi.lib().n2_trainer_read_counters(self._h, self._stream(), C.byref(r), C.byref(s), C.byref(c), C.byref(l)),
              "n2_trainer_read_counters")
        return dict(rays=int(r.value), samples=int(s.value), compacted=int(c.value), loss=float(l.value))

    # the forward pass in depth chunks pays (three rounds of sixteen samples) when a step marches this many times the
    # samples it keeps, and is switched off again below the lower figure
    DEPTH_CHUNKS_ON, DEPTH_CHUNKS_OFF = 1.6, 1.3
    DEPTH_CHUNKS = (16, 3)

    def _update_chunk_estimates(self):
        """After a step in depth chunks: its rounds' sample counts size the launches of the following steps."""
        v = capi.TrainerStepView()
        check(capi.lib().n2_trainer_last_step_view(self._h, C.byref(v)), "n2_trainer_last_step_view")
        if v.evaluated_counts and self.depth_chunks[1] >= 2:
            counts = self._view(v.evaluated_counts, 8, torch.int32).cpu().numpy().astype(np.uint32)
            check(capi.lib().n2_trainer_set_depth_chunk_estimates(self._h, counts.ctypes.data_as(C.c_void_p), C.c_uint32(self.depth_chunks[1])),
                  "n2_trainer_set_depth_chunk_estimates")

    def update_budget(self):
        c = self.read_counters()
        ok = self.budget.update(c["rays"], c["samples"], c["compacted"])
        if ok and self.auto_depth_chunks and not self.cfg.recompute_training_forward:
            ratio = c["samples"] / max(1, min(c["compacted"], self.cfg.target_batch_size))
            if ratio >= self.DEPTH_CHUNKS_ON and self.depth_chunks[1] < 2:
                self.set_depth_chunks(*self.DEPTH_CHUNKS)
            elif ratio <= self.DEPTH_CHUNKS_OFF and self.depth_chunks[1] >= 2:
                self.set_depth_chunks(0, 0)
            self._update_chunk_estimates()
        return c, ok

    def sdf(self, xyz):
        """NerfNetwork::sdf on a [3, N] tensor (N <= max_samples, multiple of 8): fp16 [16, N]."""
        n = xyz.shape[1]
        out = torch.empty((16, n), dtype=torch.float16, device=xyz.device)
        check(capi.lib().n2_field_sdf(self._field, self._stream(), ptr(xyz), C.c_uint32(1), C.c_uint32(n), C.c_uint32(n),
                                      ptr(out)), "n2_field_sdf")
        return out
