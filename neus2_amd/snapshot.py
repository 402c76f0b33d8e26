"""Snapshot files in the reference's format (Testbed::save_snapshot / load_snapshot, src/testbed.cu:3134-3244):
MessagePack of the network configuration plus a "snapshot" object.  The file is written and parsed by the C ABI
(n2_snapshot_*); this module gathers the trainer's and the occupancy grid's device buffers for it."""
import ctypes as C
import struct

import torch

from . import capi
from .capi import N2Error, check, ptr


class SnapshotDesc(C.Structure):
    """struct n2_snapshot_desc"""
    _fields_ = [("config_msgpack", C.c_void_p), ("config_bytes", C.c_uint64), ("n_params", C.c_uint32), ("d_params", C.c_void_p),
                ("include_optimizer_state", C.c_uint32), ("d_first_moments", C.c_void_p), ("d_second_moments", C.c_void_p),
                ("d_param_steps", C.c_void_p), ("d_ema_weights", C.c_void_p), ("optimizer_steps", C.c_uint32),
                ("learning_rate", C.c_float), ("d_density_grid", C.c_void_p), ("density_grid_cells", C.c_uint64),
                ("d_scratch", C.c_void_p), ("scratch_bytes", C.c_uint64), ("aabb_scale", C.c_uint32), ("rays_per_batch", C.c_uint32),
                ("measured_batch_size", C.c_uint32), ("measured_batch_size_before_compaction", C.c_uint32),
                ("training_step", C.c_uint32), ("loss", C.c_float), ("param_steps_bits", C.c_uint32)]


class SnapshotInfo(C.Structure):
    """struct n2_snapshot_info"""
    _fields_ = [("n_params", C.c_uint32), ("params_are_fp32", C.c_uint32), ("density_grid_size", C.c_uint32),
                ("density_grid_cells", C.c_uint64), ("aabb_scale", C.c_uint32), ("rays_per_batch", C.c_uint32),
                ("measured_batch_size", C.c_uint32), ("measured_batch_size_before_compaction", C.c_uint32),
                ("training_step", C.c_uint32), ("loss", C.c_float), ("has_optimizer_state", C.c_uint32),
                ("has_ema_weights", C.c_uint32), ("optimizer_steps", C.c_uint32), ("learning_rate", C.c_float)]


class SnapshotTargets(C.Structure):
    """struct n2_snapshot_targets"""
    _fields_ = [("n_params", C.c_uint32), ("d_master", C.c_void_p), ("d_params", C.c_void_p), ("d_density_grid", C.c_void_p),
                ("density_grid_cells", C.c_uint64), ("d_first_moments", C.c_void_p), ("d_second_moments", C.c_void_p),
                ("d_param_steps", C.c_void_p), ("d_ema_weights", C.c_void_p), ("d_scratch", C.c_void_p), ("scratch_bytes", C.c_uint64),
                ("param_steps_bits", C.c_uint32)]


def pack_config(obj):
    """MessagePack encoding of a JSON-like configuration (dict / list / str / int / float / bool / None), with the
    width rules nlohmann::json::to_msgpack uses (smallest integer form; float32 when exact, else float64)."""
    out = bytearray()

    def put(o):
        if o is None:
            out.append(0xc0)
        elif o is True or o is False:
            out.append(0xc3 if o else 0xc2)
        elif isinstance(o, int):
            if 0 <= o < 128:
                out.append(o)
            elif -32 <= o < 0:
                out.append(o & 0xff)
            elif o >= 0:
                for code, fmt, lim in ((0xcc, ">B", 1 << 8), (0xcd, ">H", 1 << 16), (0xce, ">I", 1 << 32), (0xcf, ">Q", 1 << 64)):
                    if o < lim:
                        out.append(code)
                        out.extend(struct.pack(fmt, o))
                        break
                else:
                    raise N2Error(f"integer {o} does not fit MessagePack")
            else:
                for code, fmt, lim in ((0xd0, ">b", 1 << 7), (0xd1, ">h", 1 << 15), (0xd2, ">i", 1 << 31), (0xd3, ">q", 1 << 63)):
                    if -lim <= o:
                        out.append(code)
                        out.extend(struct.pack(fmt, o))
                        break
                else:
                    raise N2Error(f"integer {o} does not fit MessagePack")
        elif isinstance(o, float):
            if struct.unpack(">f", struct.pack(">f", o))[0] == o:
                out.append(0xca)
                out.extend(struct.pack(">f", o))
            else:
                out.append(0xcb)
                out.extend(struct.pack(">d", o))
        elif isinstance(o, str):
            b = o.encode("utf-8")
            n = len(b)
            if n < 32:
                out.append(0xa0 | n)
            elif n < 256:
                out.extend((0xd9, n))
            elif n < 65536:
                out.append(0xda)
                out.extend(struct.pack(">H", n))
            else:
                out.append(0xdb)
                out.extend(struct.pack(">I", n))
            out.extend(b)
        elif isinstance(o, (list, tuple)):
            n = len(o)
            if n < 16:
                out.append(0x90 | n)
            elif n < 65536:
                out.append(0xdc)
                out.extend(struct.pack(">H", n))
            else:
                out.append(0xdd)
                out.extend(struct.pack(">I", n))
            for v in o:
                put(v)
        elif isinstance(o, dict):
            n = len(o)
            if n < 16:
                out.append(0x80 | n)
            elif n < 65536:
                out.append(0xde)
                out.extend(struct.pack(">H", n))
            else:
                out.append(0xdf)
                out.extend(struct.pack(">I", n))
            for k, v in o.items():
                if not isinstance(k, str):
                    raise N2Error("configuration keys must be strings")
                put(k)
                put(v)
        else:
            raise N2Error(f"cannot encode {type(o).__name__} in a configuration")

    put(obj)
    return bytes(out)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def save_snapshot(path, trainer, occupancy=None, config=None, include_optimizer_state=False, loss=0.0, aabb_scale=1):
    """Testbed::save_snapshot(path, include_optimizer_state).  ``params_binary`` holds the WORKING parameters (what
    tcnn's Trainer::serialize stores and training continues from); with the Ema wrapper on, the averaged weights that
    inference uses travel in the optimizer state (``include_optimizer_state=True``), and a file saved without it
    restarts the average from the working parameters when it is loaded."""
    d = SnapshotDesc()
    blob = pack_config(config) if config else b""
    keep = C.create_string_buffer(blob, len(blob)) if blob else None
    d.config_msgpack = C.cast(keep, C.c_void_p) if keep is not None else None
    d.config_bytes = len(blob)
    d.n_params = trainer.n_params
    d.d_params = trainer.params.data_ptr()
    st = trainer.optimizer_state()
    d.include_optimizer_state = 1 if include_optimizer_state else 0
    if include_optimizer_state:
        d.d_first_moments, d.d_second_moments, d.d_param_steps = st.first_moments, st.second_moments, st.param_steps
        d.param_steps_bits = st.param_steps_bits
        d.d_ema_weights = st.ema_weights
    d.optimizer_steps, d.learning_rate = st.optimizer_steps, st.learning_rate
    scratch = None
    if occupancy is not None:
        grid = occupancy.density_grid
        scratch = torch.empty(2 * grid.numel(), dtype=torch.uint8, device=grid.device)
        d.d_density_grid, d.density_grid_cells = grid.data_ptr(), grid.numel()
        d.d_scratch, d.scratch_bytes = scratch.data_ptr(), scratch.numel()
    d.aabb_scale = aabb_scale
    b = trainer.budget
    d.rays_per_batch, d.measured_batch_size = b.rays_per_batch, b.measured
    d.measured_batch_size_before_compaction = b.measured_before_compaction
    d.training_step, d.loss = trainer.step_index, loss
    check(capi.lib().n2_snapshot_save(str(path).encode(), C.byref(d), _stream()), "n2_snapshot_save")


def snapshot_info(path):
    h, info = C.c_void_p(), SnapshotInfo()
    check(capi.lib().n2_snapshot_open(str(path).encode(), C.byref(h), C.byref(info)), "n2_snapshot_open")
    capi.lib().n2_snapshot_close(h)
    return info


def load_snapshot(path, trainer, occupancy=None, load_optimizer_state=True):
    """Testbed::load_snapshot: parameters (fp32 master and fp16 copy), density grid (+ mean and bitfield), the ray
    budget, the training step and, when the file has it, the optimizer state.  Returns the file's info record."""
    L = capi.lib()
    h, info = C.c_void_p(), SnapshotInfo()
    check(L.n2_snapshot_open(str(path).encode(), C.byref(h), C.byref(info)), "n2_snapshot_open")
    try:
        t = SnapshotTargets()
        t.n_params = trainer.n_params
        t.d_master, t.d_params = trainer.master.data_ptr(), trainer.params.data_ptr()
        need = (4 if info.params_are_fp32 else 2) * info.n_params
        if occupancy is not None:
            grid = occupancy.density_grid
            t.d_density_grid, t.density_grid_cells = grid.data_ptr(), grid.numel()
            need = max(need, 2 * grid.numel())
        st = trainer.optimizer_state()
        with_opt = bool(load_optimizer_state and info.has_optimizer_state)
        if with_opt:
            t.d_first_moments, t.d_second_moments, t.d_param_steps = st.first_moments, st.second_moments, st.param_steps
            t.param_steps_bits = st.param_steps_bits
            if info.has_ema_weights and st.ema_weights:
                t.d_ema_weights = st.ema_weights
        scratch = torch.empty(need, dtype=torch.uint8, device=trainer.master.device)
        t.d_scratch, t.scratch_bytes = scratch.data_ptr(), need
        check(L.n2_snapshot_read(h, _stream(), C.byref(t)), "n2_snapshot_read")
        if with_opt:
            check(L.n2_trainer_set_optimizer_steps(trainer._h, C.c_uint32(info.optimizer_steps)), "n2_trainer_set_optimizer_steps")
            check(L.n2_trainer_set_learning_rate(trainer._h, C.c_float(info.learning_rate)), "n2_trainer_set_learning_rate")
        if with_opt and t.d_ema_weights:
            # the moving average continues: its fp16 copy (the inference parameters) follows from the fp32 weights
            trainer.inference_params.copy_(trainer.ema_weights.half())
            check(L.n2_trainer_restart_ema(trainer._h, _stream(), C.c_uint32(info.optimizer_steps)), "n2_trainer_restart_ema")
        else:
            # no Ema state came with the file: the average starts again from the loaded parameters, so that the
            # inference parameters are the loaded ones and the next step does not blend a stale average into them
            check(L.n2_trainer_restart_ema(trainer._h, _stream(), C.c_uint32(0)), "n2_trainer_restart_ema")
        if occupancy is not None and info.density_grid_cells:
            occupancy.update_bitfield()  # update_density_grid_mean_and_bitfield, src/testbed.cu:3225-3227
        trainer.step_index = info.training_step
        check(L.n2_trainer_set_training_step(trainer._h, C.c_uint32(info.training_step)), "n2_trainer_set_training_step")
        trainer.budget.rays_per_batch = info.rays_per_batch or trainer.budget.rays_per_batch
        trainer.budget.measured_before_compaction = info.measured_batch_size_before_compaction
        trainer.budget.measured = info.measured_batch_size
        check(L.n2_trainer_invalidate_prefetch(trainer._h), "n2_trainer_invalidate_prefetch")
    finally:
        L.n2_snapshot_close(h)
    return info
