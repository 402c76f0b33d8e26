"""ctypes binding of libneus2_amd.so (the C ABI declared in include/neus2_amd.h).

The library must have been built (``python -m neus2_amd.build``); there is no
fallback implementation: a missing library is an ImportError-class failure.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libneus2_amd.so")

N2_OK = 0
GRAD_IGNORE, GRAD_OVERWRITE, GRAD_ACCUMULATE = 0, 1, 2
LAYOUT_SOA, LAYOUT_AOS = 0, 1

_lib = None


class FieldConfig(C.Structure):
    """struct n2_field_config"""
    _fields_ = [("n_levels", C.c_uint32), ("n_features_per_level", C.c_uint32), ("log2_hashmap_size", C.c_uint32),
                ("base_resolution", C.c_uint32), ("per_level_scale", C.c_float), ("sdf_hidden_layers", C.c_uint32),
                ("rgb_hidden_layers", C.c_uint32), ("sdf_bias", C.c_float)]


class AdamConfig(C.Structure):
    """struct n2_adam_config (defaults: configs/nerf/base.json:13-26)"""
    _fields_ = [("learning_rate", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("epsilon", C.c_float),
                ("l2_reg", C.c_float)]


class CompositeConfig(C.Structure):
    """struct n2_composite_config"""
    _fields_ = [("loss_scale", C.c_float), ("ek_loss_weight", C.c_float), ("cos_anneal_ratio", C.c_float),
                ("background", C.c_float * 3), ("n_rays_norm", C.c_uint32)]


class Camera(C.Structure):
    """struct n2_camera"""
    _fields_ = [("xform", C.c_float * 12), ("focal_length", C.c_float * 2), ("principal_point", C.c_float * 2),
                ("resolution", C.c_uint32 * 2), ("pixel_offset_lo", C.c_uint32), ("pixel_offset_hi", C.c_uint32)]


class TrainerConfig(C.Structure):
    """struct n2_trainer_config"""
    _fields_ = [("field", FieldConfig), ("adam", AdamConfig), ("composite", CompositeConfig),
                ("target_batch_size", C.c_uint32), ("max_rays_per_batch", C.c_uint32), ("max_samples", C.c_uint32),
                ("loss_scale", C.c_float), ("prefetch_samples", C.c_uint32), ("ema_decay", C.c_float),
                ("recompute_training_forward", C.c_uint32)]


class TrainerOptimizerBuffers(C.Structure):
    """struct n2_trainer_optimizer_buffers"""
    _fields_ = [("first_moments", C.c_void_p), ("second_moments", C.c_void_p), ("param_steps", C.c_void_p),
                ("ema_weights", C.c_void_p), ("inference_params", C.c_void_p), ("optimizer_steps", C.c_uint32),
                ("learning_rate", C.c_float), ("param_steps_bits", C.c_uint32)]


class TrainerStepView(C.Structure):
    """struct n2_trainer_step_view"""
    _fields_ = [("coords", C.c_void_p), ("numsteps", C.c_void_p), ("rgb_target", C.c_void_p), ("ray_indices", C.c_void_p),
                ("network_output", C.c_void_p), ("coords_compacted", C.c_void_p), ("dloss_doutput", C.c_void_p),
                ("source_index", C.c_void_p), ("evaluated_samples", C.c_void_p), ("evaluated_counts", C.c_void_p)]


class OccupancyBuffers(C.Structure):
    """struct n2_occupancy_buffers"""
    _fields_ = [("density_grid", C.c_void_p), ("density_grid_tmp", C.c_void_p), ("bitfield", C.c_void_p), ("mean", C.c_void_p),
                ("positions", C.c_void_p), ("indices", C.c_void_p), ("n_samples", C.c_uint32), ("n_cascades", C.c_uint32),
                ("ema_step", C.c_uint32), ("n_uniform", C.c_uint32), ("rng_state", C.c_uint64), ("rng_inc", C.c_uint64)]


class N2Error(RuntimeError):
    """A C-ABI call returned a non-zero status (mirrors the reference's std::runtime_error)."""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise N2Error(f"{LIB_PATH} is missing: build it with `python -m neus2_amd.build` "
                          "(there is no CPU or eager fallback)")
        # torch owns the device memory and streams this library is handed, so both must share ONE HIP runtime: torch
        # ships its own copy, and whichever copy is loaded first serves every later request for that library name.
        # Loading torch first makes its copy the shared one (the other order leaves two runtimes that do not see each
        # other's allocations).
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _lib = C.CDLL(LIB_PATH)
        _lib.n2_last_error.restype = C.c_char_p
        _lib.n2_version.restype = C.c_char_p
        _lib.n2_field_encoding.restype = C.c_void_p
        _lib.n2_field_encoding.argtypes = [C.c_void_p]
        for name in ("n2_grid_n_params", "n2_grid_output_width", "n2_grid_n_levels", "n2_grid_active_levels"):
            getattr(_lib, name).restype = C.c_uint32
            getattr(_lib, name).argtypes = [C.c_void_p]
        _lib.n2_grid_workspace_bytes.restype = C.c_uint64
        _lib.n2_grid_workspace_bytes.argtypes = [C.c_void_p, C.c_uint32]
        _lib.n2_grid_destroy.restype = None
        _lib.n2_grid_destroy.argtypes = [C.c_void_p]
        for name in ("n2_mlp_n_params", "n2_mlp_input_width", "n2_mlp_output_width"):
            getattr(_lib, name).restype = C.c_uint32
            getattr(_lib, name).argtypes = [C.c_void_p]
        _lib.n2_mlp_workspace_bytes.restype = C.c_uint64
        _lib.n2_mlp_workspace_bytes.argtypes = [C.c_void_p]
        _lib.n2_mlp_destroy.restype = None
        _lib.n2_mlp_destroy.argtypes = [C.c_void_p]
        _lib.n2_field_n_params.restype = C.c_uint32
        _lib.n2_field_n_params.argtypes = [C.c_void_p]
        _lib.n2_field_workspace_bytes.restype = C.c_uint64
        _lib.n2_field_workspace_bytes.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32]
        _lib.n2_composite_workspace_bytes.restype = C.c_uint64
        _lib.n2_composite_workspace_bytes.argtypes = [C.c_uint32]
        _lib.n2_sampler_workspace_bytes.restype = C.c_uint64
        _lib.n2_sampler_workspace_bytes.argtypes = [C.c_uint32]
        _lib.n2_sdf_eikonal_workspace_bytes.restype = C.c_uint64
        _lib.n2_sdf_eikonal_workspace_bytes.argtypes = [C.c_uint32]
        _lib.n2_trainer_workspace_bytes.restype = C.c_uint64
        _lib.n2_trainer_workspace_bytes.argtypes = [C.c_void_p]
        _lib.n2_trainer_destroy.restype = None
        _lib.n2_trainer_destroy.argtypes = [C.c_void_p]
        _lib.n2_trainer_field.restype = C.c_void_p
        _lib.n2_trainer_field.argtypes = [C.c_void_p]
        _lib.n2_field_destroy.restype = None
        _lib.n2_field_destroy.argtypes = [C.c_void_p]
        _lib.n2_occupancy_workspace_bytes.restype = C.c_uint64
        _lib.n2_occupancy_workspace_bytes.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32]
        _lib.n2_snapshot_close.restype = None
        _lib.n2_snapshot_close.argtypes = [C.c_void_p]
        _lib.n2_occupancy_destroy.restype = None
        _lib.n2_occupancy_destroy.argtypes = [C.c_void_p]
    return _lib


def check(rc, what=""):
    if rc != N2_OK:
        raise N2Error(f"{what} failed with status {rc}: {lib().n2_last_error().decode()}")


def ptr(t):
    """Device (or host) address of a torch tensor / numpy array, or NULL for None."""
    if t is None:
        return C.c_void_p(0)
    if hasattr(t, "data_ptr"):
        return C.c_void_p(t.data_ptr())
    return C.c_void_p(t.ctypes.data)
