"""Python mirror of the reference's tcnn-style objects on top of the C ABI.

torch is used for device memory and streams only; every computation is a call
into libneus2_amd.so.  Method names and argument meaning follow the interface
the reference drives (``tcnn::Encoding`` / ``tcnn::Network``; call sites in
include/neural-graphics-primitives/nerf_network.h).
"""
import ctypes as C

import numpy as np
import torch

from . import capi
from .capi import (GRAD_ACCUMULATE, GRAD_IGNORE, GRAD_OVERWRITE, LAYOUT_AOS, LAYOUT_SOA, N2Error, check,  # noqa: F401
                   ptr)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _positions(xyz):
    """Accepts a 3 x N SoA float32 tensor or an N x C (C >= 3) row-per-point tensor
    (the 7-float NerfCoordinate batch, nerf.h:76-102).  Returns (tensor, point_stride, dim_stride, N)."""
    if xyz.dtype != torch.float32 or not xyz.is_cuda:
        raise N2Error("positions must be a float32 CUDA tensor")
    if not xyz.is_contiguous():
        raise N2Error("positions must be contiguous")
    if xyz.dim() == 2 and xyz.shape[0] == 3:
        return xyz, 1, max(xyz.shape[1], 1), xyz.shape[1]
    if xyz.dim() == 2 and xyz.shape[1] >= 3:
        return xyz, xyz.shape[1], 1, xyz.shape[0]
    raise N2Error(f"positions must be 3 x N or N x C, got {tuple(xyz.shape)}")


class GridEncoding:
    """tcnn::GridEncoding<__half, 3, 2> (created at nerf_network.h:46)."""

    def __init__(self, n_levels=16, n_features_per_level=2, log2_hashmap_size=19, base_resolution=16,
                 per_level_scale=1.447):
        self._h = C.c_void_p()
        check(capi.lib().n2_grid_create(C.c_uint32(n_levels), C.c_uint32(n_features_per_level),
                                        C.c_uint32(log2_hashmap_size), C.c_uint32(base_resolution),
                                        C.c_float(per_level_scale), C.byref(self._h)), "n2_grid_create")
        self.n_levels = n_levels
        self._params = self._grads = None
        self._owner = None

    @classmethod
    def _borrowed(cls, handle, owner):
        """A view of a grid that another object owns (NerfNetwork.encoding()): never destroyed from here."""
        g = cls.__new__(cls)
        g._h = C.c_void_p(handle)
        g._owner = owner
        g._params = g._grads = None
        g.n_levels = int(capi.lib().n2_grid_n_levels(g._h))
        return g

    def __del__(self):
        try:
            if getattr(self, "_owner", None) is None and getattr(self, "_h", None) is not None and self._h.value:
                capi.lib().n2_grid_destroy(self._h)
                self._h = C.c_void_p()
        except Exception:  # interpreter shutdown: the module globals may already be gone
            pass

    def n_params(self):
        return int(capi.lib().n2_grid_n_params(self._h))

    def output_width(self):
        return int(capi.lib().n2_grid_output_width(self._h))

    padded_output_width = output_width

    def input_width(self):
        return 3

    def level_table(self):
        L = self.n_levels
        scale = np.zeros(L, np.float32)
        res, ent, off = np.zeros(L, np.uint32), np.zeros(L, np.uint32), np.zeros(L + 1, np.uint32)
        check(capi.lib().n2_grid_level_table(self._h, ptr(scale), ptr(res), ptr(ent), ptr(off)), "n2_grid_level_table")
        return scale, res, ent, off

    def set_params(self, params, gradients=None):
        """params / gradients: fp16 CUDA tensors of n_params elements (kept alive by this object)."""
        for t in (params, gradients):
            if t is not None and (t.dtype != torch.float16 or not t.is_cuda or t.numel() != self.n_params()
                                  or not t.is_contiguous()):
                raise N2Error("grid params/gradients must be contiguous fp16 CUDA tensors of n_params elements")
        check(capi.lib().n2_grid_set_params(self._h, ptr(params), ptr(gradients)), "n2_grid_set_params")
        self._params, self._grads = params, gradients

    def set_point_order(self, lattice_order):
        """Hint for forwards without dy_dx: True when the points come in lattice order (get_density_on_grid)."""
        check(capi.lib().n2_grid_set_point_order(self._h, C.c_int(1 if lattice_order else 0)), "n2_grid_set_point_order")

    def set_max_level(self, value):
        """Fraction of the levels in use (GridEncoding::set_max_level, src/testbed.cu:1861-1866); 1 = all."""
        check(capi.lib().n2_grid_set_max_level(self._h, C.c_float(value)), "n2_grid_set_max_level")

    def set_max_level_gpu(self, per_point):
        """One fraction per point (fp32 CUDA tensor, kept alive here) or None (src/testbed_nerf.cu:3837-3843, 3985)."""
        if per_point is not None and (per_point.dtype != torch.float32 or not per_point.is_cuda or not per_point.is_contiguous()):
            raise N2Error("max_level_gpu must be a contiguous fp32 CUDA tensor")
        check(capi.lib().n2_grid_set_max_level_gpu(self._h, ptr(per_point)), "n2_grid_set_max_level_gpu")
        self._max_level_gpu = per_point

    def set_progressive(self, base_valid_level_scale, valid_level_scale, base_training_step):
        """Encoding keys of configs/nerf/base.json:36-38; base_training_step 0 switches the progressive mask off."""
        check(capi.lib().n2_grid_set_progressive(self._h, C.c_float(base_valid_level_scale), C.c_float(valid_level_scale),
                                                 C.c_uint32(base_training_step)), "n2_grid_set_progressive")

    def set_training_step(self, step):
        """Encoding::set_training_step (src/testbed.cu:2643-2646)."""
        check(capi.lib().n2_grid_set_training_step(self._h, C.c_uint32(max(0, int(step)))), "n2_grid_set_training_step")

    def active_levels(self):
        return int(capi.lib().n2_grid_active_levels(self._h))

    def reserve_scatter_workspace(self, max_points):
        """Scratch that lets backward passes of >= 4096 points sort their updates in LDS instead of issuing
        global atomics.  Returns False when the table shape does not support it."""
        nbytes = int(capi.lib().n2_grid_workspace_bytes(self._h, C.c_uint32(max_points)))
        if nbytes == 0:
            return False
        self._scatter_ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        check(capi.lib().n2_grid_set_workspace(self._h, ptr(self._scatter_ws), C.c_uint64(nbytes), C.c_uint32(max_points)),
              "n2_grid_set_workspace")
        return True

    def forward(self, xyz, prepare_input_gradients=False, out=None):
        """Returns (out fp16 [width, N], ctx) where ctx holds dy_dx when requested; ``out`` may be a [width, N]
        row block of a wider matrix (the encoding rows of the network input, nerf_network.h:184-190)."""
        x, ps, ds, n = _positions(xyz)
        if out is None:
            out = torch.empty((self.output_width(), n), dtype=torch.float16, device=x.device)
        else:
            _check_half(out, (self.output_width(), n), "grid output")
        dy_dx = torch.empty((self.output_width(), n, 3), dtype=torch.float32, device=x.device) \
            if prepare_input_gradients else None
        check(capi.lib().n2_grid_forward(self._h, _stream(), ptr(x), C.c_uint32(ps), C.c_uint32(ds), C.c_uint32(n),
                                         ptr(out), ptr(dy_dx)), "n2_grid_forward")
        return out, dy_dx

    def backward(self, ctx, xyz, dL_dy, want_input_grad=False, mode=GRAD_OVERWRITE):
        x, ps, ds, n = _positions(xyz)
        if dL_dy.dtype != torch.float16 or tuple(dL_dy.shape) != (self.output_width(), n) or not dL_dy.is_contiguous():
            raise N2Error("dL_dy must be a contiguous fp16 [output_width, N] tensor")
        dx = torch.empty((3, n), dtype=torch.float32, device=x.device) if want_input_grad else None
        check(capi.lib().n2_grid_backward(self._h, _stream(), ptr(x), C.c_uint32(ps), C.c_uint32(ds), C.c_uint32(n),
                                          ptr(dL_dy), ptr(ctx), ptr(dx), C.c_int(mode)), "n2_grid_backward")
        return dx

    def backward_backward_input(self, xyz, dL_ddLdx, dL_dy, want_dL_ddLdy=True, want_dL_dx=False,
                                mode=GRAD_ACCUMULATE):
        x, ps, ds, n = _positions(xyz)
        if dL_ddLdx.dtype != torch.float32 or tuple(dL_ddLdx.shape) != (3, n) or not dL_ddLdx.is_contiguous():
            raise N2Error("dL_ddLdx must be a contiguous fp32 [3, N] tensor")
        if dL_dy.dtype != torch.float16 or tuple(dL_dy.shape) != (self.output_width(), n) or not dL_dy.is_contiguous():
            raise N2Error("dL_dy must be a contiguous fp16 [output_width, N] tensor")
        o = torch.empty((self.output_width(), n), dtype=torch.float16, device=x.device) if want_dL_ddLdy else None
        dx = torch.empty((3, n), dtype=torch.float32, device=x.device) if want_dL_dx else None
        check(capi.lib().n2_grid_backward_backward_input(self._h, _stream(), ptr(x), C.c_uint32(ps), C.c_uint32(ds),
                                                         C.c_uint32(n), ptr(dL_ddLdx), ptr(dL_dy), ptr(o), ptr(dx),
                                                         C.c_int(mode)), "n2_grid_backward_backward_input")
        return o, dx

    def backward_fused(self, xyz, dL_dy, dL_ddLdx, dL_dy_second, want_dL_ddLdy=True, mode=GRAD_OVERWRITE):
        """backward (parameter gradients only) + backward_backward_input in one scatter pass."""
        x, ps, ds, n = _positions(xyz)
        w = self.output_width()
        for t, what in ((dL_dy, "dL_dy"), (dL_dy_second, "dL_dy_second")):
            if t.dtype != torch.float16 or tuple(t.shape) != (w, n) or not t.is_contiguous():
                raise N2Error(f"{what} must be a contiguous fp16 [output_width, N] tensor")
        if dL_ddLdx.dtype != torch.float32 or tuple(dL_ddLdx.shape) != (3, n) or not dL_ddLdx.is_contiguous():
            raise N2Error("dL_ddLdx must be a contiguous fp32 [3, N] tensor")
        o = torch.empty((w, n), dtype=torch.float16, device=x.device) if want_dL_ddLdy else None
        check(capi.lib().n2_grid_backward_fused(self._h, _stream(), ptr(x), C.c_uint32(ps), C.c_uint32(ds), C.c_uint32(n),
                                                ptr(dL_dy), ptr(dL_ddLdx), ptr(dL_dy_second), ptr(o), C.c_int(mode)),
              "n2_grid_backward_fused")
        return o

    def corner_indices(self, xyz):
        x, ps, ds, n = _positions(xyz)
        idx = torch.empty((self.n_levels, 8, n), dtype=torch.int32, device=x.device)
        check(capi.lib().n2_grid_corner_indices(self._h, _stream(), ptr(x), C.c_uint32(ps), C.c_uint32(ds),
                                                C.c_uint32(n), ptr(idx)), "n2_grid_corner_indices")
        return idx


def _check_half(t, shape, what):
    if t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous() or tuple(t.shape) != tuple(shape):
        raise N2Error(f"{what} must be a contiguous fp16 CUDA tensor of shape {tuple(shape)}, got {t.dtype} {tuple(t.shape)}")


class FullyFusedMLP:
    """tcnn::FullyFusedMLP<__half, 64>: ReLU hidden layers, linear 16-wide output, no bias
    (created at nerf_network.h:57 and :65)."""

    def __init__(self, n_input_dims, n_hidden_layers, n_neurons=64, n_output_dims=16):
        if n_neurons != 64 or n_output_dims != 16:
            raise N2Error("only n_neurons = 64 and n_output_dims = 16 are implemented")
        self._h = C.c_void_p()
        check(capi.lib().n2_mlp_create(C.c_uint32(n_input_dims), C.c_uint32(n_hidden_layers), C.byref(self._h)),
              "n2_mlp_create")
        self.n_hidden_layers = n_hidden_layers
        self._params = self._grads = self._ws = None

    def __del__(self):
        try:
            if getattr(self, "_h", None) is not None and self._h.value:
                capi.lib().n2_mlp_destroy(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass

    def n_params(self):
        return int(capi.lib().n2_mlp_n_params(self._h))

    def input_width(self):
        return int(capi.lib().n2_mlp_input_width(self._h))

    def padded_output_width(self):
        return int(capi.lib().n2_mlp_output_width(self._h))

    output_width = padded_output_width

    def set_params(self, params, gradients=None):
        for t in (params, gradients):
            if t is not None:
                _check_half(t, (self.n_params(),), "mlp params/gradients")
        check(capi.lib().n2_mlp_set_params(self._h, ptr(params), ptr(gradients)), "n2_mlp_set_params")
        self._params, self._grads = params, gradients
        if gradients is not None and self._ws is None:
            nbytes = int(capi.lib().n2_mlp_workspace_bytes(self._h))
            self._ws = torch.empty(nbytes, dtype=torch.uint8, device=params.device)
            check(capi.lib().n2_mlp_set_workspace(self._h, ptr(self._ws), C.c_uint64(nbytes)), "n2_mlp_set_workspace")

    def set_output_gradient_exponent(self, exponent):
        """backward() with weight gradients multiplies dL/doutput by 2**exponent while it works and divides what it
        returns by it (n2_mlp_set_output_gradient_exponent): for output gradients in fp16's subnormal range."""
        check(capi.lib().n2_mlp_set_output_gradient_exponent(self._h, C.c_int(exponent)), "n2_mlp_set_output_gradient_exponent")

    def _out(self, n, layout, device):
        shape = (n, 16) if layout == LAYOUT_AOS else (16, n)
        return torch.empty(shape, dtype=torch.float16, device=device)

    def forward(self, x, out_layout=LAYOUT_SOA, want_hidden=False, out=None):
        """x: fp16 [in_width, N].  Returns (y, hidden): y is [16, N] (SoA) or [N, 16] (AoS)."""
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        y = self._out(n, out_layout, x.device) if out is None else out
        hid = torch.empty((64 * self.n_hidden_layers, n), dtype=torch.float16, device=x.device) if want_hidden else None
        check(capi.lib().n2_mlp_forward(self._h, _stream(), ptr(x), C.c_uint32(n), ptr(y), C.c_int(out_layout),
                                        ptr(hid)), "n2_mlp_forward")
        return y, hid

    inference_mixed_precision = forward

    def backward(self, x, dL_dy, dL_layout=LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE):
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        _check_half(dL_dy, (n, 16) if dL_layout == LAYOUT_AOS else (16, n), "dL_doutput")
        dx = torch.empty((self.input_width(), n), dtype=torch.float16, device=x.device) if want_input_grad else None
        check(capi.lib().n2_mlp_backward(self._h, _stream(), ptr(x), C.c_uint32(n), ptr(dL_dy), C.c_int(dL_layout),
                                         ptr(dx), C.c_int(mode)), "n2_mlp_backward")
        return dx

    def input_gradient(self, x, dim=0):
        """d output[dim] / d input for every sample (Network::input_gradient, nerf_network.h:229): fp16 [in_width, N]."""
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        d = torch.empty((self.input_width(), n), dtype=torch.float16, device=x.device)
        check(capi.lib().n2_mlp_input_gradient(self._h, _stream(), C.c_uint32(dim), ptr(x), C.c_uint32(n), ptr(d)),
              "n2_mlp_input_gradient")
        return d

    def backward_rows(self, x, dL_dy, n_rows, dL_layout=LAYOUT_SOA, want_input_grad=True, mode=GRAD_OVERWRITE):
        """backward() that uses only the first n_rows rows of dL_dy and takes the others as zero (n2_mlp_backward_rows)."""
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        _check_half(dL_dy, (n, 16) if dL_layout == LAYOUT_AOS else (16, n), "dL_doutput")
        dx = torch.empty((self.input_width(), n), dtype=torch.float16, device=x.device) if want_input_grad else None
        check(capi.lib().n2_mlp_backward_rows(self._h, _stream(), ptr(x), C.c_uint32(n), ptr(dL_dy), C.c_int(dL_layout),
                                              C.c_uint32(n_rows), ptr(dx), C.c_int(mode)), "n2_mlp_backward_rows")
        return dx

    def forward_and_input_gradient(self, x, dim=0, out_layout=LAYOUT_SOA, out=None):
        """forward and input_gradient(dim) in one pass over the input: (y, d output[dim] / d input)."""
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        y = self._out(n, out_layout, x.device) if out is None else out
        d = torch.empty((self.input_width(), n), dtype=torch.float16, device=x.device)
        check(capi.lib().n2_mlp_forward_and_input_gradient(self._h, _stream(), C.c_uint32(dim), ptr(x), C.c_uint32(n), ptr(y),
                                                           C.c_int(out_layout), ptr(d)), "n2_mlp_forward_and_input_gradient")
        return y, d

    def set_deferred_reduction(self, enable):
        """Leave the per-workgroup weight-gradient sums of backward / backward_backward_input pending until
        reduce_deferred (no tcnn counterpart: tcnn's weight gradients are GEMMs)."""
        check(capi.lib().n2_mlp_set_deferred_reduction(self._h, C.c_int(1 if enable else 0)), "n2_mlp_set_deferred_reduction")

    def reduce_deferred(self, other=None):
        check(capi.lib().n2_mlp_reduce_deferred(self._h, other._h if other is not None else None, _stream()),
              "n2_mlp_reduce_deferred")

    def backward_backward_input(self, x, dL_ddLdinput, dL_doutput, want_dL_ddLdoutput=False, mode=GRAD_ACCUMULATE):
        """dL_doutput None: the first-order output gradient was e_0 for every sample (the SDF's own gradient)."""
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        _check_half(dL_ddLdinput, (self.input_width(), n), "dL_ddLdinput")
        if dL_doutput is not None:
            _check_half(dL_doutput, (16, n), "dL_doutput")
        o = torch.empty((16, n), dtype=torch.float16, device=x.device) if want_dL_ddLdoutput else None
        check(capi.lib().n2_mlp_backward_backward_input(self._h, _stream(), ptr(x), C.c_uint32(n), ptr(dL_ddLdinput),
                                                        ptr(dL_doutput), ptr(o), C.c_int(mode)),
              "n2_mlp_backward_backward_input")
        return o

    def backward_and_second_order(self, x, dL_dy, dL_ddLdinput, second_dL_doutput=None, dL_layout=LAYOUT_SOA, mode=GRAD_OVERWRITE):
        """backward(mode) followed by backward_backward_input(Accumulate) in one pass over the input (one hidden
        layer).  Returns dL_dx of the first-order pass."""
        n = x.shape[1]
        _check_half(x, (self.input_width(), n), "mlp input")
        _check_half(dL_dy, (n, 16) if dL_layout == LAYOUT_AOS else (16, n), "dL_doutput")
        _check_half(dL_ddLdinput, (self.input_width(), n), "dL_ddLdinput")
        if second_dL_doutput is not None:
            _check_half(second_dL_doutput, (16, n), "second dL_doutput")
        dx = torch.empty((self.input_width(), n), dtype=torch.float16, device=x.device)
        check(capi.lib().n2_mlp_backward_and_second_order(self._h, _stream(), ptr(x), C.c_uint32(n), ptr(dL_dy),
                                                          C.c_int(dL_layout), ptr(dx), ptr(dL_ddLdinput),
                                                          ptr(second_dL_doutput), C.c_int(mode)),
              "n2_mlp_backward_and_second_order")
        return dx


class NerfNetwork:
    """NerfNetwork<__half> of the reference (nerf_network.h), static scene: grid + SDF MLP +
    SH direction encoding + colour MLP + variance, with normals computed inside the forward and
    the second-order passes inside the backward."""

    def __init__(self, n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447,
                 sdf_hidden_layers=1, rgb_hidden_layers=2, sdf_bias=-0.1):
        cfg = capi.FieldConfig(n_levels, 2, log2_hashmap_size, base_resolution, per_level_scale, sdf_hidden_layers,
                               rgb_hidden_layers, sdf_bias)
        self._h = C.c_void_p()
        check(capi.lib().n2_field_create(C.byref(cfg), C.byref(self._h)), "n2_field_create")
        self._params = self._grads = self._ws = None
        self.max_batch = 0

    def __del__(self):
        try:
            if getattr(self, "_h", None) is not None and self._h.value:
                capi.lib().n2_field_destroy(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass

    def n_params(self):
        return int(capi.lib().n2_field_n_params(self._h))

    def encoding(self):
        """The field's grid encoding (NerfNetwork::encoding(), src/testbed.cu:2643-2646), for the level-mask setters."""
        return GridEncoding._borrowed(capi.lib().n2_field_encoding(self._h), self)

    def param_offsets(self):
        o = (C.c_uint32 * 5)()
        check(capi.lib().n2_field_param_offsets(self._h, o), "n2_field_param_offsets")
        return list(o)

    def padded_output_width(self):
        return 16

    def set_params(self, params, gradients=None):
        for t in (params, gradients):
            if t is not None:
                _check_half(t, (self.n_params(),), "field params/gradients")
        check(capi.lib().n2_field_set_params(self._h, ptr(params), ptr(gradients)), "n2_field_set_params")
        self._params, self._grads = params, gradients

    def reserve(self, max_batch):
        """Allocates the workspace (the reference's arena temporaries) for batches up to max_batch."""
        if max_batch <= self.max_batch:
            return
        nbytes = int(capi.lib().n2_field_workspace_bytes(self._h, C.c_uint32(max_batch), C.c_uint32(max_batch)))
        self._ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        check(capi.lib().n2_field_set_workspace(self._h, ptr(self._ws), C.c_uint64(nbytes), C.c_uint32(max_batch),
                                                C.c_uint32(max_batch)), "n2_field_set_workspace")
        self.max_batch = max_batch

    @staticmethod
    def _coords(coords):
        if coords.dtype != torch.float32 or not coords.is_cuda or not coords.is_contiguous() or coords.dim() != 2 \
                or coords.shape[1] != 7:
            raise N2Error("coords must be a contiguous float32 CUDA tensor [N, 7]")
        return coords.shape[0]

    def forward(self, coords, out=None):
        n = self._coords(coords)
        self.reserve(n)
        y = torch.empty((n, 16), dtype=torch.float16, device=coords.device) if out is None else out
        check(capi.lib().n2_field_forward(self._h, _stream(), ptr(coords), C.c_uint32(n), ptr(y)), "n2_field_forward")
        return y

    inference_mixed_precision = forward

    def backward(self, coords, dL_doutput, ek_batch_size=None, mode=GRAD_OVERWRITE):
        n = self._coords(coords)
        _check_half(dL_doutput, (n, 16), "dL_doutput")
        check(capi.lib().n2_field_backward(self._h, _stream(), ptr(coords), C.c_uint32(n), ptr(dL_doutput),
                                           C.c_uint32(n if ek_batch_size is None else ek_batch_size), C.c_int(mode)),
              "n2_field_backward")

    def select(self, source_index, n_source):
        """Makes the samples source_index (uint32/int32 CUDA tensor) of the last forward, which ran over n_source
        samples, the batch of the next backward (n2_field_select); backward is then called with their coordinates."""
        if source_index.dtype not in (torch.int32, torch.uint32) or not source_index.is_cuda or not source_index.is_contiguous():
            raise N2Error("source_index must be a contiguous 32-bit integer CUDA tensor")
        check(capi.lib().n2_field_select(self._h, _stream(), ptr(source_index), C.c_uint32(n_source), C.c_uint32(source_index.numel())),
              "n2_field_select")

    def _sdf(self, fn, xyz):
        x, ps, ds, n = _positions(xyz)
        self.reserve(n)
        out = torch.empty((16, n), dtype=torch.float16, device=x.device)
        check(getattr(capi.lib(), fn)(self._h, _stream(), ptr(x), C.c_uint32(ps), C.c_uint32(ds), C.c_uint32(n),
                                      ptr(out)), fn)
        return out

    def sdf(self, xyz):
        return self._sdf("n2_field_sdf", xyz)

    def density(self, xyz):
        return self._sdf("n2_field_density", xyz)


class Adam:
    """tcnn Adam as Trainer::optimizer_step runs it (src/testbed_nerf.cu:3498): fp32 master weights,
    fp16 working copy, per-parameter step counters, l2_reg on matrix parameters only and a skip
    for non-matrix parameters whose gradient is exactly zero."""

    def __init__(self, master, n_matrix_params, learning_rate=1e-3, beta1=0.9, beta2=0.99, epsilon=1e-15, l2_reg=1e-6):
        if master.dtype != torch.float32 or not master.is_cuda or not master.is_contiguous():
            raise N2Error("master weights must be a contiguous float32 CUDA tensor")
        self.cfg = capi.AdamConfig(learning_rate, beta1, beta2, epsilon, l2_reg)
        self.master = master
        self.n_matrix_params = n_matrix_params
        self.m1 = torch.zeros_like(master)
        self.m2 = torch.zeros_like(master)
        self.steps = torch.zeros(master.numel(), dtype=torch.int32, device=master.device)

    def step(self, params, gradients, loss_scale=128.0):
        n = self.master.numel()
        _check_half(params, (n,), "params")
        _check_half(gradients, (n,), "gradients")
        check(capi.lib().n2_adam_step(_stream(), C.byref(self.cfg), C.c_uint32(n), C.c_uint32(self.n_matrix_params),
                                      C.c_float(loss_scale), ptr(self.master), ptr(params), ptr(gradients),
                                      ptr(self.m1), ptr(self.m2), ptr(self.steps)), "n2_adam_step")


def composite_loss(numsteps, network_output, coords, rgb_target, max_samples_compacted, n_rays_norm=None,
                   loss_scale=128.0, ek_loss_weight=0.01, cos_anneal_ratio=1.0, background=(0.0, 0.0, 0.0),
                   ray_counter=None, want_loss=True):
    """compute_loss_kernel_train_nerf_with_global_movement (src/testbed_nerf.cu:1465-1996), static path.
    numsteps: int32/uint32 [n_rays, 2] (updated in place); network_output fp16 [S, 16]; coords fp32 [S, 7];
    rgb_target fp32 [n_rays, 3].  Returns dict(counter, coords, dloss, loss)."""
    n_rays = numsteps.shape[0]
    dev_ = network_output.device
    _check_half(network_output, (network_output.shape[0], 16), "network_output")
    if coords.dtype != torch.float32 or tuple(coords.shape) != (network_output.shape[0], 7) or not coords.is_contiguous():
        raise N2Error("coords must be contiguous fp32 [S, 7]")
    if rgb_target.dtype != torch.float32 or tuple(rgb_target.shape) != (n_rays, 3) or not rgb_target.is_contiguous():
        raise N2Error("rgb_target must be contiguous fp32 [n_rays, 3]")
    if numsteps.dtype != torch.int32 or not numsteps.is_contiguous() or tuple(numsteps.shape) != (n_rays, 2):
        raise N2Error("numsteps must be contiguous int32 [n_rays, 2]")
    cfg = capi.CompositeConfig(loss_scale, ek_loss_weight, cos_anneal_ratio, (C.c_float * 3)(*background),
                               n_rays if n_rays_norm is None else n_rays_norm)
    nbytes = int(capi.lib().n2_composite_workspace_bytes(C.c_uint32(max(n_rays, 1))))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev_)
    counter = torch.zeros(1, dtype=torch.int32, device=dev_)
    cout = torch.zeros((max_samples_compacted, 7), dtype=torch.float32, device=dev_)
    dloss = torch.zeros((max_samples_compacted, 16), dtype=torch.float16, device=dev_)
    loss = torch.zeros(n_rays, dtype=torch.float32, device=dev_) if want_loss else None
    check(capi.lib().n2_composite_loss(_stream(), C.byref(cfg), C.c_uint32(n_rays), ptr(ray_counter), ptr(numsteps),
                                       ptr(network_output), ptr(coords), ptr(rgb_target),
                                       C.c_uint32(max_samples_compacted), ptr(counter), ptr(cout), ptr(dloss), ptr(loss),
                                       ptr(ws), C.c_uint64(nbytes)), "n2_composite_loss")
    return dict(counter=counter, coords=cout, dloss=dloss, loss=loss)


def fill_rollover(inout, n_in):
    """tcnn fill_rollover (fp32) / fill_rollover_and_rescale (fp16) on a [n_total, stride] tensor, in place;
    n_in is a device int32 scalar tensor (the compacted counter)."""
    n_total, stride = inout.shape[0], (inout.shape[1] if inout.dim() > 1 else 1)
    if inout.dtype == torch.float32:
        check(capi.lib().n2_fill_rollover_f32(_stream(), C.c_uint32(n_total), C.c_uint32(stride), ptr(n_in), ptr(inout)),
              "n2_fill_rollover_f32")
    elif inout.dtype == torch.float16:
        check(capi.lib().n2_fill_rollover_and_rescale_f16(_stream(), C.c_uint32(n_total), C.c_uint32(stride), ptr(n_in),
                                                          ptr(inout)), "n2_fill_rollover_and_rescale_f16")
    else:
        raise N2Error("fill_rollover supports float32 and float16")
    return inout


def pack_cameras(cams, device="cuda"):
    """List of dicts (xform[12], focal[2], principal[2], res[2], pixel_offset) -> device byte tensor of n2_camera."""
    arr = (capi.Camera * len(cams))()
    for a, c in zip(arr, cams):
        po = int(c["pixel_offset"])
        a.xform[:] = [float(v) for v in c["xform"]]
        a.focal_length[:] = [float(v) for v in c["focal"]]
        a.principal_point[:] = [float(v) for v in c["principal"]]
        a.resolution[:] = [int(v) for v in c["res"]]
        a.pixel_offset_lo, a.pixel_offset_hi = po & 0xFFFFFFFF, po >> 32
    raw = np.frombuffer(bytes(arr), dtype=np.uint8).copy()
    return torch.from_numpy(raw).to(device)


def generate_training_samples(n_rays, n_rays_total, seed, cameras, n_images, rgba, background, bitfield, max_samples):
    """generate_training_samples_nerf_with_global_movement (src/testbed_nerf.cu:1253-1446), static path.
    cameras: device byte tensor from pack_cameras; rgba fp32 [pixels, 4]; bitfield uint8 device tensor."""
    dev_ = rgba.device
    nbytes = int(capi.lib().n2_sampler_workspace_bytes(C.c_uint32(max(n_rays, 1))))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev_)
    out = dict(ray_counter=torch.zeros(1, dtype=torch.int32, device=dev_),
               sample_counter=torch.zeros(1, dtype=torch.int32, device=dev_),
               ray_indices=torch.zeros(n_rays, dtype=torch.int32, device=dev_),
               numsteps=torch.zeros((n_rays, 2), dtype=torch.int32, device=dev_),
               rgb_target=torch.zeros((n_rays, 3), dtype=torch.float32, device=dev_),
               coords=torch.zeros((max_samples, 7), dtype=torch.float32, device=dev_))
    bg = (C.c_float * 3)(*background)
    check(capi.lib().n2_generate_training_samples(_stream(), C.c_uint32(n_rays), C.c_uint32(n_rays_total), C.c_uint32(seed),
                                                  ptr(cameras), C.c_uint32(n_images), ptr(rgba), bg, ptr(bitfield),
                                                  C.c_uint32(max_samples), ptr(out["ray_counter"]),
                                                  ptr(out["sample_counter"]), ptr(out["ray_indices"]), ptr(out["numsteps"]),
                                                  ptr(out["rgb_target"]), ptr(out["coords"]), ptr(ws), C.c_uint64(nbytes)),
          "n2_generate_training_samples")
    return out
