"""The SDF network with its eikonal second-order path, composed from the encoding and the MLP the way
NerfNetwork does it (nerf_network.h:184-234 forward and normals, :402-429 first-order backward, :534-571
second-order backward), without the colour branch:

    input  = [x - 0.5 | grid(x) | 0]                (48 rows)
    sdf    = MLP(input)[0],   normal = d sdf / d x = dy_dx^T g[3:35] + g[0:3],  g = d sdf / d input
    loss   = mean |sdf| + w_ek * mean (|normal| - 1)^2

``loss_backward`` leaves d loss / d parameters (times loss_scale) in the gradient buffers of the two objects.
Every arithmetic step runs in the library; torch only owns the buffers,
which are allocated once per batch size.
"""
import ctypes as C

import torch

from . import capi
from .capi import check, ptr
from .tcnn_api import GRAD_ACCUMULATE, GRAD_IGNORE, GRAD_OVERWRITE, LAYOUT_SOA, FullyFusedMLP, GridEncoding


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class SdfNet:
    def __init__(self, n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447, max_batch=1 << 18):
        self.grid = GridEncoding(n_levels, 2, log2_hashmap_size, base_resolution, per_level_scale)
        self.enc_w = 2 * n_levels
        self.in_w = (3 + self.enc_w + 15) // 16 * 16
        self.mlp = FullyFusedMLP(self.in_w, 1)
        self.grid.reserve_scatter_workspace(max_batch)
        self._n = 0

    def set_params(self, grid_params, grid_grads, mlp_params, mlp_grads):
        self.grid.set_params(grid_params, grid_grads)
        self.mlp.set_params(mlp_params, mlp_grads)

    def _buffers(self, n, device):
        if n != self._n:
            h = lambda rows: torch.empty((rows, n), dtype=torch.float16, device=device)
            f = lambda rows: torch.empty((rows, n), dtype=torch.float32, device=device)
            self._inp, self._g, self._y, self._dL_dy, self._v_in, self._d_inp = h(self.in_w), h(self.in_w), h(16), h(16), h(self.in_w), h(self.in_w)
            self._dy_dx = torch.empty((self.enc_w, n, 3), dtype=torch.float32, device=device)
            self._normal_enc, self._normal, self._v = f(3), f(3), f(3)
            self._loss = torch.empty(1, dtype=torch.float32, device=device)
            nb = int(capi.lib().n2_sdf_eikonal_workspace_bytes(C.c_uint32(n)))
            self._ws = torch.empty(nb, dtype=torch.uint8, device=device)
            self._ws_bytes = nb
            self._n = n

    def forward(self, x, ek_weight=0.1, loss_scale=128.0):
        """x fp32 [3, N].  Returns a context dict with sdf (fp16 [N]), normal (fp32 [3, N]), the loss (one-element device
        tensor) and what backward needs.  The tensors are the net's own buffers: they are overwritten by the next
        forward of the same batch size."""
        L, s = capi.lib(), _stream()
        n = x.shape[1]
        self._buffers(n, x.device)
        inp, g, y = self._inp, self._g, self._y
        check(L.n2_sdf_pack_input(s, ptr(x), C.c_uint32(1), C.c_uint32(n), C.c_uint32(n), C.c_uint32(self.enc_w), C.c_uint32(self.in_w), ptr(inp)),
              "n2_sdf_pack_input")
        enc = inp[3:3 + self.enc_w]
        check(L.n2_grid_forward(self.grid._h, s, ptr(x), C.c_uint32(1), C.c_uint32(n), C.c_uint32(n), ptr(enc), ptr(self._dy_dx)), "n2_grid_forward")
        check(L.n2_mlp_forward_and_input_gradient(self.mlp._h, s, C.c_uint32(0), ptr(inp), C.c_uint32(n), ptr(y), C.c_int(LAYOUT_SOA), ptr(g)),
              "n2_mlp_forward_and_input_gradient")
        # encoding backward of d sdf / d encoding without parameter gradients: J^T g (nerf_network.h:230-234)
        check(L.n2_grid_backward(self.grid._h, s, ptr(x), C.c_uint32(1), C.c_uint32(n), C.c_uint32(n), ptr(g[3:3 + self.enc_w]), ptr(self._dy_dx),
                                 ptr(self._normal_enc), C.c_int(GRAD_IGNORE)), "n2_grid_backward")
        ctx = dict(x=x, inp=inp, dy_dx=self._dy_dx, y=y, g=g, sdf=y[0], normal=self._normal, loss=self._loss)
        self._eikonal(ctx, ek_weight, loss_scale)
        return ctx

    def _eikonal(self, ctx, ek_weight, loss_scale):
        n = ctx["x"].shape[1]
        check(capi.lib().n2_sdf_eikonal_loss(_stream(), C.c_uint32(n), C.c_uint32(self.enc_w), C.c_uint32(self.in_w), ptr(ctx["y"]), ptr(ctx["g"]),
                                             ptr(self._normal_enc), ptr(self._normal), C.c_float(ek_weight), C.c_float(loss_scale), ptr(self._dL_dy),
                                             ptr(self._v), ptr(self._v_in), ptr(self._loss), ptr(self._ws), C.c_uint64(self._ws_bytes),
                                             ptr(ctx["dy_dx"])),
              "n2_sdf_eikonal_loss")
        ctx["weights"] = (ek_weight, loss_scale)

    def loss_backward(self, ctx, ek_weight=0.1, loss_scale=128.0):
        """Returns the loss as a one-element device tensor (no host synchronisation)."""
        L, s = capi.lib(), _stream()
        x, inp, g, n = ctx["x"], ctx["inp"], ctx["g"], ctx["x"].shape[1]
        if ctx["weights"] != (ek_weight, loss_scale):
            self._eikonal(ctx, ek_weight, loss_scale)
        # first order through the MLP, then both orders through the grid in one pass; the grid's dL_ddLdoutput (rows 3.. of
        # the MLP's second-order input) was already formed from the saved Jacobian by n2_sdf_eikonal_loss
        check(L.n2_mlp_backward(self.mlp._h, s, ptr(inp), C.c_uint32(n), ptr(self._dL_dy), C.c_int(LAYOUT_SOA), ptr(self._d_inp), C.c_int(GRAD_OVERWRITE)),
              "n2_mlp_backward")
        check(L.n2_grid_backward_fused(self.grid._h, s, ptr(x), C.c_uint32(1), C.c_uint32(n), C.c_uint32(n), ptr(self._d_inp[3:3 + self.enc_w]),
                                       ptr(self._v), ptr(g[3:3 + self.enc_w]), None, C.c_int(GRAD_OVERWRITE)),
              "n2_grid_backward_fused")
        # second order through the MLP: its first-order output gradient was e_0
        check(L.n2_mlp_backward_backward_input(self.mlp._h, s, ptr(inp), C.c_uint32(n), ptr(self._v_in), None, None, C.c_int(GRAD_ACCUMULATE)),
              "n2_mlp_backward_backward_input")
        return self._loss
