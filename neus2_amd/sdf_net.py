"""The SDF network with its eikonal second-order path, composed from the encoding and the MLP the way
NerfNetwork does it (nerf_network.h:184-234 forward and normals, :402-429 first-order backward, :534-571
second-order backward), without the colour branch:

    input  = [x - 0.5 | grid(x) | 0]                (48 rows)
    sdf    = MLP(input)[0],   normal = d sdf / d x = dy_dx^T g[3:35] + g[0:3],  g = d sdf / d input
    loss   = mean |sdf| + w_ek * mean (|normal| - 1)^2

``loss_backward`` leaves d loss / d parameters (times loss_scale) in the gradient buffers of the two objects.
torch is used for the element-wise glue between the kernels only.
"""
import torch

from .tcnn_api import GRAD_ACCUMULATE, GRAD_OVERWRITE, FullyFusedMLP, GridEncoding


class SdfNet:
    def __init__(self, n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447, max_batch=1 << 18):
        self.grid = GridEncoding(n_levels, 2, log2_hashmap_size, base_resolution, per_level_scale)
        self.enc_w = 2 * n_levels
        self.in_w = (3 + self.enc_w + 15) // 16 * 16
        self.mlp = FullyFusedMLP(self.in_w, 1)
        self.grid.reserve_scatter_workspace(max_batch)

    def set_params(self, grid_params, grid_grads, mlp_params, mlp_grads):
        self.grid.set_params(grid_params, grid_grads)
        self.mlp.set_params(mlp_params, mlp_grads)

    def forward(self, x):
        """x fp32 [3, N].  Returns a context dict with sdf (fp16 [N]), normal (fp32 [3, N]) and what backward needs."""
        n = x.shape[1]
        inp = torch.zeros((self.in_w, n), dtype=torch.float16, device=x.device)
        inp[0:3] = x.half() - 0.5
        _, dy_dx = self.grid.forward(x, prepare_input_gradients=True, out=inp[3:3 + self.enc_w])
        y, _ = self.mlp.forward(inp)
        g = self.mlp.input_gradient(inp, 0)
        normal = torch.einsum("rnd,rn->dn", dy_dx, g[3:3 + self.enc_w].float()) + g[0:3].float()
        return dict(x=x, inp=inp, dy_dx=dy_dx, y=y, g=g, sdf=y[0], normal=normal)

    def loss_backward(self, ctx, ek_weight=0.1, loss_scale=128.0):
        x, inp, g, n = ctx["x"], ctx["inp"], ctx["g"], ctx["x"].shape[1]
        sdf, normal = ctx["sdf"].float(), ctx["normal"]
        norm = normal.norm(dim=0).clamp_min(1e-12)
        loss = sdf.abs().mean() + ek_weight * ((norm - 1) ** 2).mean()
        dL_dy = torch.zeros((16, n), dtype=torch.float16, device=x.device)
        dL_dy[0] = (torch.sign(sdf) * (loss_scale / n)).half()
        v = (normal * (2 * ek_weight * (norm - 1) / norm * (loss_scale / n))).contiguous()  # d loss / d normal
        # first order through the MLP, then both orders through the grid in one pass
        d_inp = self.mlp.backward(inp, dL_dy, want_input_grad=True, mode=GRAD_OVERWRITE)
        jv = self.grid.backward_fused(x, d_inp[3:3 + self.enc_w], v, g[3:3 + self.enc_w], want_dL_ddLdy=True, mode=GRAD_OVERWRITE)
        # second order through the MLP: its first-order output gradient was e_0
        v_in = torch.zeros_like(inp)
        v_in[0:3] = v.half()
        v_in[3:3 + self.enc_w] = jv
        self.mlp.backward_backward_input(inp, v_in, None, mode=GRAD_ACCUMULATE)
        return loss
