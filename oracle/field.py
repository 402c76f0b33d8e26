"""CPU oracle of the NeuS field: the composition NerfNetwork<T> performs around the
grid encoding and the two MLPs (include/neural-graphics-primitives/nerf_network.h).

TEST INFRASTRUCTURE ONLY (see oracle/neus2_oracle.cpp).  Static scene: the delta
network is off (m_use_delta = false, src/testbed.cu:2695-2697).

Pinned by tests/test_oracle_field.py: torch autograd (with create_graph for the
normals) of an independent fp64 forward reproduces every parameter gradient this
module assembles from first- and second-order pieces.

With ``fp16=True`` every buffer the reference stores as __half is rounded to
fp16 at the point where the reference stores it; the arithmetic in between stays
fp32.  With ``fp16=False`` nothing is rounded (used for the autograd pin).
"""
import numpy as np

from . import oracle as orc


class Field:
    """Parameter order (nerf_network.h:728-772): [SDF MLP | colour MLP | grid | variance(4)]."""

    def __init__(self, n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447,
                 sdf_bias=-0.1, fp16=True):
        self.grid = orc.Grid(n_levels, log2_hashmap_size, base_resolution, per_level_scale)
        self.enc_w = self.grid.n_out
        # next_multiple(3 + enc, 16), nerf_network.h:41-47
        self.sdf_in_w = (3 + self.enc_w + 15) // 16 * 16
        self.sdf = orc.Mlp(self.sdf_in_w, 64, 1, 16)
        # next_multiple(3 + 3 + 16 + 16, 16), nerf_network.h:60
        self.rgb_in_w = 48
        self.rgb = orc.Mlp(self.rgb_in_w, 64, 2, 16)
        self.sdf_bias = np.float32(sdf_bias)
        self.fp16 = fp16
        self.off_sdf = 0
        self.off_rgb = self.sdf.n_params
        self.off_grid = self.off_rgb + self.rgb.n_params
        self.off_var = self.off_grid + self.grid.n_params
        self.n_params = self.off_var + 4
        self.n_matrix_params = self.off_grid  # what Adam's l2_reg / zero-skip rules key on

    def q(self, a):
        a = np.asarray(a, np.float32)
        return orc.round_fp16(a) if self.fp16 else a

    def split(self, params):
        p = np.asarray(params, np.float32)
        return (p[self.off_sdf:self.off_rgb], p[self.off_rgb:self.off_grid], p[self.off_grid:self.off_var],
                p[self.off_var:self.off_var + 4])

    # nerf_network.h:132-315
    def forward(self, params, coords):
        """coords: [N, 7] float32 rows (x y z dt dx dy dz), nerf.h:76-102.
        Returns (output [16, N], ctx)."""
        Ws, Wr, G, var = self.split(params)
        coords = np.asarray(coords, np.float32)
        n = coords.shape[0]
        xyz = np.ascontiguousarray(coords[:, 0:3].T)
        dirs = np.ascontiguousarray(coords[:, 4:7].T)
        enc, dy_dx = self.grid.forward(G, xyz, want_dy_dx=True)
        sdf_in = np.zeros((self.sdf_in_w, n), np.float32)
        # fill_positions_view_with_fixed_offset: (T)pos - (T)0.5, common_operation.cuh:186-199
        sdf_in[0:3] = self.q(self.q(xyz) - np.float32(0.5))
        sdf_in[3:3 + self.enc_w] = self.q(enc)
        sdf_out, h_sdf = self.sdf.forward(Ws, sdf_in, round_hidden=self.fp16)
        sdf_out = self.q(sdf_out)
        # normals inside the forward: backward of e_0 through MLP and grid, :215-240
        e0 = np.zeros((16, n), np.float32)
        e0[0] = 1
        dsdf_din, _ = self.sdf.backward(Ws, sdf_in, h_sdf, e0, want_dW=False)
        dsdf_din = self.q(dsdf_din)
        g_enc = np.ascontiguousarray(dsdf_din[3:3 + self.enc_w])
        normal = np.einsum("kn,knd->dn", g_enc, dy_dx).astype(np.float32)
        normal = normal + dsdf_din[0:3]  # add_positions_view<float, T>, :236-238
        rgb_in = np.zeros((self.rgb_in_w, n), np.float32)
        rgb_in[0:16] = sdf_out
        rgb_in[16:32] = self.q(orc.sh4(dirs))
        rgb_in[32:35] = self.q(xyz)
        rgb_in[35:38] = self.q(normal)
        rgb_out, h_rgb = self.rgb.forward(Wr, rgb_in, round_hidden=self.fp16)
        out = self.q(rgb_out)
        out[3] = self.q(sdf_out[0] + self.q(self.sdf_bias))  # extract_sdf_value_view_with_bias
        out[4:7] = self.q(normal)
        out[7] = self.q(var[0])
        out[8:11] = self.q(dirs)
        ctx = dict(xyz=xyz, dirs=dirs, sdf_in=sdf_in, h_sdf=h_sdf, rgb_in=rgb_in, h_rgb=h_rgb, g_enc=g_enc,
                   normal=normal, n=n)
        return out, ctx

    # nerf_network.h:317-588
    def backward(self, params, ctx, dL_dout, ek_batch_size=None):
        """dL_dout: [16, N].  Returns the full gradient vector (n_params,) in Overwrite mode."""
        Ws, Wr, G, var = self.split(params)
        n = ctx["n"]
        if ek_batch_size is None:
            ek_batch_size = n
        dL_dout = np.asarray(dL_dout, np.float32)
        grad = np.zeros(self.n_params, np.float32)
        # colour net: only rows 0..2 carry gradient (extract_rgb), :332-340
        dL_drgb = np.zeros((16, n), np.float32)
        dL_drgb[0:3] = dL_dout[0:3]
        d_rgb_in, dWr = self.rgb.backward(Wr, ctx["rgb_in"], ctx["h_rgb"], dL_drgb)
        d_rgb_in = self.q(d_rgb_in)
        grad[self.off_rgb:self.off_grid] = dWr
        # SDF net: colour-net input gradient rows 0..15, plus dL/dsdf on row 0, :388-402
        d_sdf_out = d_rgb_in[0:16].copy()
        d_sdf_out[0] = self.q(d_sdf_out[0] + dL_dout[3])
        d_sdf_in, dWs = self.sdf.backward(Ws, ctx["sdf_in"], ctx["h_sdf"], d_sdf_out)
        d_sdf_in = self.q(d_sdf_in)
        grad[self.off_sdf:self.off_rgb] = dWs
        # grid first order, :410-429
        gG, _ = self.grid.backward(G, ctx["xyz"], np.ascontiguousarray(d_sdf_in[3:3 + self.enc_w]), want_dx=False)
        # variance: plain sum of row 7, :447-461
        grad[self.off_var] = np.float32(dL_dout[7].astype(np.float64).sum())
        # dL/dnormal: colour-net input rows 35..37 + eikonal rows 4..6 / batch + cos rows 8..10, :464-491
        v = (d_rgb_in[35:38] + dL_dout[4:7] / np.float32(ek_batch_size) + dL_dout[8:11]).astype(np.float32)
        # second order through the grid (Accumulate), :529-544
        gG, pos_enc_dy, _ = self.grid.backward_backward_input(G, ctx["xyz"], v, ctx["g_enc"], grad=gG,
                                                                want_dinput=False)
        grad[self.off_grid:self.off_var] = gG
        # second order through the SDF MLP (Accumulate), :546-571
        d_density_input = np.zeros((self.sdf_in_w, n), np.float32)
        d_density_input[0:3] = self.q(v)
        d_density_input[3:3 + self.enc_w] = self.q(pos_enc_dy)
        e0 = np.zeros((16, n), np.float32)
        e0[0] = 1
        dWs2, _ = self.sdf.backward_backward_input(Ws, ctx["h_sdf"], d_density_input, e0)
        grad[self.off_sdf:self.off_rgb] += dWs2
        return grad

    # nerf_network.h:643-709
    def sdf_values(self, params, xyz):
        """xyz [3, N] -> [16, N] SDF-net output with the bias added on row 0."""
        Ws, _, G, _ = self.split(params)
        xyz = np.asarray(xyz, np.float32)
        n = xyz.shape[1]
        sdf_in = np.zeros((self.sdf_in_w, n), np.float32)
        sdf_in[0:3] = self.q(self.q(xyz) - np.float32(0.5))
        sdf_in[3:3 + self.enc_w] = self.q(self.grid.forward(G, xyz))
        out, _ = self.sdf.forward(Ws, sdf_in, round_hidden=self.fp16)
        out = self.q(out)
        out[0] = self.q(out[0] + self.q(self.sdf_bias))
        return out

    # nerf_network.h:711-726 + common_operation.cuh:310-328
    def density(self, params, xyz):
        out = self.sdf_values(params, xyz)
        var = self.q(self.split(params)[3][0])
        s = self.q(np.exp(self.q(var * np.float32(10.0))))
        sig = self.q(1.0 / (1.0 + np.exp(-self.q(out[0] * s))))
        out[0] = self.q(s * sig * (np.float32(1.0) - sig))
        return out
