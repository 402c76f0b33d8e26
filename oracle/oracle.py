"""numpy/ctypes front end of the CPU oracle (test infrastructure only).

Only tests, ``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  The product package never does.

Every matrix is ``rows x N`` C-contiguous float32 (element (r, i) at r*N + i).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libneus2_oracle.so")
_lib = None

_f = C.POINTER(C.c_float)
_u = C.POINTER(C.c_uint32)


def build(force=False):
    """Compile the oracle with its Makefile (g++ -O3 -fopenmp)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL)
    else:
        subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_num_threads.restype = C.c_int
        _lib.orc_mlp_n_params.restype = C.c_uint32
    return _lib


def num_threads():
    return int(lib().orc_num_threads())


def _fp(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_f)


def _up(a):
    if a is None:
        return None
    assert a.dtype == np.uint32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_u)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Grid:
    """Level table + the grid functions of the oracle."""

    def __init__(self, n_levels=16, log2_hashmap_size=19, base_resolution=16, per_level_scale=1.447):
        self.n_levels = n_levels
        self.n_features = 2
        self.scale = np.zeros(n_levels, np.float32)
        self.resolution = np.zeros(n_levels, np.uint32)
        self.entries = np.zeros(n_levels, np.uint32)
        self.offset = np.zeros(n_levels + 1, np.uint32)
        lib().orc_grid_make_levels(C.c_uint32(n_levels), C.c_uint32(log2_hashmap_size), C.c_uint32(base_resolution),
                                   C.c_float(per_level_scale), _fp(self.scale), _up(self.resolution),
                                   _up(self.entries), _up(self.offset))
        self.n_params = int(self.offset[-1]) * 2
        self.n_out = n_levels * 2

    def _tab(self):
        return (C.c_uint32(self.n_levels), _fp(self.scale), _up(self.resolution), _up(self.entries))

    def indices(self, xyz):
        xyz = _f32(xyz)
        n = xyz.shape[1]
        idx = np.zeros((self.n_levels, 8, n), np.uint32)
        w = np.zeros((self.n_levels, 3, n), np.float32)
        lib().orc_grid_indices(*self._tab(), _fp(xyz), C.c_uint32(n), _up(idx), _fp(w))
        return idx, w

    def forward(self, params, xyz, want_dy_dx=False):
        params, xyz = _f32(params), _f32(xyz)
        n = xyz.shape[1]
        y = np.zeros((self.n_out, n), np.float32)
        j = np.zeros((self.n_out, n, 3), np.float32) if want_dy_dx else None
        lib().orc_grid_forward(*self._tab(), _up(self.offset), _fp(params), _fp(xyz), C.c_uint32(n), _fp(y), _fp(j))
        return (y, j) if want_dy_dx else y

    def backward(self, params, xyz, dL_dy, want_grad=True, want_dx=True):
        params, xyz, dL_dy = _f32(params), _f32(xyz), _f32(dL_dy)
        n = xyz.shape[1]
        grad = np.zeros(self.n_params, np.float32) if want_grad else None
        dx = np.zeros((3, n), np.float32) if want_dx else None
        lib().orc_grid_backward(*self._tab(), _up(self.offset), _fp(params), _fp(xyz), C.c_uint32(n), _fp(dL_dy),
                                _fp(grad), _fp(dx))
        return grad, dx

    def backward_backward_input(self, params, xyz, v, g, grad=None, want_dinput=True):
        """Returns (grad, dL_ddLdoutput, dL_dinput); ``grad`` is accumulated into when given."""
        params, xyz, v, g = _f32(params), _f32(xyz), _f32(v), _f32(g)
        n = xyz.shape[1]
        if grad is None:
            grad = np.zeros(self.n_params, np.float32)
        out = np.zeros((self.n_out, n), np.float32)
        din = np.zeros((3, n), np.float32) if want_dinput else None
        lib().orc_grid_backward_backward_input(*self._tab(), _up(self.offset), _fp(params), _fp(xyz), C.c_uint32(n),
                                               _fp(v), _fp(g), _fp(grad), _fp(out), _fp(din))
        return grad, out, din


def level_mask(n_levels, n_points, max_level=1.0, valid_levels=None, n_features=2):
    """bool [n_levels, n_points], True where a level is switched OFF.  tcnn's grid kernels (NVlabs tiny-cuda-nn
    include/tiny-cuda-nn/encodings/grid.h, kernel_grid: "max_level = (max_level * num_grid_features) /
    N_FEATURES_PER_LEVEL; if (level >= max_level + 1e-3f) -> zeros"), driven from src/testbed.cu:1861-1866 (global
    fraction) and src/testbed_nerf.cu:1305, 1440-1444, 3837-3843 (one fraction per point); ``valid_levels`` adds the
    progressive cut level >= valid_levels."""
    frac = np.broadcast_to(np.asarray(max_level, np.float32), (n_points,))
    limit = (frac * np.float32(n_levels * n_features)) / np.float32(n_features)
    lv = np.arange(n_levels, dtype=np.float32)[:, None]
    off = lv >= (limit[None, :] + np.float32(1e-3))
    if valid_levels is not None:
        off = off | (np.arange(n_levels)[:, None] >= valid_levels)
    return off


def progressive_levels(n_levels, base_valid_level_scale, valid_level_scale, base_training_step, step):
    """Levels in use at a training step under the encoding keys of configs/nerf/base.json:36-38.  PARITY UNPINNED:
    the arithmetic is in the tcnn fork the reference tree does not hold; this is the reading this build adopted
    (fraction = base + scale * (step // base_training_step), floor(fraction * n_levels + 1e-3) clamped to
    [1, n_levels]; the 1e-3 keeps a fraction that reaches 1 up to rounding from losing the last level)."""
    if base_training_step == 0:
        return n_levels
    frac = np.float32(base_valid_level_scale) + np.float32(valid_level_scale) * np.float32(step // base_training_step)
    lv = np.float32(frac) * np.float32(n_levels) + np.float32(1e-3)
    return int(min(n_levels, max(1, int(np.floor(lv))))) if lv < n_levels else n_levels


class Mlp:
    def __init__(self, in_width, width, n_hidden, out_width):
        self.in_w, self.width, self.n_hidden, self.out_w = in_width, width, n_hidden, out_width
        self.n_params = int(lib().orc_mlp_n_params(in_width, width, n_hidden, out_width))

    def _d(self):
        return (C.c_uint32(self.in_w), C.c_uint32(self.width), C.c_uint32(self.n_hidden), C.c_uint32(self.out_w))

    def layer_shapes(self):
        s = [(self.width, self.in_w)] + [(self.width, self.width)] * (self.n_hidden - 1) + [(self.out_w, self.width)]
        return s

    def split(self, W):
        out, o = [], 0
        for r, c in self.layer_shapes():
            out.append(np.asarray(W[o:o + r * c]).reshape(r, c))
            o += r * c
        return out

    def forward(self, W, x, round_hidden=False):
        """round_hidden: keep hidden activations at fp16 precision between layers (reference storage type)."""
        W, x = _f32(W), _f32(x)
        n = x.shape[1]
        y = np.zeros((self.out_w, n), np.float32)
        h = np.zeros((self.n_hidden, self.width, n), np.float32)
        lib().orc_mlp_forward(*self._d(), _fp(W), _fp(x), C.c_uint32(n), _fp(y), _fp(h), C.c_int(int(round_hidden)))
        return y, h

    def backward(self, W, x, hidden, dL_dy, want_dx=True, want_dW=True):
        W, x, hidden, dL_dy = _f32(W), _f32(x), _f32(hidden), _f32(dL_dy)
        n = x.shape[1]
        dx = np.zeros((self.in_w, n), np.float32) if want_dx else None
        dW = np.zeros(self.n_params, np.float32) if want_dW else None
        lib().orc_mlp_backward(*self._d(), _fp(W), _fp(x), _fp(hidden), _fp(dL_dy), C.c_uint32(n), _fp(dx), _fp(dW))
        return dx, dW

    def backward_backward_input(self, W, hidden, v, g, dW=None):
        W, hidden, v, g = _f32(W), _f32(hidden), _f32(v), _f32(g)
        n = v.shape[1]
        if dW is None:
            dW = np.zeros(self.n_params, np.float32)
        out = np.zeros((self.out_w, n), np.float32)
        lib().orc_mlp_backward_backward_input(*self._d(), _fp(W), _fp(hidden), _fp(v), _fp(g), C.c_uint32(n),
                                              _fp(dW), _fp(out))
        return dW, out


def round_fp16(a):
    a = _f32(a)
    out = np.empty_like(a)
    lib().orc_round_fp16(_fp(a), _fp(out), C.c_uint32(a.size))
    return out


def sh4(dirs):
    dirs = _f32(dirs)
    n = dirs.shape[1]
    out = np.zeros((16, n), np.float32)
    lib().orc_sh4(_fp(dirs), C.c_uint32(n), _fp(out))
    return out


def adam_step(w, grad, m1, m2, steps, n_matrix_params, loss_scale=128.0, lr=1e-3, beta1=0.9, beta2=0.99,
              eps=1e-15, l2_reg=1e-6):
    """In place on w, m1, m2 (float32) and steps (uint32)."""
    grad = _f32(grad)
    for a in (w, m1, m2):
        assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    lib().orc_adam_step(C.c_uint32(w.size), C.c_uint32(n_matrix_params), C.c_float(loss_scale), C.c_float(lr),
                        C.c_float(beta1), C.c_float(beta2), C.c_float(eps), C.c_float(l2_reg), _fp(w), _fp(grad),
                        _fp(m1), _fp(m2), _up(steps))


class CompositeCfg(C.Structure):
    _fields_ = [("loss_scale", C.c_float), ("ek_loss_weight", C.c_float), ("cos_anneal_ratio", C.c_float),
                ("background", C.c_float * 3), ("n_rays_norm", C.c_uint32), ("min_step", C.c_float),
                ("max_step", C.c_float), ("exact_inv_s", C.c_int)]


MIN_STEP = float(np.float32(1.73205080757) / np.float32(1024))  # STEPSIZE(), src/testbed_nerf.cu:51-53
MAX_STEP = float(np.float32(MIN_STEP) * np.float32(128))        # * 2^(NERF_CASCADES-1)


def composite_loss(numsteps, net_out, coords, rgb_target, max_compacted, n_rays_norm=None, loss_scale=128.0,
                   ek_loss_weight=0.01, cos_anneal_ratio=1.0, background=(0.0, 0.0, 0.0), exact_inv_s=False):
    """numsteps [n_rays, 2] uint32 (count, base); net_out [S, 16]; coords [S, 7]; rgb_target [n_rays, 3].
    Returns dict(numsteps, dloss [max_compacted,16], coords [max_compacted,7], loss [n_rays], counter, rgb_ray)."""
    numsteps = np.ascontiguousarray(numsteps, np.uint32).copy()
    n_rays = numsteps.shape[0]
    net_out, coords, rgb_target = _f32(net_out), _f32(coords), _f32(rgb_target)
    cfg = CompositeCfg(loss_scale, ek_loss_weight, cos_anneal_ratio, (C.c_float * 3)(*background),
                       n_rays if n_rays_norm is None else n_rays_norm, MIN_STEP, MAX_STEP, int(exact_inv_s))
    dloss = np.zeros((max_compacted, 16), np.float32)
    cout = np.zeros((max_compacted, 7), np.float32)
    loss = np.zeros(n_rays, np.float32)
    rgb_ray = np.zeros((n_rays, 3), np.float32)
    counter = C.c_uint32(0)
    lib().orc_composite_loss(C.byref(cfg), C.c_uint32(n_rays), _up(numsteps), _fp(net_out), _fp(coords), _fp(rgb_target),
                             C.c_uint32(max_compacted), _fp(dloss), _fp(cout), _fp(loss), C.byref(counter), _fp(rgb_ray))
    return dict(numsteps=numsteps, dloss=dloss, coords=cout, loss=loss, counter=int(counter.value), rgb_ray=rgb_ray)


def fill_rollover(a, n_in, rescale=False):
    """a: [n_total, stride] float32, in place."""
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    lib().orc_fill_rollover(C.c_uint32(a.shape[0]), C.c_uint32(a.shape[1] if a.ndim > 1 else 1), C.c_uint32(n_in), _fp(a),
                            C.c_int(int(rescale)))
    return a


class Camera(C.Structure):
    """Matches struct n2_camera of the product ABI."""
    _fields_ = [("xform", C.c_float * 12), ("focal", C.c_float * 2), ("principal", C.c_float * 2),
                ("res", C.c_uint32 * 2), ("pixel_offset_lo", C.c_uint32), ("pixel_offset_hi", C.c_uint32)]


def morton3d(x, y, z):
    lib().orc_morton3d.restype = C.c_uint32
    return int(lib().orc_morton3d(C.c_uint32(x), C.c_uint32(y), C.c_uint32(z)))


def morton3d_invert(m):
    out = (C.c_uint32 * 3)()
    lib().orc_morton3d_invert(C.c_uint32(m), out)
    return tuple(out)


def generate_training_samples(n_rays, n_rays_total, seed, cameras, rgba, background, bitfield, max_samples):
    """cameras: numpy structured bytes (n_images * sizeof(Camera)) or list of Camera; rgba [pixels, 4] float32;
    bitfield uint8 [128^3/8].  Returns dict(ray_counter, sample_counter, ray_indices, numsteps, rgb_target, coords)."""
    cams = (Camera * len(cameras))(*cameras)
    rgba = _f32(rgba)
    bg = (C.c_float * 3)(*background)
    bitfield = np.ascontiguousarray(bitfield, np.uint8)
    ray_counter, sample_counter = C.c_uint32(0), C.c_uint32(0)
    ray_indices = np.zeros(n_rays, np.uint32)
    numsteps = np.zeros((n_rays, 2), np.uint32)
    target = np.zeros((n_rays, 3), np.float32)
    coords = np.zeros((max_samples, 7), np.float32)
    lib().orc_generate_training_samples(C.c_uint32(n_rays), C.c_uint32(n_rays_total), C.c_uint32(seed), cams,
                                        C.c_uint32(len(cameras)), _fp(rgba), bg,
                                        bitfield.ctypes.data_as(C.POINTER(C.c_uint8)), C.c_uint32(max_samples),
                                        C.byref(ray_counter), C.byref(sample_counter), _up(ray_indices), _up(numsteps),
                                        _fp(target), _fp(coords))
    return dict(ray_counter=int(ray_counter.value), sample_counter=int(sample_counter.value), ray_indices=ray_indices,
                numsteps=numsteps, rgb_target=target, coords=coords)


# ---------------------------------------------------------------------------
# occupancy-grid update (src/testbed_nerf.cu:3286-3391)
# ---------------------------------------------------------------------------
_u64 = C.POINTER(C.c_uint64)
GRID_CELLS = 128 ** 3
MIN_OPTICAL_THICKNESS = 0.1  # NERF_MIN_OPTICAL_THICKNESS() with SDF_GRID 0, src/testbed_nerf.cu:39, 65


class Pcg32:
    """Published PCG32 in the form tiny-cuda-nn ships (pcg32(initstate, initseq = 1))."""

    def __init__(self, initstate=None, initseq=1):
        self.s = np.zeros(2, np.uint64)
        if initstate is None:  # default-constructed generator
            self.s[0], self.s[1] = 0x853c49e6748fea9b, 0xda3e39cb94b95bdb
        else:
            lib().orc_pcg32_seed(C.c_uint64(initstate), C.c_uint64(initseq), self.s.ctypes.data_as(_u64))

    def copy(self):
        r = Pcg32()
        r.s[:] = self.s
        return r

    def next_uints(self, n, skip=0):
        out = np.zeros(n, np.uint32)
        lib().orc_pcg32_draw(self.s.ctypes.data_as(_u64), C.c_uint64(skip), C.c_uint32(n), _up(out), None)
        return out

    def next_floats(self, n, skip=0):
        out = np.zeros(n, np.float32)
        lib().orc_pcg32_draw(self.s.ctypes.data_as(_u64), C.c_uint64(skip), C.c_uint32(n), None, _fp(out))
        return out

    def advance(self, delta=1 << 32):
        lib().orc_pcg32_advance(self.s.ctypes.data_as(_u64), C.c_uint64(delta))


def generate_grid_samples(n, rng, step, grid, n_cascades, thresh):
    """generate_grid_samples_nerf_nonuniform: positions [n, 3] and cell indices [n] (rng is taken by value)."""
    grid = _f32(grid)
    pos, idx = np.zeros((n, 3), np.float32), np.zeros(n, np.uint32)
    if n:
        lib().orc_generate_grid_samples(C.c_uint32(n), rng.s.ctypes.data_as(_u64), C.c_uint32(step), _fp(grid), C.c_uint32(n_cascades),
                                        C.c_float(thresh), _fp(pos), _up(idx))
    return pos, idx


def splat_grid_max(indices, density, grid_tmp):
    density = _f32(density)
    lib().orc_splat_grid_max(C.c_uint32(len(indices)), _up(indices), _fp(density), _fp(grid_tmp))


def ema_grid(grid, grid_tmp, decay):
    lib().orc_ema_grid(C.c_uint32(grid.size), C.c_float(decay), _fp(grid), _fp(grid_tmp))


def grid_mean(grid):
    lib().orc_grid_mean.restype = C.c_float
    return float(lib().orc_grid_mean(_fp(grid)))


def grid_to_bitfield(grid, n_cascades, mean):
    bits = np.zeros(8 * GRID_CELLS // 8, np.uint8)
    lib().orc_grid_to_bitfield(_fp(grid), C.c_uint32(n_cascades), C.c_float(mean), C.c_float(MIN_OPTICAL_THICKNESS),
                               bits.ctypes.data_as(C.POINTER(C.c_uint8)))
    return bits


class OccupancyGrid:
    """State and update of the density grid: Testbed::update_density_grid_nerf + update_density_grid_mean_and_bitfield.
    ``density_fn(xyz [3, n]) -> [n]`` stands for NerfNetwork::density."""

    def __init__(self, n_cascades=1, seed=1337):
        self.n_cascades = n_cascades
        self.grid = np.zeros(n_cascades * GRID_CELLS, np.float32)
        self.rng = Pcg32(seed)
        self.ema_step = 0
        self.mean = 0.0
        self.bitfield = np.zeros(GRID_CELLS, np.uint8)

    def update(self, density_fn, decay, n_uniform, n_nonuniform, chunk=1 << 18):
        tmp = np.zeros_like(self.grid)
        p0, i0 = generate_grid_samples(n_uniform, self.rng, self.ema_step, self.grid, self.n_cascades, -0.01)
        self.rng.advance()
        p1, i1 = generate_grid_samples(n_nonuniform, self.rng, self.ema_step, self.grid, self.n_cascades, MIN_OPTICAL_THICKNESS)
        self.rng.advance()
        pos, idx = np.concatenate([p0, p1]), np.concatenate([i0, i1])
        dens = np.concatenate([density_fn(np.ascontiguousarray(pos[a:a + chunk].T)) for a in range(0, len(pos), chunk)]) \
            if len(pos) else np.zeros(0, np.float32)
        splat_grid_max(idx, dens, tmp)
        ema_grid(self.grid, tmp, decay)
        self.ema_step += 1
        self.mean = grid_mean(self.grid)
        self.bitfield = grid_to_bitfield(self.grid, self.n_cascades, self.mean)
        return dict(positions=pos, indices=idx, density=dens, tmp=tmp)


# ---------------------------------------------------------------------------
# optimizer wrappers (configs/nerf/base.json:5-13)
# ---------------------------------------------------------------------------
def ema_step(weights16, tmp, step, decay=0.95):
    """One Ema step after nested step ``step`` (1-based); tmp (float32) is updated in place, returns the fp16-rounded EMA."""
    weights16 = _f32(weights16)
    out = np.zeros_like(weights16)
    lib().orc_ema_step(C.c_uint32(weights16.size), C.c_float(decay), C.c_uint32(step), _fp(weights16), _fp(tmp), _fp(out))
    return out


def exponential_decay_lr(base_lr, steps_done, decay_start=20000, decay_interval=10000, decay_base=0.33):
    lib().orc_exponential_decay_lr.restype = C.c_float
    return float(lib().orc_exponential_decay_lr(C.c_float(base_lr), C.c_uint32(decay_start), C.c_uint32(decay_interval),
                                                C.c_float(decay_base), C.c_uint32(steps_done)))


# ---------------------------------------------------------------------------
# training images (src/nerf_loader.cu:59-81, common_device.cuh:31-37, 635-655)
# ---------------------------------------------------------------------------
def srgb_to_linear(c):
    c = np.asarray(c, np.float32)
    with np.errstate(invalid="ignore"):
        return np.where(c <= np.float32(0.04045), c / np.float32(12.92),
                        np.power((c + np.float32(0.055)) / np.float32(1.055), np.float32(2.4))).astype(np.float32)


def convert_rgba8(rgba8, white_transparent=False, black_transparent=False, mask_color=0):
    """uint8 [n, 4] -> float32 [n, 4]: convert_rgba32's transparency rules, then read_rgba's Byte branch."""
    px = np.ascontiguousarray(rgba8, np.uint8).reshape(-1, 4).copy()
    rgb = px[:, :3]
    if white_transparent:
        px[(rgb == 255).all(1), 3] = 0
    if black_transparent:
        px[(rgb == 0).all(1), 3] = 0
    word = px.view(np.uint32).ravel()
    masked = word == np.uint32(0x00FF00FF)
    if mask_color:
        masked |= word == np.uint32(mask_color)
    a = px[:, 3].astype(np.float32) * np.float32(1.0 / 255.0)
    lin = srgb_to_linear(px[:, :3].astype(np.float32) * np.float32(1.0 / 255.0))
    out = np.concatenate([lin * a[:, None], a[:, None]], 1).astype(np.float32)
    out[masked] = -1.0
    return out
