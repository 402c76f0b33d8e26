"""Synthetic scene used by the benchmark and the tests: an analytic sphere, Lambertian-textured,
seen by pinhole cameras on a sphere around it, plus the 128^3 morton-ordered occupancy bitfield
of a band around its surface.  numpy only; stands in for the dataset loader (out of scope)."""
import numpy as np

GRIDSIZE = 128  # NERF_GRIDSIZE, include/neural-graphics-primitives/nerf.h:24-26


def _expand_bits(v):
    v = v.astype(np.uint32)
    v = (v * np.uint32(0x00010001)) & np.uint32(0xFF0000FF)
    v = (v * np.uint32(0x00000101)) & np.uint32(0x0F00F00F)
    v = (v * np.uint32(0x00000011)) & np.uint32(0xC30C30C3)
    v = (v * np.uint32(0x00000005)) & np.uint32(0x49249249)
    return v


def morton3d(x, y, z):
    with np.errstate(over="ignore"):
        return _expand_bits(x) | (_expand_bits(y) << np.uint32(1)) | (_expand_bits(z) << np.uint32(2))


def sphere_bitfield(radius=0.3, band=0.03, center=(0.5, 0.5, 0.5), n_mips=8):
    """Occupancy bitfield (grid_to_bitfield format, src/testbed_nerf.cu:738-759): bit idx%8 of byte idx/8 with
    idx = morton3D(x, y, z); a cell is occupied when its centre is within `band` of the sphere surface.
    All 8 mip levels are allocated (grid_mip_offset(mip)/8), only mip 0 is filled: the unit cube reads no other."""
    g = (np.arange(GRIDSIZE) + 0.5) / GRIDSIZE
    z, y, x = np.meshgrid(g, g, g, indexing="ij")
    d = np.sqrt((x - center[0]) ** 2 + (y - center[1]) ** 2 + (z - center[2]) ** 2)
    occ = np.abs(d - radius) <= band
    iz, iy, ix = np.nonzero(occ)
    idx = morton3d(ix, iy, iz)
    bits = np.zeros(GRIDSIZE ** 3 // 8 * n_mips, np.uint8)
    np.bitwise_or.at(bits, idx // 8, (1 << (idx % 8)).astype(np.uint8))
    return bits


def cameras_on_sphere(n_cameras=64, resolution=512, cam_radius=2.0, fov_deg=25.0, center=(0.5, 0.5, 0.5)):
    """Pinhole cameras on a Fibonacci sphere looking at the centre.  Returns a list of dicts with the fields of
    struct n2_camera: xform (3x4 row-major camera-to-world, +z forward), focal, principal, res, pixel_offset."""
    cams = []
    c = np.asarray(center, np.float64)
    focal = 0.5 * resolution / np.tan(0.5 * np.deg2rad(fov_deg))
    for k in range(n_cameras):
        zc = 1 - 2 * (k + 0.5) / n_cameras
        r = np.sqrt(max(0.0, 1 - zc * zc))
        phi = k * np.pi * (3 - np.sqrt(5))
        pos = c + cam_radius * np.array([r * np.cos(phi), r * np.sin(phi), zc])
        fwd = (c - pos) / np.linalg.norm(c - pos)
        up = np.array([0.0, 0.0, 1.0]) if abs(fwd[2]) < 0.99 else np.array([0.0, 1.0, 0.0])
        right = np.cross(fwd, up)
        right /= np.linalg.norm(right)
        down = np.cross(fwd, right)
        xform = np.stack([right, down, fwd, pos], axis=1).astype(np.float32)  # columns
        cams.append(dict(xform=xform.reshape(-1), focal=(np.float32(focal),) * 2, principal=(0.5, 0.5),
                         res=(resolution, resolution), pixel_offset=k * resolution * resolution))
    return cams


def render_sphere_images(cams, radius=0.3, center=(0.5, 0.5, 0.5), light=(0.3, 0.5, 0.8)):
    """Analytic render: RGBA float32 [n_images*H*W, 4], premultiplied alpha; albedo is a smooth function of the
    surface point, shading Lambertian plus ambient."""
    out = []
    c = np.asarray(center, np.float64)
    L = np.asarray(light, np.float64)
    L /= np.linalg.norm(L)
    for cam in cams:
        w, h = cam["res"]
        X = cam["xform"].reshape(3, 4).astype(np.float64)
        px = (np.arange(w) + 0.5) / w
        py = (np.arange(h) + 0.5) / h
        yy, xx = np.meshgrid(py, px, indexing="ij")
        d = np.stack([(xx - cam["principal"][0]) * w / cam["focal"][0], (yy - cam["principal"][1]) * h / cam["focal"][1],
                      np.ones_like(xx)], -1)
        dw = d @ X[:, :3].T
        dw /= np.linalg.norm(dw, axis=-1, keepdims=True)
        o = X[:, 3]
        oc = o - c
        b = (dw * oc).sum(-1)
        disc = b * b - (oc @ oc - radius * radius)
        hit = disc > 0
        t = -b - np.sqrt(np.where(hit, disc, 0))
        p = o + t[..., None] * dw
        n = (p - c) / radius
        albedo = 0.5 + 0.5 * np.sin(np.stack([n[..., 0] * 9, n[..., 1] * 7 + 1, n[..., 2] * 5 + 2], -1))
        shade = 0.25 + 0.75 * np.clip((n * L).sum(-1), 0, 1)
        rgb = np.where(hit[..., None], albedo * shade[..., None], 0.0)
        rgba = np.concatenate([rgb, hit[..., None].astype(np.float64)], -1)
        out.append(rgba.reshape(-1, 4).astype(np.float32))
    return np.concatenate(out, 0)
