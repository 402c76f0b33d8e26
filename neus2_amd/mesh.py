"""Mesh extraction on the host side: the lattice of SDF values, marching cubes through the C ABI and the reference's
OBJ / PLY writers (Testbed::compute_and_save_marching_cubes_mesh, src/testbed.cu:298-306; marching_cubes,
src/testbed_nerf.cu:4161-4212; save_mesh, src/marching_cubes.cu:824-975)."""
import ctypes as C

import numpy as np
import torch

from . import capi
from .capi import N2Error, check, ptr


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _u3(v):
    return (C.c_uint32 * 3)(*[int(x) for x in v])


def _f3(v):
    return (C.c_float * 3)(*[float(x) for x in v])


def marching_cubes_resolution(res_1d, aabb_min=(0, 0, 0), aabb_max=(1, 1, 1)):
    """get_marching_cubes_res (src/marching_cubes.cu:47-55): res_1d cells along the longest side, each side rounded up
    to a multiple of 16."""
    ext = np.asarray(aabb_max, np.float32) - np.asarray(aabb_min, np.float32)
    scale = np.float32(res_1d) / ext.max()
    r = (ext * scale + np.float32(0.5)).astype(np.int32)
    return tuple(int((x + 15) // 16 * 16) for x in r)


def case_table():
    t = np.zeros((256, 16), np.int8)
    check(capi.lib().n2_marching_cubes_table(ptr(t)), "n2_marching_cubes_table")
    return t


def density_on_grid(field_handle, res, aabb_min=(0, 0, 0), aabb_max=(1, 1, 1), chunk=1 << 20, device="cuda"):
    """Testbed::get_density_on_grid: fp32 tensor [rz, ry, rx] of the field's SDF on the lattice."""
    L = capi.lib()
    L.n2_density_on_grid_scratch_bytes.restype = C.c_uint64
    n = int(res[0]) * int(res[1]) * int(res[2])
    chunk = max(8, min(chunk, (n + 7) // 8 * 8) // 8 * 8)
    nbytes = int(L.n2_density_on_grid_scratch_bytes(C.c_uint32(chunk)))
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=device)
    out = torch.empty(n, dtype=torch.float32, device=device)
    check(L.n2_density_on_grid(field_handle, _stream(), _u3(res), _f3(aabb_min), _f3(aabb_max), ptr(out), ptr(scratch), C.c_uint64(nbytes),
                               C.c_uint32(chunk)), "n2_density_on_grid")
    return out.view(int(res[2]), int(res[1]), int(res[0]))


def marching_cubes(density, thresh, aabb_min=(0, 0, 0), aabb_max=(1, 1, 1), want_normals=True):
    """marching_cubes_gpu on a float32 CUDA tensor [rz, ry, rx].  Returns (vertices [V, 3] fp32, indices [T, 3] int32
    holding uint32 values, normals [V, 3] fp32 or None)."""
    if density.dtype != torch.float32 or not density.is_cuda or density.dim() != 3 or not density.is_contiguous():
        raise N2Error("density must be a contiguous float32 CUDA tensor [rz, ry, rx]")
    L = capi.lib()
    L.n2_marching_cubes_workspace_bytes.restype = C.c_uint64
    res = (density.shape[2], density.shape[1], density.shape[0])
    nbytes = int(L.n2_marching_cubes_workspace_bytes(_u3(res)))
    if nbytes == 0:
        raise N2Error("n2_marching_cubes_workspace_bytes: " + L.n2_last_error().decode())
    ws = torch.empty(nbytes, dtype=torch.uint8, device=density.device)
    nv, nt = C.c_uint32(), C.c_uint32()
    check(L.n2_marching_cubes_count(_stream(), _u3(res), _f3(aabb_min), _f3(aabb_max), C.c_float(thresh), ptr(density), ptr(ws),
                                    C.c_uint64(nbytes), C.byref(nv), C.byref(nt)), "n2_marching_cubes_count")
    verts = torch.empty((nv.value, 3), dtype=torch.float32, device=density.device)
    idx = torch.empty((nt.value, 3), dtype=torch.int32, device=density.device)
    normals = torch.empty((nv.value, 3), dtype=torch.float32, device=density.device) if want_normals else None
    check(L.n2_marching_cubes_emit(_stream(), _u3(res), _f3(aabb_min), _f3(aabb_max), C.c_float(thresh), ptr(density), ptr(ws),
                                   ptr(verts) if nv.value else None, ptr(idx) if nt.value else None,
                                   ptr(normals) if (want_normals and nv.value) else None, nv, nt), "n2_marching_cubes_emit")
    return verts, idx, normals


def save_mesh(path, verts, normals, indices, colors=None, nerf_scale=1.0, nerf_offset=(0.0, 0.0, 0.0), invert_normals=False):
    """save_mesh without texture unwrapping (src/marching_cubes.cu:880-975): '.ply' writes ASCII PLY, anything else
    OBJ with per-vertex colours; positions are mapped back with (p - offset) / scale, faces are written with
    reversed winding unless invert_normals."""
    v = np.asarray(verts, np.float32)
    n = np.asarray(normals, np.float32)
    f = np.asarray(indices).astype(np.int64).reshape(-1, 3)
    c = np.ones_like(v) if colors is None else np.asarray(colors, np.float32)
    p = (v - np.asarray(nerf_offset, np.float32)) / np.float32(nerf_scale)
    ln = np.linalg.norm(n, axis=1, keepdims=True)
    nn = np.divide(n, ln, out=np.zeros_like(n), where=ln > 0)
    order = (0, 1, 2) if invert_normals else (2, 1, 0)
    with open(path, "w") as out:
        if str(path).endswith(".ply"):
            out.write("ply\nformat ascii 1.0\ncomment output from https://github.com/NVlabs/instant-ngp\n"
                      f"element vertex {len(v)}\nproperty float x\nproperty float y\nproperty float z\n"
                      "property float nx\nproperty float ny\nproperty float nz\n"
                      "property uchar red\nproperty uchar green\nproperty uchar blue\n"
                      f"element face {len(f)}\nproperty list uchar int vertex_index\nend_header\n")
            c8 = np.clip(c * 255.0, 0.0, 255.0).astype(np.uint8)
            for i in range(len(v)):
                out.write("%0.5f %0.5f %0.5f %0.3f %0.3f %0.3f %d %d %d\n" % (*p[i], *nn[i], *c8[i]))
            for t in f:
                out.write("3 %d %d %d\n" % (t[order[0]], t[order[1]], t[order[2]]))
        else:
            cc = np.clip(c, 0.0, 1.0)
            for i in range(len(v)):
                out.write("v %0.5f %0.5f %0.5f %0.3f %0.3f %0.3f\n" % (*p[i], *cc[i]))
            for i in range(len(v)):
                out.write("vn %0.5f %0.5f %0.5f\n" % tuple(nn[i]))
            for t in f:
                a, b, d = t[order[0]] + 1, t[order[1]] + 1, t[order[2]] + 1
                out.write("f %u//%u %u//%u %u//%u\n" % (a, a, b, b, d, d))
