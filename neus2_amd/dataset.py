"""Dataset loader for the reference's ``transforms.json`` scenes (load_nerf, src/nerf_loader.cu:197-757;
DATA_CONVENTION.md; NerfDataset::nerf_matrix_to_ngp, nerf_loader.h:114-137).

The camera part is host logic; images are decoded with PIL (the reference uses stb_image), uploaded as 8-bit RGBA and
converted on the GPU by n2_convert_rgba8 into the linear, premultiplied fp32 RGBA the ray generator reads.
Not read: depth maps, ray files, EXR images, rolling shutter, lens distortion, per-frame light directions."""
import ctypes as C
import json
import math
import os

import numpy as np

NERF_SCALE = 0.33  # nerf_loader.h:31


class DatasetError(ValueError):
    """Counterpart of the std::runtime_error / std::invalid_argument the reference's loader throws."""


def fov_to_focal_length(resolution, degrees):
    """common.h: 0.5 * resolution / tan(0.5 * fov)"""
    return 0.5 * float(resolution) / math.tan(0.5 * degrees * math.pi / 180.0)


def nerf_matrix_to_ngp(m, scale, offset, from_na=False, from_mitsuba=False):
    """NerfDataset::nerf_matrix_to_ngp on a 3x4 camera-to-world matrix (nerf_loader.h:114-137)."""
    r = np.array(m, np.float32)[:3, :4].copy()
    r[:, 1] *= -1
    r[:, 2] *= -1
    r[:, 3] = r[:, 3] * np.float32(scale) + np.asarray(offset, np.float32)
    if from_na:
        r[:, 1] *= -1
        r[:, 2] *= -1
    elif from_mitsuba:
        r[:, 0] *= -1
        r[:, 2] *= -1
    else:
        r = r[[1, 2, 0], :]  # cycle axes xyz <- yzx
    return r


def _strip_comments(text):
    """The reference parses with nlohmann's comment-tolerant mode (its own configs carry // comments)."""
    out, i, in_str = [], 0, False
    while i < len(text):
        c = text[i]
        if in_str:
            out.append(c)
            if c == "\\":
                out.append(text[i + 1])
                i += 1
            elif c == '"':
                in_str = False
        elif c == '"':
            in_str = True
            out.append(c)
        elif text.startswith("//", i):
            while i < len(text) and text[i] != "\n":
                i += 1
            continue
        elif text.startswith("/*", i):
            i = text.index("*/", i) + 2
            continue
        else:
            out.append(c)
        i += 1
    return "".join(out)


def load_transforms(paths):
    """Parses one or more transforms files.  Returns a dict: scale, offset, aabb_scale, from_na, from_mitsuba,
    white_transparent, black_transparent, and ``frames``: a list of dicts with file (absolute path), xform (3x4 float32,
    already in the trainer's coordinates), focal (fx, fy in pixels), principal (cx / w, cy / h), res (w, h) or None when
    the file does not state it (then the image decides)."""
    if isinstance(paths, (str, os.PathLike)):
        paths = [paths]
    docs = []
    for p in paths:
        with open(p) as f:
            docs.append((os.path.dirname(os.path.abspath(p)), json.loads(_strip_comments(f.read()))))
    if sum(len(d.get("frames", [])) for _, d in docs) == 0:
        raise DatasetError("No training images were found for NeRF training!")
    ds = dict(scale=NERF_SCALE, offset=(0.5, 0.5, 0.5), aabb_scale=1, from_na=False, from_mitsuba=False,
              white_transparent=False, black_transparent=False, frames=[])
    for base, d in docs:
        if "normal_mts_args" in d:
            ds["from_mitsuba"] = True
        if "from_na" in d:  # presence counts, not the value (src/nerf_loader.cu:346-348)
            ds["from_na"] = True
        if ds["from_mitsuba"]:
            ds["scale"] = 0.66
            ds["offset"] = (0.25 * 0.66,) * 3
        if "white_transparent" in d:
            ds["white_transparent"] = bool(d["white_transparent"])
        if "black_transparent" in d:
            ds["black_transparent"] = bool(d["black_transparent"])
        if "scale" in d:
            ds["scale"] = float(d["scale"])
        if "aabb_scale" in d:
            ds["aabb_scale"] = int(d["aabb_scale"])
        if "offset" in d:
            o = d["offset"]
            ds["offset"] = tuple(float(v) for v in o) if isinstance(o, list) else (float(o),) * 3
    for base, d in docs:
        frames = list(d.get("frames", []))  # file order (the sort by path is commented out, src/nerf_loader.cu:262-264)
        if "n_frames" in d:
            frames = frames[:int(d["n_frames"])]
        for fr in frames:
            res = (int(d["w"]), int(d["h"])) if "w" in d and "h" in d else None
            if "w" in fr and "h" in fr:
                res = (int(fr["w"]), int(fr["h"]))

            def focal(axis, extent):
                if axis + "_fov" in fr:
                    return fov_to_focal_length(extent, float(fr[axis + "_fov"]))
                if "fl_" + axis in d:
                    return float(d["fl_" + axis])
                if "camera_angle_" + axis in d:
                    return fov_to_focal_length(extent, float(d["camera_angle_" + axis]) * 180.0 / math.pi)
                if "fl_" + axis in fr:
                    return float(fr["fl_" + axis])
                if "camera_angle_" + axis in fr:
                    return fov_to_focal_length(extent, float(fr["camera_angle_" + axis]) * 180.0 / math.pi)
                return 0.0

            need_res = any(k.endswith("_fov") or k.startswith("camera_angle_") for k in list(fr) + list(d))
            if need_res and res is None:
                res = "image"  # the field of view needs the image size: resolved by load_images
            fx = focal("x", res[0]) if res not in (None, "image") else (focal("x", 1) if not need_res else None)
            fy = focal("y", res[1]) if res not in (None, "image") else (focal("y", 1) if not need_res else None)
            principal = [0.5, 0.5]
            if fx is not None and fx != 0:
                fl = [fx, fy if fy else fx]
            elif fy:
                fl = [fy, fy]
            elif fx is None:
                fl = None
            elif "intrinsic_matrix" in fr:
                K = fr["intrinsic_matrix"]
                fl = [float(K[0][0]), float(K[1][1])]
                principal = [float(K[0][2]) / float(d["w"]), float(K[1][2]) / float(d["h"])]
            else:
                raise DatasetError("Couldn't read fov.")
            if "cx" in fr:
                principal[0] = float(fr["cx"]) / float(fr["w"])
            if "cy" in fr:
                principal[1] = float(fr["cy"]) / float(fr["h"])
            path = fr["file_path"]
            full = os.path.join(base, path)
            if not os.path.splitext(path)[1]:
                full += ".png"  # the reference appends .png to extension-less paths
            xform = nerf_matrix_to_ngp(np.asarray(fr["transform_matrix"], np.float32), ds["scale"], ds["offset"], ds["from_na"],
                                       ds["from_mitsuba"])
            ds["frames"].append(dict(file=full, xform=xform, focal=fl, principal=tuple(principal), res=res if res != "image" else None,
                                     raw=fr, top=d))
    return ds


def load_images(ds, device="cuda"):
    """Decodes every frame's image, converts it on the GPU and returns (cameras, n_images, rgba) ready for
    Trainer.set_scene: the packed n2_camera array, and one fp32 [total_pixels, 4] tensor with the images back to back."""
    import torch
    from PIL import Image
    from . import capi
    from .capi import check, ptr
    from .tcnn_api import pack_cameras
    arrays, cams, offset = [], [], 0
    for fr in ds["frames"]:
        if not os.path.exists(fr["file"]):
            raise DatasetError("image not found: " + fr["file"])
        img = np.asarray(Image.open(fr["file"]).convert("RGBA"), np.uint8)
        h, w = img.shape[:2]
        alpha_path = fr["file"][:-len(os.path.splitext(fr["file"])[1])] + ".alpha" + os.path.splitext(fr["file"])[1]
        if os.path.exists(alpha_path):
            a = np.asarray(Image.open(alpha_path).convert("RGBA"), np.uint8)
            if a.shape[:2] != (h, w):
                raise DatasetError("Alpha image has wrong resolution: " + alpha_path)
            from_srgb = np.where(a[..., 0] / 255.0 <= 0.04045, a[..., 0] / 255.0 / 12.92, ((a[..., 0] / 255.0 + 0.055) / 1.055) ** 2.4)
            img = img.copy()
            img[..., 3] = (255.0 * from_srgb).astype(np.uint8)
        focal = fr["focal"]
        if focal is None:  # field of view given, resolution taken from the image
            raw, top = fr["raw"], fr["top"]

            def fl(axis, extent):
                for src, key, deg in ((raw, axis + "_fov", 1.0), (top, "camera_angle_" + axis, 180.0 / math.pi), (raw, "camera_angle_" + axis, 180.0 / math.pi)):
                    if key in src:
                        return fov_to_focal_length(extent, float(src[key]) * deg)
                return 0.0
            fx, fy = fl("x", w), fl("y", h)
            if fx == 0 and fy == 0:
                raise DatasetError("Couldn't read fov.")
            focal = [fx or fy, fy or fx]
        cams.append(dict(xform=fr["xform"].reshape(-1), focal=tuple(np.float32(v) for v in focal), principal=fr["principal"], res=(w, h),
                         pixel_offset=offset))
        arrays.append(img.reshape(-1, 4))
        offset += w * h
    bytes_dev = torch.from_numpy(np.concatenate(arrays)).to(device)
    rgba = torch.empty((offset, 4), dtype=torch.float32, device=device)
    check(capi.lib().n2_convert_rgba8(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.c_uint64(offset), ptr(bytes_dev), ptr(rgba),
                                      C.c_int(int(ds["white_transparent"])), C.c_int(int(ds["black_transparent"])), C.c_uint32(0)),
          "n2_convert_rgba8")
    return pack_cameras(cams, device=device), len(cams), rgba, cams
