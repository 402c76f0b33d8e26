"""A transforms.json scene written to disk, loaded through the dataset module and trained on: the loader's cameras and
images drive the same sample generator as the synthetic scene they were rendered from."""
import json
import os

import numpy as np
import pytest
import torch

from gpu_util import dev, host
from neus2_amd import scene

pytestmark = pytest.mark.gpu


def test_rgba8_conversion_matches_oracle(oracle):
    import ctypes as C
    from neus2_amd import capi
    rng = np.random.default_rng(0)
    px = rng.integers(0, 256, (50_001, 4), dtype=np.uint8)
    px[:64, :3] = 255
    px[64:128, :3] = 0
    px[128:160] = [255, 0, 255, 0]
    px[160:170] = [9, 8, 7, 6]
    for wt, bt, mask in ((0, 0, 0), (1, 1, 0), (0, 0, 0x06070809)):
        out = torch.empty((len(px), 4), dtype=torch.float32, device="cuda")
        capi.check(capi.lib().n2_convert_rgba8(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.c_uint64(len(px)), capi.ptr(dev(px)), capi.ptr(out),
                                               C.c_int(wt), C.c_int(bt), C.c_uint32(mask)), "n2_convert_rgba8")
        want = oracle.convert_rgba8(px, bool(wt), bool(bt), mask)
        np.testing.assert_allclose(host(out), want, rtol=3e-6, atol=1e-9)  # powf differs by an ulp or two between host and device
        assert ((host(out) == -1) == (want == -1)).all()


def test_scene_from_disk_trains_like_the_synthetic_one(tmp_path):
    from PIL import Image
    from neus2_amd.dataset import load_images, load_transforms
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    cams = scene.cameras_on_sphere(6, 64)
    rgba = scene.render_sphere_images(cams)  # linear premultiplied fp32
    os.makedirs(tmp_path / "images")
    frames = []
    for i, c in enumerate(cams):
        img = rgba[i * 64 * 64:(i + 1) * 64 * 64].reshape(64, 64, 4)
        a = img[..., 3:4]
        straight = np.divide(img[..., :3], a, out=np.zeros_like(img[..., :3]), where=a > 0)
        srgb = np.where(straight <= 0.0031308, 12.92 * straight, 1.055 * np.power(np.maximum(straight, 1e-12), 1 / 2.4) - 0.055)
        png = np.concatenate([np.round(srgb * 255), np.round(a * 255)], -1).clip(0, 255).astype(np.uint8)
        Image.fromarray(png, "RGBA").save(tmp_path / "images" / f"{i:06d}.png")
        X = np.eye(4, dtype=np.float32)
        X[:3, :4] = c["xform"].reshape(3, 4)
        X[:3, 3] = (X[:3, 3] - 0.5) / 0.5  # undo scale 0.5 / offset 0.5
        K = [[float(c["focal"][0]), 0, 32.0, 0], [0, float(c["focal"][1]), 32.0, 0], [0, 0, 1, 0], [0, 0, 0, 1]]
        frames.append(dict(file_path=f"images/{i:06d}.png", transform_matrix=X.tolist(), intrinsic_matrix=K))
    (tmp_path / "transforms.json").write_text(json.dumps(dict(from_na=True, w=64, h=64, aabb_scale=1.0, scale=0.5, offset=[0.5, 0.5, 0.5], frames=frames)))
    ds = load_transforms(tmp_path / "transforms.json")
    d_cams, n_images, d_rgba, loaded = load_images(ds)
    assert n_images == 6 and d_rgba.shape == (6 * 64 * 64, 4)
    for c, l in zip(cams, loaded):
        np.testing.assert_allclose(l["xform"], c["xform"], atol=1e-6)
        np.testing.assert_allclose(l["focal"], c["focal"], rtol=1e-6)
        assert tuple(l["res"]) == (64, 64) and l["pixel_offset"] == c["pixel_offset"] and tuple(l["principal"]) == (0.5, 0.5)
    # 8-bit quantisation is all that separates the decoded images from the rendered ones
    assert np.abs(host(d_rgba) - rgba).max() < 0.01
    results = []
    for cam_buf, img in ((d_cams, d_rgba), (pack_cameras(cams), dev(rgba))):
        tr = Trainer(default_config(target_batch_size=4096, max_rays_per_batch=1024, max_samples=1 << 16))
        tr.set_scene(cam_buf, 6, img, dev(scene.sphere_bitfield()))
        tr.initialize_params(seed=5)
        tr.step(n_rays=256, n_inference=1 << 16, seed=3)
        results.append(tr.read_counters())
    a, b = results
    assert a["rays"] == b["rays"] and a["samples"] == b["samples"] and a["samples"] > 0  # same cameras, same rays
    assert abs(a["loss"] - b["loss"]) < 0.02 * abs(b["loss"])                            # colours differ by the quantisation only
