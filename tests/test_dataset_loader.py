"""Host logic of the transforms.json loader against the reference's conventions (nerf_loader.h:114-137,
src/nerf_loader.cu:640-712) and the image conversion oracle against the sRGB definition."""
import json
import math

import numpy as np
import pytest

from neus2_amd.dataset import DatasetError, fov_to_focal_length, load_transforms, nerf_matrix_to_ngp


def rot(axis, deg):
    c, s = math.cos(math.radians(deg)), math.sin(math.radians(deg))
    m = {"x": [[1, 0, 0], [0, c, -s], [0, s, c]], "y": [[c, 0, s], [0, 1, 0], [-s, 0, c]], "z": [[c, -s, 0], [s, c, 0], [0, 0, 1]]}[axis]
    return np.array(m, np.float32)


def c2w(R, t):
    m = np.eye(4, dtype=np.float32)
    m[:3, :3], m[:3, 3] = R, t
    return m


def test_matrix_conventions():
    R, t = rot("x", 20) @ rot("y", -35), np.array([0.3, -1.2, 2.0], np.float32)
    # NeuS2's own format: the two double sign flips cancel, only the translation is rescaled into the unit cube
    m = nerf_matrix_to_ngp(c2w(R, t), 0.5, (0.5, 0.5, 0.5), from_na=True)
    np.testing.assert_allclose(m[:, :3], R, atol=1e-7)
    np.testing.assert_allclose(m[:, 3], t * 0.5 + 0.5, atol=1e-7)
    # original NeRF format: camera y and z axes flipped (OpenGL -> +z forward), then world axes cycled xyz <- yzx
    m = nerf_matrix_to_ngp(c2w(R, t), 0.33, (0.5, 0.5, 0.5))
    want = np.concatenate([R * np.array([1, -1, -1], np.float32), (t * np.float32(0.33) + 0.5)[:, None]], 1)[[1, 2, 0]]
    np.testing.assert_allclose(m, want, atol=1e-7)
    assert abs(np.linalg.det(m[:, :3].astype(np.float64)) - 1.0) < 1e-5  # still a rotation
    # mitsuba scenes flip x and z instead
    m = nerf_matrix_to_ngp(c2w(R, t), 0.66, (0.165,) * 3, from_mitsuba=True)
    np.testing.assert_allclose(m[:, :3], R * np.array([-1, -1, 1], np.float32), atol=1e-7)


def write_scene(tmp_path, top, frames, name="transforms.json"):
    doc = dict(top, frames=frames)
    p = tmp_path / name
    p.write_text(json.dumps(doc))
    return p


def test_neus2_format_with_intrinsic_matrices(tmp_path):
    K = [[2892.33, -0.0002, 823.2, 0], [0, 2883.17, 619.07, 0], [0, 0, 1, 0], [0, 0, 0, 1]]
    frames = [dict(file_path=f"images/{i:06d}.png", transform_matrix=c2w(rot("y", 30 * i), [0.1 * i, 0.2, -2.5]).tolist(), intrinsic_matrix=K)
              for i in (2, 0, 1)]
    p = write_scene(tmp_path, dict(from_na=True, w=1600, h=1200, aabb_scale=1.0, scale=0.5, offset=[0.5, 0.5, 0.5]), frames)
    ds = load_transforms(p)
    assert ds["from_na"] and ds["scale"] == 0.5 and ds["aabb_scale"] == 1 and len(ds["frames"]) == 3
    assert [f["file"][-10:] for f in ds["frames"]] == ["000002.png", "000000.png", "000001.png"]  # file order is kept
    f0 = ds["frames"][0]
    assert f0["focal"] == [2892.33, 2883.17] and f0["res"] == (1600, 1200)
    np.testing.assert_allclose(f0["principal"], (823.2 / 1600, 619.07 / 1200), rtol=1e-6)
    np.testing.assert_allclose(ds["frames"][0]["xform"][:, 3], np.array([0.2, 0.2, -2.5]) * 0.5 + 0.5, atol=1e-6)
    np.testing.assert_allclose(ds["frames"][2]["xform"][:, :3], rot("y", 30), atol=1e-6)


def test_original_nerf_format_and_focal_sources(tmp_path):
    frames = [dict(file_path="./train/r_0", transform_matrix=c2w(np.eye(3), [0, 0, 4]).tolist())]
    ds = load_transforms(write_scene(tmp_path, dict(camera_angle_x=0.6911112070083618, w=800, h=800), frames))
    f = ds["frames"][0]
    assert ds["scale"] == 0.33 and ds["offset"] == (0.5, 0.5, 0.5) and not ds["from_na"]
    assert f["file"].endswith("train/r_0.png")
    want = 0.5 * 800 / math.tan(0.5 * 0.6911112070083618)
    np.testing.assert_allclose(f["focal"], [want, want], rtol=1e-6)   # y falls back to x
    assert abs(fov_to_focal_length(800, 90.0) - 400.0) < 1e-9
    # explicit focal lengths and principal point in the frame
    frames = [dict(file_path="a.png", transform_matrix=np.eye(4).tolist(), fl_x=1000.0, fl_y=1100.0, cx=300.0, cy=260.0, w=640, h=480)]
    f = load_transforms(write_scene(tmp_path, {}, frames, "t2.json"))["frames"][0]
    assert f["focal"] == [1000.0, 1100.0] and f["principal"] == (300.0 / 640, 260.0 / 480) and f["res"] == (640, 480)
    # nothing to derive the focal length from: the reference's error
    frames = [dict(file_path="a.png", transform_matrix=np.eye(4).tolist())]
    with pytest.raises(DatasetError, match="fov"):
        load_transforms(write_scene(tmp_path, dict(w=10, h=10), frames, "t3.json"))
    with pytest.raises(DatasetError, match="No training images"):
        load_transforms(write_scene(tmp_path, {}, [], "t4.json"))


def test_comments_and_several_files(tmp_path):
    a = tmp_path / "transforms_train.json"
    a.write_text('{ "from_na": true, // NeuS2 data\n "w": 4, "h": 4, "scale": 0.5, /* block */ "frames": [ {"file_path": "x//y.png", '
                 '"transform_matrix": [[1,0,0,0],[0,1,0,0],[0,0,1,0],[0,0,0,1]], "intrinsic_matrix": [[5,0,2,0],[0,5,2,0],[0,0,1,0],[0,0,0,1]]} ] }')
    b = write_scene(tmp_path, dict(w=4, h=4), [dict(file_path="z.png", transform_matrix=np.eye(4).tolist(),
                                                    intrinsic_matrix=[[6, 0, 2, 0], [0, 6, 2, 0], [0, 0, 1, 0], [0, 0, 0, 1]])], "transforms_test.json")
    ds = load_transforms([a, b])
    assert len(ds["frames"]) == 2 and ds["frames"][0]["file"].endswith("x//y.png") and ds["frames"][1]["focal"] == [6.0, 6.0]
    assert ds["from_na"]  # stated by one file, holds for the data set


def test_srgb_oracle_against_the_standard(oracle):
    # IEC 61966-2-1: linear segment below 0.04045, (c + 0.055)/1.055 to the power 2.4 above; the two pieces meet there
    assert abs(float(oracle.srgb_to_linear(0.04045)) - 0.04045 / 12.92) < 1e-9
    assert abs(float(oracle.srgb_to_linear(np.float32(0.0404501))) - ((0.0404501 + 0.055) / 1.055) ** 2.4) < 1e-7
    np.testing.assert_allclose(oracle.srgb_to_linear([0.0, 0.5, 1.0]), [0.0, 0.21404114, 1.0], rtol=1e-6)
    px = np.array([[255, 255, 255, 255], [255, 255, 255, 128], [0, 0, 0, 255], [188, 0, 0, 255], [255, 0, 255, 0], [10, 20, 30, 0]], np.uint8)
    out = oracle.convert_rgba8(px)
    np.testing.assert_allclose(out[0], [1, 1, 1, 1], rtol=1e-6)
    np.testing.assert_allclose(out[1], [128 / 255] * 4, rtol=1e-6)       # premultiplied
    np.testing.assert_allclose(out[3], [float(oracle.srgb_to_linear(188 / 255)), 0, 0, 1], rtol=1e-6)
    assert (out[4] == -1).all() and (out[5] == 0).all()                   # the mask marker; a transparent pixel
    assert (oracle.convert_rgba8(px, white_transparent=True)[0] == 0).all() and oracle.convert_rgba8(px, black_transparent=True)[2][3] == 0
    assert (oracle.convert_rgba8(px, mask_color=0xFF0000BC)[3] == -1).all()
