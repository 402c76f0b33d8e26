"""The snapshot file format against an independent MessagePack implementation (the msgpack package): what the
configuration encoder writes, and that the C ABI rejects malformed files.  No GPU: nothing here touches device memory."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

msgpack = pytest.importorskip("msgpack")

CONFIG = {
    "loss": {"otype": "Huber"},
    "optimizer": {"otype": "Ema", "decay": 0.95, "nested": {"otype": "ExponentialDecay", "decay_start": 20000, "decay_interval": 10000,
                                                             "decay_base": 0.33, "nested": {"otype": "Adam", "learning_rate": 1e-3, "beta1": 0.9,
                                                                                          "beta2": 0.99, "epsilon": 1e-15, "l2_reg": 1e-6,
                                                                                          "optimize_canonical_params": True}}},
    "encoding": {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 19, "base_resolution": 16},
    "misc": [1, -1, -33, 127, 128, 255, 256, 65535, 65536, 2 ** 32, -2 ** 31, 0.5, 1.0 / 3.0, None, False, "x" * 40, "y" * 300, list(range(20))],
}


def test_config_encoder_matches_msgpack_library():
    from neus2_amd.snapshot import pack_config
    blob = pack_config(CONFIG)
    assert msgpack.unpackb(blob, raw=False, strict_map_key=False) == CONFIG
    # same bytes as the library for the value kinds JSON has (integers in their smallest form, exact floats as float32)
    assert pack_config(128) == msgpack.packb(128) and pack_config(-33) == msgpack.packb(-33) and pack_config(2 ** 32) == msgpack.packb(2 ** 32)
    assert pack_config(0.5) == b"\xca" + struct.pack(">f", 0.5) and pack_config(0.1) == msgpack.packb(0.1)
    assert pack_config("y" * 300) == msgpack.packb("y" * 300) and pack_config(list(range(20))) == msgpack.packb(list(range(20)))


def open_snapshot(path):
    from neus2_amd import capi
    from neus2_amd.snapshot import SnapshotInfo
    h, info = C.c_void_p(), SnapshotInfo()
    rc = capi.lib().n2_snapshot_open(str(path).encode(), C.byref(h), C.byref(info))
    if rc == 0:
        capi.lib().n2_snapshot_close(h)
    return rc, info, capi.lib().n2_last_error().decode()


def reference_style_file(n_params=24, params_type="__half", cells=0, with_optimizer=False):
    """A file as nlohmann::json::to_msgpack would write the reference's m_network_config, built with the msgpack package."""
    rng = np.random.default_rng(0)
    dt = np.float16 if params_type == "__half" else np.float32
    snap = {"n_params": n_params, "params_type": params_type, "params_binary": rng.standard_normal(n_params).astype(dt).tobytes(),
            "density_grid_size": 128, "density_grid_binary": rng.random(cells).astype(np.float16).tobytes(),
            "nerf": {"aabb_scale": 1, "rgb": {"rays_per_batch": 4096, "measured_batch_size": 250000, "measured_batch_size_before_compaction": 260000},
                     "dataset": {"n_images": 3, "paths": ["a.png", "b.png"]}},
            "training_step": 1234, "loss": 0.03125}
    if with_optimizer:
        adam = {"current_step": 1234, "base_learning_rate": 1e-3, "first_moments_binary": np.zeros(n_params, np.float32).tobytes(),
                "second_moments_binary": np.ones(n_params, np.float32).tobytes(), "param_steps_binary": np.full(n_params, 7, np.uint32).tobytes()}
        snap["optimizer"] = {"ema_weights_binary": np.full(n_params, 0.5, np.float32).tobytes(), "nested": {"nested": adam}}
    return dict(CONFIG, snapshot=snap)


@pytest.mark.parametrize("params_type", ["__half", "float"])
def test_reader_accepts_files_written_by_another_implementation(tmp_path, params_type):
    doc = reference_style_file(params_type=params_type, cells=64, with_optimizer=True)
    p = tmp_path / "ref.msgpack"
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    rc, info, err = open_snapshot(p)
    assert rc == 0, err
    assert info.n_params == 24 and info.params_are_fp32 == (params_type == "float") and info.density_grid_size == 128
    assert info.density_grid_cells == 64 and info.aabb_scale == 1 and info.rays_per_batch == 4096
    assert info.measured_batch_size == 250000 and info.measured_batch_size_before_compaction == 260000
    assert info.training_step == 1234 and info.loss == 0.03125
    assert info.has_optimizer_state == 1 and info.has_ema_weights == 1 and info.optimizer_steps == 1234 and abs(info.learning_rate - 1e-3) < 1e-9


def test_reader_rejects_bad_files(tmp_path):
    p = tmp_path / "x.msgpack"
    rc, _, err = open_snapshot(tmp_path / "missing.msgpack")
    assert rc != 0 and "cannot open" in err
    p.write_bytes(msgpack.packb(CONFIG, use_bin_type=True))
    rc, _, err = open_snapshot(p)
    assert rc != 0 and "does not contain a snapshot" in err  # the reference's message, src/testbed.cu:3183
    good = msgpack.packb(reference_style_file(), use_bin_type=True)
    for cut in (1, len(good) // 2, len(good) - 1):
        p.write_bytes(good[:cut])
        rc, _, err = open_snapshot(p)
        assert rc != 0 and ("truncated" in err or "not a MessagePack map" in err or "no parameters" in err or "snapshot" in err), (cut, err)
    doc = reference_style_file()
    doc["snapshot"]["n_params"] = 25  # announces more than params_binary holds
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    rc, _, err = open_snapshot(p)
    assert rc != 0 and "params_binary" in err
    doc = reference_style_file()
    doc["snapshot"]["params_type"] = "double"
    p.write_bytes(msgpack.packb(doc, use_bin_type=True))
    rc, _, err = open_snapshot(p)
    assert rc != 0 and "params_type" in err
    p.write_bytes(msgpack.packb([1, 2, 3]))
    assert open_snapshot(p)[0] != 0
