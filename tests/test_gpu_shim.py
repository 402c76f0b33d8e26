"""The C++ shim (include/neus2_amd.hpp) driven by a C++ program, checked against the oracle: grid forward with
Jacobian, SDF MLP forward and input gradient, grid backward (parameter scatter + input gradient)."""
import os
import subprocess

import numpy as np
import pytest

from gpu_util import RTOL, assert_close, q16, rel_l2

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "shim_check")


def test_shim_program_matches_oracle(oracle, tmp_path):
    assert os.path.exists(EXE), "tests/cpp/shim_check is missing: run __graft_entry__.build()"
    rng = np.random.default_rng(3)
    n = 2048
    og = oracle.Grid(16, 19, 16, 1.447)
    om = oracle.Mlp(48, 64, 1, 16)
    P = q16(rng.uniform(-0.5, 0.5, og.n_params))
    W = q16(np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy")) + rng.normal(0, 0.05, 4096))
    xyz = rng.random((3, n), dtype=np.float32)
    dy = q16(rng.standard_normal((32, n)))
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        f.write(np.uint32(n).tobytes())
        for a, t in ((P, np.float16), (W, np.float16), (xyz, np.float32), (dy, np.float16)):
            f.write(np.ascontiguousarray(a).astype(t).tobytes())
    r = subprocess.run([EXE, "gpu", str(fin), str(fout)], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    raw = open(fout, "rb").read()
    o = 0

    def take(count, t):
        nonlocal o
        a = np.frombuffer(raw, dtype=t, count=count, offset=o).astype(np.float32)
        o += count * np.dtype(t).itemsize
        return a

    enc = take(32 * n, np.float16).reshape(32, n)
    y = take(16 * n, np.float16).reshape(16, n)
    g = take(48 * n, np.float16).reshape(48, n)
    grad = take(og.n_params, np.float16)
    dx = take(3 * n, np.float32).reshape(3, n)
    assert o == len(raw)
    ref_enc, J = og.forward(P, xyz, want_dy_dx=True)
    assert_close(enc, ref_enc, what="encoding")
    inp = np.zeros((48, n), np.float32)
    inp[3:35] = q16(ref_enc)
    ref_y, h = om.forward(W, inp, round_hidden=True)
    assert_close(y, ref_y, what="sdf net output", outlier_frac=1e-3)
    e0 = np.zeros((16, n), np.float32)
    e0[0] = 1
    ref_g, _ = om.backward(W, inp, h, e0, want_dW=False)
    assert_close(g, ref_g, what="input gradient", outlier_frac=2e-3)
    ref_grad, ref_dx = og.backward(P, xyz, dy)
    assert_close(dx, ref_dx, what="dL_dx")
    assert rel_l2(grad, ref_grad) < 2e-2  # packed fp16 atomics without a scatter workspace
