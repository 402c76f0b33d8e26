"""Writes the fixtures under tests/golden/ from the reference's own DATA files.

Run in the build container (needs /root/reference):  python tests/golden/make_fixtures.py

  sdf_mlp_weights_48.npy  <- utils/mlp_weights.txt (4096 fp32: W0[64][48] then W1[16][64],
                             the geometric-init weights loaded at nerf_network.h:774-803)
  sdf_mlp_weights_32.npy  <- utils/mlp_weights_hidden_layer_num_1_hidden_size_32.txt (3072 fp32)

Only numbers are read (text parsed as floats); nothing from the reference is executed.
"""
import os

import numpy as np

REF = "/root/reference/utils"
HERE = os.path.dirname(os.path.abspath(__file__))

if __name__ == "__main__":
    for src, dst, n in (("mlp_weights.txt", "sdf_mlp_weights_48.npy", 4096),
                        ("mlp_weights_hidden_layer_num_1_hidden_size_32.txt", "sdf_mlp_weights_32.npy", 3072)):
        w = np.loadtxt(os.path.join(REF, src), dtype=np.float64).astype(np.float32)
        assert w.size == n, (src, w.size)
        np.save(os.path.join(HERE, dst), w)
        print(dst, w.size, float(np.abs(w).max()))
