"""Writes tests/golden/placement_patterns.npz: a few layers of the placement patterns that the reference's own
placement tests hold as data (omni/accelerators/placement/tests/patterns/*.npy), bit-packed.

Run once in a container that has the reference tree:  python tests/golden/make_placement_fixture.py
The files are loaded with numpy.load(allow_pickle=False); nothing of the reference is executed.
"""
import os

import numpy as np

SRC = "/root/reference/omni/accelerators/placement/tests/patterns"
PICK = {
    # name in the fixture: (file, layers kept)
    "dies32_copies4": ("placement_pattern_3d_v3_supersuperrr4_32devices_SC.npy", [0, 7, 57]),
    "dies64_copies12": ("DSV3_RedFullLays_+58_58_MoELayers_64_dies_Rand_0411.npy", [0, 30]),
    "dies32_decode": ("DSV3_0427_GSM8K_decode_RedFullLays_+10_58_MoELayers_32_dies_epmaxdeploy_12.npy", [3, 40, 57]),
    "dies16_base": ("placement_pattern_3d_v3_naivebalance3_16devices_HE.npy", [0, 12]),
}


def main():
    out = {}
    for name, (fname, layers) in PICK.items():
        a = np.load(os.path.join(SRC, fname), allow_pickle=False)
        assert set(np.unique(a).tolist()) <= {0, 1}
        sub = a[:, layers, :].astype(np.uint8)
        out[name + "_bits"] = np.packbits(sub.reshape(-1))
        out[name + "_shape"] = np.array(sub.shape, dtype=np.int64)
        out[name + "_layers"] = np.array(layers, dtype=np.int64)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "placement_patterns.npz")
    np.savez_compressed(dst, **out)
    print(dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
