"""Writes tests/golden/pack_fixture.npz: packed bytes produced by the
reference's own packer (gpu/pack_weight.py:76-98) for small seeded ternary
matrices.  Run once, in the build container only (the reference tree is not
present anywhere else); the .npz it writes is the committed fixture.

    python tests/golden/make_pack_fixture.py [/root/reference]

Only inputs and outputs are stored -- no reference code.
"""
import os
import sys

import numpy as np


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, os.path.join(ref_root, "gpu"))
    import torch
    from pack_weight import convert_weight_int8_to_int2  # the reference packer

    out = {}
    # (N, K, seed); shapes chosen to cover >1 tile in both directions, a
    # non-square case each way and one K that is a multiple of 32 but not 128.
    for n, k, seed in [(16, 32, 1), (32, 256, 2), (48, 128, 3), (64, 96, 4), (16, 2560, 5)]:
        rng = np.random.Generator(np.random.Philox(seed))
        w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
        packed = convert_weight_int8_to_int2(torch.from_numpy(w.copy()))
        assert packed.shape == (n, k // 4) and packed.dtype == torch.int8
        out[f"w_{n}x{k}"] = w
        out[f"packed_{n}x{k}"] = packed.numpy().copy()
    # one structured matrix: W[n, k] encodes position, so a transposed or
    # mis-tiled layout cannot pass by chance
    n, k = 32, 64
    w = (((np.arange(n)[:, None] * 7 + np.arange(k)[None, :] * 3) % 3) - 1).astype(np.int8)
    out[f"w_struct_{n}x{k}"] = w
    out[f"packed_struct_{n}x{k}"] = convert_weight_int8_to_int2(torch.from_numpy(w.copy())).numpy().copy()
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pack_fixture.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
