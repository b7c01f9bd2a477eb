"""The package's packer (the drop-in for gpu/pack_weight.py:76) against the
golden bytes and the oracle."""
import numpy as np
import pytest
import torch

from bitnet_amd import convert, pack_weight
from oracle import bitlinear_oracle as o


def test_packer_reproduces_reference_bytes(golden_pack):
    for key in golden_pack.files:
        if not key.startswith("w_"):
            continue
        w = golden_pack[key]
        got = pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w))
        assert got.dtype == torch.int8 and tuple(got.shape) == (w.shape[0], w.shape[1] // 4)
        assert np.array_equal(got.numpy(), golden_pack["packed_" + key[2:]]), key
        assert np.array_equal(pack_weight.convert_weight_int2_to_int8(got).numpy(), w)


@pytest.mark.parametrize("n,k", [(16, 32), (48, 160), (2560, 128), (32, 6912)])
def test_packer_equals_oracle(n, k):
    w = np.random.default_rng(n + k).integers(-1, 2, size=(n, k), dtype=np.int8)
    got = pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w)).numpy()
    assert np.array_equal(got, o.pack_int2(w))


def test_packer_rejects_bad_input():
    with pytest.raises(ValueError):
        pack_weight.convert_weight_int8_to_int2(torch.zeros(15, 32, dtype=torch.int8))
    with pytest.raises(ValueError):
        pack_weight.convert_weight_int8_to_int2(torch.zeros(16, 48, dtype=torch.int8))
    with pytest.raises(ValueError):
        pack_weight.convert_weight_int8_to_int2(torch.full((16, 32), 2, dtype=torch.int8))


def test_convert_matches_oracle():
    rng = np.random.default_rng(0)
    parts = [(rng.standard_normal((r, 128)) * sd).astype(np.float32) for r, sd in [(32, 0.02), (16, 0.04), (16, 0.01)]]
    packed, scale = convert.pack_fused([torch.from_numpy(p) for p in parts])
    w, ws = o.fused_weight_and_scales(parts)
    assert np.array_equal(packed.numpy(), o.pack_int2(w))
    assert np.array_equal(scale.view(torch.int16).numpy().view(np.uint16), ws)
