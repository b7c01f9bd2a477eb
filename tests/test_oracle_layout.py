"""Pins the oracle's weight layout (pack / unpack / decode / kernel-address
emulation) without a GPU: golden bytes from the reference packer, two
independent restatements, and the closed form (integer matmul)."""
import numpy as np
import pytest

from oracle import bitlinear_oracle as o


def _keys(golden):
    return [k[2:] for k in golden.files if k.startswith("w_")]


def test_golden_bytes_match_both_restatements(golden_pack):
    names = _keys(golden_pack)
    assert len(names) >= 6
    for name in names:
        w = golden_pack["w_" + name]
        ref = golden_pack["packed_" + name]
        assert ref.dtype == np.int8 and ref.shape == (w.shape[0], w.shape[1] // 4)
        assert np.array_equal(o.pack_int2(w), ref), name
        assert np.array_equal(o.pack_int2_closed_form(w), ref), name
        assert np.array_equal(o.unpack_int2(ref, *w.shape), w), name


def test_golden_never_contains_code_zero(golden_pack):
    for name in _keys(golden_pack):
        b = golden_pack["packed_" + name].view(np.uint8)
        for sh in (0, 2, 4, 6):
            assert np.all(((b >> sh) & 3) != 0)


@pytest.mark.parametrize("n,k,seed", [(16, 32, 0), (32, 64, 1), (80, 160, 2), (16, 6912, 3), (160, 128, 4)])
def test_staged_equals_closed_form_and_roundtrips(n, k, seed):
    w = np.random.default_rng(seed).integers(-1, 2, size=(n, k), dtype=np.int8)
    p = o.pack_int2(w)
    assert np.array_equal(p, o.pack_int2_closed_form(w))
    assert np.array_equal(o.unpack_int2(p, n, k), w)


def test_single_nonzero_weight_lands_where_the_closed_form_says():
    n, k = 32, 128
    for (r, c, v) in [(0, 0, 1), (5, 17, -1), (15, 31, 1), (16, 32, -1), (31, 127, 1), (9, 77, -1)]:
        w = np.zeros((n, k), dtype=np.int8)
        w[r, c] = v
        words = o.pack_int2(w).view(np.uint8).reshape(-1).view("<u4")
        base = np.uint32(0xAAAAAAAA)  # code 2 (= weight 0) in all 16 fields
        diff = np.nonzero(words != base)[0]
        word, bit = o.packed_word_index(r, c, k)
        assert list(diff) == [int(word)]
        assert (int(words[word]) >> int(bit)) & 3 == v + 2


def test_decode_exhaustive_per_field():
    # every field position x every code, other fields held at code 2
    for e in range(16):
        bit = (e % 4) * 8 + (e // 4) * 2
        for code in range(4):
            word = (0xAAAAAAAA & ~(3 << bit)) | (code << bit)
            dec = o.decode_i2s_to_i8s(np.uint32(word))
            expect = np.zeros(16, dtype=np.int8)
            expect[e] = code - 2
            assert np.array_equal(dec, expect), (e, code)


def test_decode_matches_unpack_on_random_words():
    rng = np.random.default_rng(7)
    w = rng.integers(-1, 2, size=(16, 32), dtype=np.int8)
    words = o.pack_int2(w).view(np.uint8).reshape(-1).view("<u4")
    dec = o.decode_i2s_to_i8s(words)  # [32, 16]
    for t in range(32):
        row = (t // 16) * 8 + t % 8
        h = (t // 8) % 2
        assert np.array_equal(dec[t], w[row, h * 16 : h * 16 + 16])


@pytest.mark.parametrize("n,k", [(16, 128), (48, 256), (32, 2560), (16, 6912)])
def test_kernel_address_emulation_equals_integer_matmul(n, k):
    rng = np.random.default_rng(n * 131 + k)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    a = rng.integers(-128, 128, size=k, dtype=np.int8)
    got = o.ladder_kernel_emulate(a, o.pack_int2(w), n, k)
    assert np.array_equal(got, o.acc_int32(a[None], w)[0])


def test_acc_invariants():
    rng = np.random.default_rng(11)
    n, k = 32, 256
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    a = rng.integers(-64, 64, size=(3, k), dtype=np.int8)
    b = rng.integers(-63, 64, size=(3, k), dtype=np.int8)
    # brute force on a corner
    assert o.acc_int32(a, w)[1, 5] == sum(int(a[1, i]) * int(w[5, i]) for i in range(k))
    # linearity in the activations
    assert np.array_equal(o.acc_int32((a + b).astype(np.int8), w), o.acc_int32(a, w) + o.acc_int32(b, w))
    # all-zero weights, and a weight matrix that picks single activations
    assert not o.acc_int32(a, np.zeros_like(w)).any()
    pick = np.zeros((16, k), dtype=np.int8)
    pick[np.arange(16), np.arange(16) * 3] = -1
    assert np.array_equal(o.acc_int32(a, pick), -a[:, np.arange(16) * 3].astype(np.int32))


def test_acc_large_path_equals_integer_path():
    rng = np.random.default_rng(12)
    w = rng.integers(-1, 2, size=(272, 2560), dtype=np.int8)
    a = rng.integers(-128, 128, size=(40, 2560), dtype=np.int8)  # 40*272*2560 > 2**24: float64 route
    assert np.array_equal(o.acc_int32(a, w), (a.astype(np.int64) @ w.astype(np.int64).T).astype(np.int32))


def test_ws_num_table_and_slots():
    assert o.ws_num_for_shape(3840, 2560) == 3
    assert o.ws_num_for_shape(2560, 2560) == 1
    assert o.ws_num_for_shape(13824, 2560) == 2
    assert o.ws_num_for_shape(2560, 6912) == 1
    assert o.ws_num_for_shape(4800, 3200) == 6
    assert o.ws_num_for_shape(1024, 1024) == 1
    slot = o.ws_slot(3840, 3)
    # the equal-thirds rule of the kernel, not the 2560/640/640 segments
    assert slot[1279] == 0 and slot[1280] == 1 and slot[2559] == 1 and slot[2560] == 2 and slot[3839] == 2
    assert o.reference_supports(1, 2560, 2560) and not o.reference_supports(2, 2560, 2560)
