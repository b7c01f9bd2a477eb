"""I2_S <-> GPU-layout transcoder against the oracle's two layout statements,
and (on the GPU) the product on a transcoded tensor against the CPU I2_S path."""
import numpy as np
import pytest
import torch

from bitnet_amd import i2s
from oracle import bitlinear_oracle as o


def _ternary(n, k, seed):
    return np.random.default_rng(seed).integers(-1, 2, size=(n, k), dtype=np.int8)


@pytest.mark.parametrize("n,k", [(16, 128), (48, 384), (2560, 2560)])
def test_unpack_and_pack_match_the_oracle(n, k):
    w = _ternary(n, k, n + k)
    codes = o.i2s_pack_x86(w).reshape(-1)
    got = i2s.i2s_unpack(torch.from_numpy(codes), n, k)
    assert np.array_equal(got.numpy(), w)
    assert np.array_equal(i2s.i2s_pack(torch.from_numpy(w)).numpy(), codes)


def test_single_element_lands_where_the_reference_puts_it():
    # element j of a 128-block -> byte j % 32, shift 6 - 2 * (j / 32)   (ggml-bitnet-mad.cpp:82-87)
    for j in (0, 31, 32, 77, 127):
        w = np.zeros((16, 128), dtype=np.int8)
        w[3, j] = 1
        codes = i2s.i2s_pack(torch.from_numpy(w)).numpy().reshape(16, 32)
        base = np.full(32, 0x55, dtype=np.uint8)  # all codes 1 (= weight 0)
        want = base.copy()
        want[j % 32] = (0x55 & ~(3 << (6 - 2 * (j // 32)))) | (2 << (6 - 2 * (j // 32)))
        assert np.array_equal(codes[3], want), j
        assert np.array_equal(codes[2], base)


def test_fusing_three_i2s_tensors_gives_the_gpu_layout_and_scale_slots():
    k = 256
    parts_np = [(_ternary(64, k, 1), 0.0213), (_ternary(32, k, 2), 0.0177), (_ternary(32, k, 3), 0.0251)]
    parts = [(torch.from_numpy(o.i2s_pack_x86(w).reshape(-1)), s, w.shape[0]) for w, s in parts_np]
    packed, scale = i2s.i2s_to_int2(parts, k)
    want = o.pack_int2(np.concatenate([w for w, _ in parts_np], axis=0))
    assert np.array_equal(packed.numpy(), want)
    want_scale = o.f32_to_bf16_bits(np.array([s for _, s in parts_np] + [0.0], dtype=np.float32))
    assert np.array_equal(scale.view(torch.int16).numpy().astype(np.uint16), want_scale)
    back = i2s.int2_to_i2s(packed, scale, [64, 32, 32])
    for (codes, s, _), (codes2, s2) in zip(parts, back):
        assert torch.equal(codes, codes2)
        assert abs(s2 - s) <= s * 2.0 ** -8  # bf16 rounding of the stored scale


def test_stored_tensor_split_and_join():
    w = _ternary(16, 128, 9)
    codes = i2s.i2s_pack(torch.from_numpy(w))
    raw = i2s.join_i2s_tensor(codes, 0.03125)
    assert raw.numel() == 16 * 128 // 4 + 32  # code bytes + 32 (ggml-bitnet-mad.cpp:95-96)
    c2, s2 = i2s.split_i2s_tensor(raw, 16, 128)
    assert torch.equal(c2, codes) and s2 == 0.03125
    with pytest.raises(ValueError):
        i2s.i2s_unpack(codes[:-1], 16, 128)


@pytest.mark.gpu
def test_product_on_a_transcoded_tensor_equals_the_cpu_i2s_path():
    from bitnet_amd import bitlinear

    n, k, m = 2560, 2560, 3
    w = _ternary(n, k, 21)
    y = np.random.default_rng(22).integers(-128, 128, size=(m, k), dtype=np.int8)
    codes = torch.from_numpy(o.i2s_pack_x86(w).reshape(-1)).cuda()
    packed, _ = i2s.i2s_to_int2([(codes, 1.0, n)], k)
    got = bitlinear.bitnet_int8xint2_acc(torch.from_numpy(y).cuda(), packed).cpu().numpy()
    # the CPU stack: sum (w + 1) * y per row, minus sum(y)
    cpu = o.i2s_vec_dot(o.i2s_pack_x86(w), y, n, k) - y.astype(np.int64).sum(axis=1, keepdims=True).astype(np.int32)
    assert np.array_equal(got, cpu)


@pytest.mark.parametrize("layout", ["x86", "neon", "rows4"])
@pytest.mark.parametrize("n,k", [(4, 128), (8, 256), (16, 384)])
def test_every_on_disk_layout_matches_the_reference_loops(layout, n, k):
    """quantize_i2_s writes one of three byte layouts depending on the build (ggml-bitnet-mad.cpp:78-88,
    121-141, 175-186); the oracle restates each as the reference's own loops."""
    w = _ternary(n, k, 7 * n + k)
    want = o.i2s_pack_loops(w, layout)
    got = i2s.i2s_pack(torch.from_numpy(w), layout)
    assert np.array_equal(got.numpy(), want)
    assert np.array_equal(i2s.i2s_unpack(torch.from_numpy(want), n, k, layout).numpy(), w)
    if layout == "x86":
        assert np.array_equal(want, o.i2s_pack_x86(w).reshape(-1))


def test_single_elements_in_the_neon_and_four_row_layouts():
    # neon: element j of a 64-block -> byte j % 16, shift 6 - 2 * (j / 16)   (ggml-bitnet-mad.cpp:179-184)
    for j in (0, 15, 16, 37, 63):
        w = np.zeros((4, 64), dtype=np.int8)
        w[2, j] = -1
        codes = i2s.i2s_pack(torch.from_numpy(w), "neon").numpy().reshape(4, 16)
        want = np.full(16, 0x55, dtype=np.uint8)
        want[j % 16] = 0x55 & ~(3 << (6 - 2 * (j // 16)))  # code 0 in that field
        assert np.array_equal(codes[2], want), j
        assert np.array_equal(codes[1], np.full(16, 0x55, dtype=np.uint8))
    # rows4: row r, column c -> byte (r / 4) * k + c, shift 6 - 2 * (r % 4)   (ggml-bitnet-mad.cpp:127-140)
    for r, c in ((0, 0), (3, 5), (5, 127), (6, 64)):
        w = np.zeros((8, 128), dtype=np.int8)
        w[r, c] = 1
        codes = i2s.i2s_pack(torch.from_numpy(w), "rows4").numpy().reshape(2, 128)
        want = np.full((2, 128), 0x55, dtype=np.uint8)
        want[r // 4, c] = (0x55 & ~(3 << (6 - 2 * (r % 4)))) | (2 << (6 - 2 * (r % 4)))
        assert np.array_equal(codes, want), (r, c)
    with pytest.raises(ValueError):
        i2s.i2s_pack(torch.zeros(6, 128, dtype=torch.int8), "rows4")
    with pytest.raises(ValueError):
        i2s.i2s_unpack(torch.zeros(16 * 96 // 4, dtype=torch.uint8), 16, 96, "x86")
    with pytest.raises(ValueError):
        i2s.i2s_pack(torch.zeros(4, 128, dtype=torch.int8), "avx512")


def test_fusing_and_gguf_round_trip_in_the_neon_layout(tmp_path):
    from bitnet_amd import decoder, gguf

    k = 128
    parts_np = [(_ternary(32, k, 4), 0.02), (_ternary(16, k, 5), 0.03)]
    parts = [(torch.from_numpy(o.i2s_pack_loops(w, "neon")), s, w.shape[0]) for w, s in parts_np]
    packed, scale = i2s.i2s_to_int2(parts, k, "neon")
    assert np.array_equal(packed.numpy(), o.pack_int2(np.concatenate([w for w, _ in parts_np], axis=0)))
    back = i2s.int2_to_i2s(packed, scale, [32, 16], "neon")
    assert all(torch.equal(c, c2) for (c, _, _), (c2, _) in zip(parts, back))
    # a whole (tiny) model through a GGUF file written and read in that layout
    args = decoder.ModelArgs(dim=128, n_layers=1, n_heads=2, n_kv_heads=1, vocab_size=32, ffn_dim=256)
    rng = np.random.default_rng(3)
    st = {}
    for key, (n, kk) in {"attention.wqkv": (256, 128), "attention.wo": (128, 128), "feed_forward.w13": (512, 128),
                         "feed_forward.w2": (128, 256)}.items():
        st[f"layers.0.{key}.weight"] = torch.from_numpy(o.pack_int2(rng.integers(-1, 2, size=(n, kk), dtype=np.int8)))
        st[f"layers.0.{key}.weight_scale"] = torch.tensor([0.02, 0.03, 0.04, 0.0], dtype=torch.bfloat16) if "wqkv" in key else \
            torch.tensor([0.02, 0.03 if "w13" in key else 0.0, 0.0, 0.0], dtype=torch.bfloat16)
    for key, n in (("attention_norm", 128), ("ffn_norm", 128), ("attention.attn_sub_norm", 128), ("feed_forward.ffn_sub_norm", 256)):
        st[f"layers.0.{key}.weight"] = torch.ones(n, dtype=torch.bfloat16)
    st["tok_embeddings.weight"] = torch.zeros(32, 128, dtype=torch.bfloat16)
    st["output.weight"] = st["tok_embeddings.weight"]
    st["norm.weight"] = torch.ones(128, dtype=torch.bfloat16)
    path = str(tmp_path / "neon.gguf")
    gguf.int2_state_to_gguf(st, args, path, embed_dtype=torch.bfloat16, layout="neon")
    with gguf.GGUFReader(path) as r:
        same = gguf.gguf_to_int2_state(r, layout="neon")
        other = gguf.gguf_to_int2_state(r, layout="x86")
    assert all(torch.equal(same[key], st[key]) for key in st)
    assert not torch.equal(other["layers.0.attention.wo.weight"], st["layers.0.attention.wo.weight"])  # the layout matters
