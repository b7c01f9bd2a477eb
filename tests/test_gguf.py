"""GGUF container reader / writer and the GGUF <-> decoder-state mapping.

The container parser is checked against a file assembled byte by byte in this
test from the published GGUF layout (not with the module's own writer); the
tensor contents against the oracle's I2_S and GPU-layout statements and einops
for the rotary row order.  The reference holds no GGUF file and does not vendor
the package that defines the I2_S type id and the tensor names: those two stay
parity unpinned."""
import struct

import numpy as np
import pytest
import torch

from bitnet_amd import decoder, gguf, i2s
from oracle import bitlinear_oracle as o

ARGS = decoder.ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=96, ffn_dim=512)


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _hand_made_file(path, alignment=32, version=3):
    """header, 5 metadata entries, an F32 [2, 3] tensor and an I2_S [16, 128] tensor."""
    w = np.random.default_rng(5).integers(-1, 2, size=(16, 128), dtype=np.int8)
    codes = o.i2s_pack_x86(w).reshape(-1)
    f32 = np.arange(6, dtype=np.float32).reshape(2, 3)
    kv = _s("general.architecture") + struct.pack("<I", 8) + _s("bitnet-b1.58")
    kv += _s("general.file_type") + struct.pack("<II", 4, 40)
    kv += _s("bitnet-b1.58.rope.freq_base") + struct.pack("<If", 6, 500000.0)
    kv += _s("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, 3) + _s("a") + _s("bc") + _s("")
    kv += _s("some.flags") + struct.pack("<IIQ", 9, 7, 2) + struct.pack("<??", True, False)
    n_kv = 5
    if alignment != 32:
        kv += _s("general.alignment") + struct.pack("<II", 4, alignment)
        n_kv += 1
    t0 = f32.tobytes()
    t1 = codes.tobytes() + struct.pack("<f", 0.0625) + b"\0" * 28
    off1 = -(-len(t0) // alignment) * alignment
    infos = _s("first") + struct.pack("<I", 2) + struct.pack("<QQ", 3, 2) + struct.pack("<IQ", 0, 0)  # dims innermost first
    infos += _s("blk.0.attn_q.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 128, 16) + struct.pack("<IQ", 36, off1)
    head = struct.pack("<IIQQ", 0x46554747, version, 2, n_kv) + kv + infos
    pad = -len(head) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad + t0 + b"\0" * (off1 - len(t0)) + t1)
    return w, f32


@pytest.mark.parametrize("alignment,version", [(32, 3), (64, 3), (32, 2)])
def test_reader_on_a_file_assembled_by_hand(tmp_path, alignment, version):
    path = str(tmp_path / "hand.gguf")
    w, f32 = _hand_made_file(path, alignment, version)
    with gguf.GGUFReader(path) as r:
        assert r.version == version and r.alignment == alignment
        assert r.kv["general.architecture"] == "bitnet-b1.58" and r.kv["general.file_type"] == gguf.FTYPE_MOSTLY_I2_S
        assert r.kv["bitnet-b1.58.rope.freq_base"] == 500000.0
        assert r.kv["tokenizer.ggml.tokens"] == ["a", "bc", ""] and r.kv["some.flags"] == [True, False]
        assert r.data_start % alignment == 0
        assert r.tensors["first"].shape == (2, 3) and r.tensors["blk.0.attn_q.weight"].shape == (16, 128)
        assert r.tensors["blk.0.attn_q.weight"].nbytes == 16 * 128 // 4 + 32
        assert torch.equal(r.plain("first"), torch.from_numpy(f32))
        codes, scale, n, k = r.i2s("blk.0.attn_q.weight")
        assert (n, k, scale) == (16, 128, 0.0625)
        assert np.array_equal(i2s.i2s_unpack(codes, n, k).numpy(), w)
        with pytest.raises(gguf.GGUFError):
            r.i2s("first")
        with pytest.raises(gguf.GGUFError):
            r.plain("blk.0.attn_q.weight")


def test_writer_output_reads_back(tmp_path):
    path = str(tmp_path / "w.gguf")
    w = np.random.default_rng(1).integers(-1, 2, size=(32, 256), dtype=np.int8)
    codes = torch.from_numpy(o.i2s_pack_x86(w).reshape(-1))
    kv = {"general.architecture": "x", "n": 7, "neg": -3, "big": 2 ** 40, "eps": 1e-5, "flag": True, "names": ["p", "q"],
          "empty": [], "forced": (2, 65535)}
    tensors = {"a": torch.arange(5, dtype=torch.float32), "b": (codes, 0.5, 32, 256),
               "c": torch.randn(3, 4).to(torch.bfloat16), "d": torch.randn(2, 2, 2).to(torch.float16)}
    gguf.write_gguf(path, kv, tensors)
    with gguf.GGUFReader(path) as r:
        assert r.kv["n"] == 7 and r.kv["neg"] == -3 and r.kv["big"] == 2 ** 40 and r.kv["flag"] is True
        assert r.kv["eps"] == np.float32(1e-5) and r.kv["names"] == ["p", "q"] and r.kv["empty"] == [] and r.kv["forced"] == 65535
        assert list(r.tensors) == ["a", "b", "c", "d"]
        assert all(t.offset % 32 == 0 for t in r.tensors.values())
        assert torch.equal(r.plain("a"), tensors["a"]) and torch.equal(r.plain("c"), tensors["c"]) and torch.equal(r.plain("d"), tensors["d"])
        c2, s2, n, k = r.i2s("b")
        assert torch.equal(c2, codes) and s2 == 0.5 and (n, k) == (32, 256)
    # the same bytes, parsed by hand: magic, version, counts, first key
    with open(path, "rb") as f:
        raw = f.read()
    assert struct.unpack_from("<IIQQ", raw) == (0x46554747, 3, 4, len(kv))
    assert raw[24 : 24 + 8 + 20] == _s("general.architecture")


def test_malformed_files_are_refused(tmp_path):
    path = str(tmp_path / "bad.gguf")
    _hand_made_file(path)
    with open(path, "rb") as f:
        good = f.read()
    cases = {"magic": b"GGUX" + good[4:], "version": good[:4] + struct.pack("<I", 1) + good[8:], "short": good[:10],
             "truncated directory": good[:120], "truncated data": good[:-40]}
    for what, data in cases.items():
        p = str(tmp_path / "case.gguf")
        with open(p, "wb") as f:
            f.write(data)
        with pytest.raises(gguf.GGUFError):
            gguf.GGUFReader(p)


def _decoder_state(seed=0):
    """A packed decoder state dict with known ternary weights, built with the oracle's packer."""
    rng = np.random.default_rng(seed)
    a = ARGS
    hd = a.dim // a.n_heads
    tern = {}
    st = {}

    def lin(key, rows, k):
        ws = [rng.integers(-1, 2, size=(n, k), dtype=np.int8) for n in rows]
        sc = rng.uniform(0.01, 0.05, size=len(rows)).astype(np.float32)
        tern[key] = (ws, sc)
        st[key + ".weight"] = torch.from_numpy(o.pack_int2(np.concatenate(ws, axis=0)))
        scale = torch.zeros(4, dtype=torch.bfloat16)
        scale[: len(rows)] = torch.from_numpy(sc).to(torch.bfloat16)
        st[key + ".weight_scale"] = scale

    g = torch.Generator().manual_seed(seed)
    norm = lambda n: (1 + 0.02 * torch.randn(n, generator=g)).to(torch.bfloat16)
    for layer in range(a.n_layers):
        p = f"layers.{layer}."
        lin(p + "attention.wqkv", [a.n_heads * hd, a.n_kv_heads * hd, a.n_kv_heads * hd], a.dim)
        lin(p + "attention.wo", [a.dim], a.dim)
        lin(p + "feed_forward.w13", [a.ffn_dim, a.ffn_dim], a.dim)
        lin(p + "feed_forward.w2", [a.dim], a.ffn_dim)
        st[p + "attention_norm.weight"] = norm(a.dim)
        st[p + "ffn_norm.weight"] = norm(a.dim)
        st[p + "attention.attn_sub_norm.weight"] = norm(a.dim)
        st[p + "feed_forward.ffn_sub_norm.weight"] = norm(a.ffn_dim)
    st["tok_embeddings.weight"] = (0.02 * torch.randn(a.vocab_size, a.dim, generator=g)).to(torch.bfloat16)
    st["output.weight"] = st["tok_embeddings.weight"]
    st["norm.weight"] = norm(a.dim)
    return st, tern


def test_decoder_state_round_trip_through_a_gguf_file(tmp_path):
    st, _ = _decoder_state(2)
    path = str(tmp_path / "model.gguf")
    gguf.int2_state_to_gguf(st, ARGS, path, embed_dtype=torch.bfloat16)
    with gguf.GGUFReader(path) as r:
        a = gguf.model_args_from_gguf(r)
        assert a == ARGS
        assert r.kv["general.file_type"] == 40
        assert "output.weight" not in r.tensors  # tied
        assert r.tensors["blk.1.ffn_down.weight"].shape == (ARGS.dim, ARGS.ffn_dim)
        assert r.tensors["blk.0.attn_norm.weight"].ggml_type == 0  # norms stay fp32
        back = gguf.gguf_to_int2_state(r)
    assert set(back) == set(st)
    for key in st:
        assert back[key].dtype == st[key].dtype and torch.equal(back[key], st[key]), key
    # the state loads strictly into the kernel-backed decoder's module tree
    model = decoder.Transformer(ARGS)
    model.load_state_dict(back, strict=True)


def test_file_with_hugging_face_row_order_gives_the_decoders_rotary_order(tmp_path):
    """A file as the reference's converter writes it (q/k rows in Hugging Face order, every projection its own
    I2_S tensor with its own fp32 scale) -> wqkv = (q | k | v) with q, k rearranged '(h l d) i -> (h d l) i'."""
    from einops import rearrange

    a = ARGS
    hd = a.dim // a.n_heads
    rng = np.random.default_rng(11)
    arch = "bitnet-b1.58"
    kv = {"general.architecture": arch, f"{arch}.embedding_length": a.dim, f"{arch}.block_count": 1, f"{arch}.feed_forward_length": a.ffn_dim,
          f"{arch}.attention.head_count": a.n_heads, f"{arch}.attention.head_count_kv": a.n_kv_heads}
    shapes = {"attn_q": (a.n_heads * hd, a.dim), "attn_k": (a.n_kv_heads * hd, a.dim), "attn_v": (a.n_kv_heads * hd, a.dim),
              "attn_output": (a.dim, a.dim), "ffn_gate": (a.ffn_dim, a.dim), "ffn_up": (a.ffn_dim, a.dim), "ffn_down": (a.dim, a.ffn_dim)}
    tern, scales, tensors = {}, {}, {"token_embd.weight": torch.zeros(a.vocab_size, a.dim, dtype=torch.float16),
                                     "output_norm.weight": torch.ones(a.dim)}
    for name, (n, k) in shapes.items():
        tern[name] = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
        scales[name] = float(np.float32(rng.uniform(0.01, 0.05)))
        tensors[f"blk.0.{name}.weight"] = (torch.from_numpy(o.i2s_pack_x86(tern[name]).reshape(-1)), scales[name], n, k)
    for name, n in (("attn_norm", a.dim), ("ffn_norm", a.dim), ("attn_sub_norm", a.dim), ("ffn_sub_norm", a.ffn_dim)):
        tensors[f"blk.0.{name}.weight"] = torch.full((n,), 1.5)
    path = str(tmp_path / "hf_order.gguf")
    gguf.write_gguf(path, kv, tensors)
    with gguf.GGUFReader(path) as r:
        args = gguf.model_args_from_gguf(r)
        assert args.vocab_size == a.vocab_size and args.n_layers == 1 and args.norm_eps == 1e-5
        st = gguf.gguf_to_int2_state(r)
    q = rearrange(torch.from_numpy(tern["attn_q"]), "(h l d) i -> (h d l) i", h=a.n_heads, l=2).numpy()
    k_ = rearrange(torch.from_numpy(tern["attn_k"]), "(h l d) i -> (h d l) i", h=a.n_kv_heads, l=2).numpy()
    want = o.pack_int2(np.concatenate([q, k_, tern["attn_v"]], axis=0))
    assert np.array_equal(st["layers.0.attention.wqkv.weight"].numpy(), want)
    want_scale = o.f32_to_bf16_bits(np.array([scales["attn_q"], scales["attn_k"], scales["attn_v"], 0.0], dtype=np.float32))
    assert np.array_equal(st["layers.0.attention.wqkv.weight_scale"].view(torch.int16).numpy().astype(np.uint16), want_scale)
    assert np.array_equal(st["layers.0.feed_forward.w13.weight"].numpy(), o.pack_int2(np.concatenate([tern["ffn_gate"], tern["ffn_up"]], axis=0)))
    assert np.array_equal(st["layers.0.feed_forward.w2.weight"].numpy(), o.pack_int2(tern["ffn_down"]))
    assert np.array_equal(st["layers.0.attention.wo.weight"].numpy(), o.pack_int2(tern["attn_output"]))
    assert st["layers.0.ffn_norm.weight"].dtype == torch.bfloat16 and float(st["layers.0.ffn_norm.weight"][0]) == 1.5
    assert st["output.weight"] is st["tok_embeddings.weight"]


def test_rotary_row_orders_are_inverse():
    from bitnet_amd.checkpoint import rope_rows_hf_to_interleaved

    w = torch.arange(4 * 2 * 8 * 3).reshape(4 * 2 * 8, 3)
    assert torch.equal(gguf.rope_rows_interleaved_to_hf(rope_rows_hf_to_interleaved(w, 4), 4), w)
    with pytest.raises(ValueError):
        gguf.rope_rows_interleaved_to_hf(w[:10], 4)


def test_absurd_counts_are_refused_not_allocated(tmp_path):
    """A count field far beyond the file's size ends in GGUFError before anything is sized by it."""
    p = str(tmp_path / "huge.gguf")
    head = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + _s("k") + struct.pack("<IIQ", 9, 4, 2 ** 62)
    with open(p, "wb") as f:
        f.write(head + b"\0" * 64)
    with pytest.raises(gguf.GGUFError):
        gguf.GGUFReader(p)
    head = struct.pack("<IIQQ", 0x46554747, 3, 2 ** 40, 0)
    with open(p, "wb") as f:
        f.write(head + b"\0" * 64)
    with pytest.raises(gguf.GGUFError):
        gguf.GGUFReader(p)
    head = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 2 ** 50) + b"abc"
    with open(p, "wb") as f:
        f.write(head + b"\0" * 64)
    with pytest.raises(gguf.GGUFError):
        gguf.GGUFReader(p)
