"""Checkpoint converter (HF safetensors -> fused decoder tensors -> packed int2
state dict) against independent restatements: einops for the rotary row
order, the oracle for ternarisation, scales and packing."""
import numpy as np
import pytest
import torch

from bitnet_amd import checkpoint, decoder
from oracle import bitlinear_oracle as o

ARGS = decoder.ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=96, ffn_dim=512)


def _hf_state(dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    a = ARGS
    hd = a.dim // a.n_heads
    st = {}
    r = lambda *shape: (torch.randn(*shape, generator=g) * 0.02).to(dtype)
    for layer in range(a.n_layers):
        b = f"model.layers.{layer}."
        st[b + "self_attn.q_proj.weight"] = r(a.n_heads * hd, a.dim)
        st[b + "self_attn.k_proj.weight"] = r(a.n_kv_heads * hd, a.dim)
        st[b + "self_attn.v_proj.weight"] = r(a.n_kv_heads * hd, a.dim)
        st[b + "self_attn.o_proj.weight"] = r(a.dim, a.n_heads * hd)
        st[b + "input_layernorm.weight"] = 1 + r(a.dim)
        st[b + "post_attention_layernorm.weight"] = 1 + r(a.dim)
        st[b + "self_attn.attn_sub_norm.weight"] = 1 + r(a.dim)
        st[b + "mlp.ffn_sub_norm.weight"] = 1 + r(a.ffn_dim)
        st[b + "mlp.gate_proj.weight"] = r(a.ffn_dim, a.dim)
        st[b + "mlp.up_proj.weight"] = r(a.ffn_dim, a.dim)
        st[b + "mlp.down_proj.weight"] = r(a.dim, a.ffn_dim)
    st["model.embed_tokens.weight"] = r(a.vocab_size, a.dim)
    st["model.norm.weight"] = 1 + r(a.dim)
    return st


def test_rotary_row_order_matches_einops():
    from einops import rearrange

    w = torch.arange(4 * 2 * 8 * 3, dtype=torch.float32).reshape(4 * 2 * 8, 3)
    want = rearrange(w, "(h l d) i -> (h d l) i", h=4, l=2)  # the reference's own expression, convert_safetensors.py:44
    assert torch.equal(checkpoint.rope_rows_hf_to_interleaved(w, 4), want)
    # row (h, d, l) of the result is row (h, l, d) of the input: first pair of head 1 = rows 16 and 24
    got = checkpoint.rope_rows_hf_to_interleaved(w, 4)
    assert torch.equal(got[16], w[16]) and torch.equal(got[17], w[24])
    with pytest.raises(ValueError):
        checkpoint.rope_rows_hf_to_interleaved(w[:10], 4)


def test_hf_names_fuse_into_the_decoder_state():
    st = _hf_state()
    state = checkpoint.hf_to_model_state(st, ARGS)
    a = ARGS
    hd = a.dim // a.n_heads
    assert state["layers.1.attention.wqkv.weight"].shape == ((a.n_heads + 2 * a.n_kv_heads) * hd, a.dim)
    assert torch.equal(state["layers.0.attention.wqkv.weight"][a.n_heads * hd + a.n_kv_heads * hd :],
                       st["model.layers.0.self_attn.v_proj.weight"])
    assert torch.equal(state["layers.0.feed_forward.w13.weight"][a.ffn_dim :], st["model.layers.0.mlp.up_proj.weight"])
    assert state["output.weight"] is state["tok_embeddings.weight"] or torch.equal(state["output.weight"], state["tok_embeddings.weight"])
    assert len(state) == 8 * a.n_layers + 3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_int2_state_matches_oracle_and_loads_strict(dtype):
    st = _hf_state(dtype, seed=3)
    state = checkpoint.hf_to_model_state(st, ARGS)
    int2, fp16 = checkpoint.model_state_to_int2(state, ARGS, with_fp16=True)
    a = ARGS
    hd = a.dim // a.n_heads
    # wqkv: three sub-tensors, three scales + a zero slot
    full = state["layers.1.attention.wqkv.weight"]
    bounds = [0, a.n_heads * hd, a.n_heads * hd + a.n_kv_heads * hd, full.shape[0]]
    tern, scales = [], []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        if dtype == torch.float32:
            w, sb = o.quant_weight_int8(full[lo:hi].numpy())
        else:  # the oracle restates the fp32 formula; in bf16 the reference formula itself is the restatement
            sub = full[lo:hi]
            s = 1.0 / sub.abs().mean().clamp_(min=1e-5)
            w = (sub * s).round().clamp(-1, 1).to(torch.int8).numpy()
            sb = (1.0 / s).to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16).reshape(1)
        tern.append(w)
        scales.append(np.asarray(sb, dtype=np.uint16).reshape(-1))
    want_packed = o.pack_int2(np.concatenate(tern, axis=0))
    assert np.array_equal(int2["layers.1.attention.wqkv.weight"].numpy(), want_packed)
    got_scale = int2["layers.1.attention.wqkv.weight_scale"].view(torch.int16).numpy().astype(np.uint16)
    assert np.array_equal(got_scale[:3], np.concatenate(scales)) and got_scale[3] == 0
    # w13: two scales; wo / w2: one
    assert int(int2["layers.0.feed_forward.w13.weight_scale"].view(torch.int16)[2:].abs().sum()) == 0
    assert int(int2["layers.0.feed_forward.w2.weight_scale"].view(torch.int16)[1:].abs().sum()) == 0
    assert int2["layers.0.attention_norm.weight"].dtype == dtype
    # fp path: ternary values times the scale
    d = fp16["layers.1.attention.wo.weight"].float()
    sc = d.abs().max()
    assert set(torch.unique((d / sc).round()).tolist()) <= {-1.0, 0.0, 1.0}
    # what the decoder's modules expect, name for name
    model = decoder.Transformer(ARGS)
    cast = {k: (v if v.dtype in (torch.int8,) or "weight_scale" in k else v.to(model.norm.weight.dtype)) for k, v in int2.items()}
    missing = model.load_state_dict(cast, strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys


def test_convert_hf_checkpoint_file_round_trip(tmp_path):
    from safetensors.torch import save_file

    st = _hf_state(torch.bfloat16, seed=5)
    src = tmp_path / "model.safetensors"
    save_file(st, str(src))
    out = checkpoint.convert_hf_checkpoint(str(src), str(tmp_path / "ckpt"), ARGS)
    loaded = torch.load(out, map_location="cpu", weights_only=True)
    direct = checkpoint.model_state_to_int2(checkpoint.hf_to_model_state(st, ARGS), ARGS)
    assert loaded.keys() == direct.keys()
    for k in direct:
        assert torch.equal(loaded[k], direct[k]), k
