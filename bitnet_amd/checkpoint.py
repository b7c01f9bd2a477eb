"""Checkpoint conversion for the int8 x int2 decoder: Hugging Face safetensors
names -> the decoder's fused tensors -> ternary weights, 4-slot scale vectors
and packed bytes.  Mirrors gpu/convert_safetensors.py:43-93 (tensor names,
q/k row order, fusing, tied LM head) and gpu/convert_checkpoint.py:37-90 (which
tensors are ternarised, how the scale slots are filled) of the reference; the
arithmetic itself lives in convert.py and pack_weight.py.
"""
import os
from typing import Dict, Optional

import torch

from .convert import pack_fused, quant_weight_fp16
from .decoder import ModelArgs


def rope_rows_hf_to_interleaved(w: torch.Tensor, n_heads: int) -> torch.Tensor:
    """Row order of a q/k projection: Hugging Face keeps, per head, the two
    rotary halves one after the other ((h, l, d) with l = 2); the decoder
    rotates adjacent pairs and wants (h, d, l)
    (convert_safetensors.py:43-47, rearrange '(h l d) i -> (h d l) i')."""
    rows, cols = w.shape
    if rows % (2 * n_heads):
        raise ValueError(f"{rows} rows do not split into {n_heads} heads of two halves")
    d = rows // (2 * n_heads)
    return w.reshape(n_heads, 2, d, cols).transpose(1, 2).reshape(rows, cols)


def hf_to_model_state(st: Dict[str, torch.Tensor], args: Optional[ModelArgs] = None) -> Dict[str, torch.Tensor]:
    """Hugging Face BitNet tensors -> the decoder's (unquantised) state dict:
    wqkv = (q | k | v) with q and k in interleaved rotary order, w13 = (gate |
    up), the four norms per layer, and the embedding used for both
    tok_embeddings and output (convert_safetensors.py:49-93)."""
    a = args or ModelArgs()
    out: Dict[str, torch.Tensor] = {}
    for layer in range(a.n_layers):
        b = f"model.layers.{layer}."
        wq = rope_rows_hf_to_interleaved(st[b + "self_attn.q_proj.weight"], a.n_heads)
        wk = rope_rows_hf_to_interleaved(st[b + "self_attn.k_proj.weight"], a.n_kv_heads)
        wv = st[b + "self_attn.v_proj.weight"]
        p = f"layers.{layer}."
        out[p + "attention.wqkv.weight"] = torch.cat([wq, wk, wv], dim=0)
        out[p + "attention.wo.weight"] = st[b + "self_attn.o_proj.weight"]
        out[p + "attention_norm.weight"] = st[b + "input_layernorm.weight"]
        out[p + "ffn_norm.weight"] = st[b + "post_attention_layernorm.weight"]
        out[p + "attention.attn_sub_norm.weight"] = st[b + "self_attn.attn_sub_norm.weight"]
        out[p + "feed_forward.ffn_sub_norm.weight"] = st[b + "mlp.ffn_sub_norm.weight"]
        out[p + "feed_forward.w13.weight"] = torch.cat([st[b + "mlp.gate_proj.weight"], st[b + "mlp.up_proj.weight"]], dim=0)
        out[p + "feed_forward.w2.weight"] = st[b + "mlp.down_proj.weight"]
    out["tok_embeddings.weight"] = st["model.embed_tokens.weight"]
    out["output.weight"] = st["model.embed_tokens.weight"]
    out["norm.weight"] = st["model.norm.weight"]
    return out


def model_state_to_int2(state: Dict[str, torch.Tensor], args: Optional[ModelArgs] = None, with_fp16: bool = False):
    """The decoder's state dict -> what BitLinearKernel modules load: every
    wqkv / w13 / wo / w2 weight is ternarised per sub-tensor (q, k, v; w1, w3),
    packed, and gets a `weight_scale` of four bf16 slots; everything else is
    copied (convert_checkpoint.py:37-80).  with_fp16 also returns the
    dequantised-ternary state of the reference's fp path."""
    a = args or ModelArgs()
    hd = a.dim // a.n_heads
    int2: Dict[str, torch.Tensor] = {}
    fp16: Dict[str, torch.Tensor] = {}
    for key, value in state.items():
        if "wqkv" in key:
            nq, nk = a.n_heads * hd, a.n_kv_heads * hd
            parts = [value[:nq], value[nq : nq + nk], value[nq + nk :]]
        elif "w13" in key:
            parts = [value[: a.ffn_dim], value[a.ffn_dim :]]
        elif "w2" in key or "wo" in key:
            parts = [value]
        else:
            int2[key] = value.clone()
            if with_fp16:
                fp16[key] = value.clone()
            continue
        packed, scale = pack_fused(parts)  # in the checkpoint's own dtype, as the reference does
        int2[key] = packed
        int2[key.replace("weight", "weight_scale")] = scale
        if with_fp16:
            fp16[key] = torch.cat([quant_weight_fp16(p) for p in parts], dim=0)
    return (int2, fp16) if with_fp16 else int2


def convert_hf_checkpoint(safetensors_path: str, output_dir: str, args: Optional[ModelArgs] = None) -> str:
    """model.safetensors -> <output_dir>/model_state_int2.pt (the file name the
    reference's generate.py opens, gpu/generate.py:66-71)."""
    from safetensors.torch import load_file

    state = hf_to_model_state(load_file(safetensors_path), args)
    int2 = model_state_to_int2(state, args)
    os.makedirs(output_dir, exist_ok=True)
    path = os.path.join(output_dir, "model_state_int2.pt")
    torch.save(int2, path)
    return path
