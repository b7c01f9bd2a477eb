"""Weight ternarisation and scale assembly of the int8 x int2 checkpoint
(gpu/convert_checkpoint.py:23-27, 42-77), as plain functions."""
import torch

from .pack_weight import convert_weight_int8_to_int2


def quant_weight_int8(weight: torch.Tensor):
    """absmean ternarisation: s = 1/mean|w|.clamp(1e-5); round(w*s).clamp(-1,1)
    as int8, and 1/s as a 1-element bf16 scale (convert_checkpoint.py:23-27)."""
    s = 1.0 / weight.abs().mean().clamp_(min=1e-5)
    new_weight = (weight * s).round().clamp(-1, 1).to(torch.int8)
    new_scale = (1.0 / s).to(torch.bfloat16)
    return new_weight, new_scale.reshape(1)


def quant_weight_fp16(weight: torch.Tensor) -> torch.Tensor:
    """Dequantised ternary weights of the fp path (convert_checkpoint.py:29-32)."""
    s = 1.0 / weight.abs().mean().clamp_(min=1e-5)
    return (weight * s).round().clamp(-1, 1) / s


def pack_fused(parts):
    """Ternarise each sub-tensor on its own, stack along N, pack, and put the
    scales in consecutive slots of a 4-slot bf16 vector padded with zeros:
    (q, k, v, 0) for wqkv, (w1, w3, 0, 0) for w13, (w, 0, 0, 0) for wo / w2
    (convert_checkpoint.py:42-77).  Returns (packed int8 [N, K/4], bf16 [4])."""
    if not 1 <= len(parts) <= 4:
        raise ValueError("1 to 4 sub-tensors")
    ws, scales = [], []
    for p in parts:
        w, sc = quant_weight_int8(p)
        ws.append(w)
        scales.append(sc)
    scale = torch.zeros(4, dtype=torch.bfloat16)
    scale[: len(scales)] = torch.cat(scales)
    return convert_weight_int8_to_int2(torch.cat(ws, dim=0)), scale
