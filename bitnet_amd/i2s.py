"""I2_S <-> int8 x int2 weight layout transcoder: lets the GPU library consume
ternary tensors stored in the CPU stack's on-disk format and write them back.

I2_S (x86 flavour, src/ggml-bitnet-mad.cpp:78-91 of the reference): codes
q = w + 1 in {0, 1, 2}; the flat element stream is cut into blocks of 128;
byte p (0..31) of a block holds elements p, 32+p, 64+p, 96+p at bit shifts
6, 4, 2, 0; one fp32 scale (the tensor's max |w|) follows the n/4 code bytes,
and the tensor is padded by 32 bytes.  The GPU layout is pack_weight.py's.
Everything here is bit shuffling with torch ops and runs on any device.
"""
import struct
from typing import Sequence, Tuple

import torch

from .pack_weight import convert_weight_int2_to_int8, convert_weight_int8_to_int2

I2S_BLOCK = 128
I2S_TAIL_BYTES = 32  # the scale's four bytes plus alignment padding (ggml-bitnet-mad.cpp:90-96)


def i2s_unpack(codes: torch.Tensor, n: int, k: int) -> torch.Tensor:
    """uint8 [n*k/4] I2_S code bytes -> ternary int8 [n, k]."""
    if k % I2S_BLOCK or codes.numel() != n * k // 4:
        raise ValueError(f"I2_S tensor of {n} x {k}: need k % 128 == 0 and n*k/4 = {n * k // 4} code bytes, got {codes.numel()}")
    b = codes.reshape(n, k // I2S_BLOCK, 1, 32).to(torch.uint8)
    shifts = torch.tensor([6, 4, 2, 0], dtype=torch.uint8, device=codes.device).reshape(1, 1, 4, 1)
    q = torch.bitwise_and(torch.bitwise_right_shift(b, shifts), 3)  # [n, blocks, 4, 32]
    return (q.reshape(n, k).to(torch.int8) - 1)


def i2s_pack(w: torch.Tensor) -> torch.Tensor:
    """ternary int8 [n, k] -> uint8 [n*k/4] I2_S code bytes."""
    n, k = w.shape
    if k % I2S_BLOCK:
        raise ValueError("k must be a multiple of 128")
    if w.dtype != torch.int8 or int(w.abs().max()) > 1:
        raise ValueError("ternary int8 weights expected")
    q = (w + 1).to(torch.uint8).reshape(n, k // I2S_BLOCK, 4, 32)
    byt = (q[:, :, 0] << 6) | (q[:, :, 1] << 4) | (q[:, :, 2] << 2) | q[:, :, 3]
    return byt.reshape(-1)


def split_i2s_tensor(raw: torch.Tensor, n: int, k: int) -> Tuple[torch.Tensor, float]:
    """The bytes of one I2_S tensor as stored (codes, fp32 scale, padding) ->
    (code bytes [n*k/4], scale)."""
    nb = n * k // 4
    if raw.dtype != torch.uint8 or raw.numel() < nb + 4:
        raise ValueError("uint8 buffer of at least n*k/4 + 4 bytes expected")
    scale = struct.unpack("<f", bytes(raw[nb : nb + 4].cpu().tolist()))[0]
    return raw[:nb], scale


def join_i2s_tensor(codes: torch.Tensor, scale: float) -> torch.Tensor:
    tail = torch.zeros(I2S_TAIL_BYTES, dtype=torch.uint8, device=codes.device)
    tail[:4] = torch.tensor(list(struct.pack("<f", scale)), dtype=torch.uint8, device=codes.device)
    return torch.cat([codes.reshape(-1), tail])


def i2s_to_int2(parts: Sequence[Tuple[torch.Tensor, float, int]], k: int):
    """One to four I2_S tensors that share k -- (code bytes, scale, rows) each,
    e.g. q, k, v of a layer -- fused along N into the GPU layout: returns
    (packed int8 [N, k/4], weight_scale bf16 [4]) as BitLinearKernel holds them.
    The fp32 scales are rounded to bf16, the precision the GPU format stores."""
    if not 1 <= len(parts) <= 4:
        raise ValueError("1 to 4 tensors")
    ws = [i2s_unpack(c, n, k) for c, _, n in parts]
    dev = ws[0].device
    scale = torch.zeros(4, dtype=torch.bfloat16, device=dev)
    scale[: len(parts)] = torch.tensor([s for _, s, _ in parts], dtype=torch.float32, device=dev).to(torch.bfloat16)
    return convert_weight_int8_to_int2(torch.cat(ws, dim=0), keep_device=True), scale


def int2_to_i2s(packed: torch.Tensor, weight_scale: torch.Tensor, rows: Sequence[int]):
    """The inverse: a packed GPU tensor of N = sum(rows) rows -> one
    (code bytes, scale) pair per sub-tensor."""
    n, k4 = packed.shape
    if sum(rows) != n:
        raise ValueError("rows must add up to N")
    w = convert_weight_int2_to_int8(packed)
    out, lo = [], 0
    for i, r in enumerate(rows):
        out.append((i2s_pack(w[lo : lo + r].contiguous()), float(weight_scale[i].float())))
        lo += r
    return out
