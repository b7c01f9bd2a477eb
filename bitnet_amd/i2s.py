"""I2_S <-> int8 x int2 weight layout transcoder: lets the GPU library consume
ternary tensors stored in the CPU stack's on-disk format and write them back.

I2_S (src/ggml-bitnet-mad.cpp:51-197 of the reference): codes q = w + 1 in
{0, 1, 2}, four to a byte at bit shifts 6, 4, 2, 0; which four elements share a
byte depends on the build that wrote the tensor (three layouts, see
I2S_LAYOUTS below; the default is the x86 one, blocks of 128 elements with byte
p holding elements p, 32+p, 64+p, 96+p); one fp32 scale (the tensor's max |w|)
follows the n/4 code bytes, and the tensor is padded by 32 bytes.  The GPU
layout is pack_weight.py's.  Everything here is bit shuffling with torch ops
and runs on any device.
"""
import struct
from typing import Sequence, Tuple

import torch

from .pack_weight import convert_weight_int2_to_int8, convert_weight_int8_to_int2

I2S_BLOCK = 128
I2S_TAIL_BYTES = 32  # the scale's four bytes plus alignment padding (ggml-bitnet-mad.cpp:90-96)
# The byte layout depends on the build of the CPU stack that wrote the tensor (the file does not say which):
#   "x86"   blocks of 128 elements: byte p (0..31) = elements p, 32+p, 64+p, 96+p   (ggml-bitnet-mad.cpp:78-88;
#           also what the reference's Python converters write, utils/convert-hf-to-gguf-bitnet.py:705-717)
#   "neon"  blocks of 64 elements:  byte p (0..15) = elements p, 16+p, 32+p, 48+p   (ggml-bitnet-mad.cpp:175-186)
#   "rows4" x86 built without the activation-parallel kernels: byte (r / 4) * k + c = rows 4g .. 4g+3 of column c
#           (ggml-bitnet-mad.cpp:121-141)
# always at bit shifts 6, 4, 2, 0.
I2S_LAYOUTS = {"x86": 128, "neon": 64}


def _check_layout(layout: str, n: int, k: int) -> None:
    if layout == "rows4":
        if n % 4:
            raise ValueError(f"I2_S rows4 layout: {n} rows are not a multiple of 4")
    elif layout in I2S_LAYOUTS:
        if k % I2S_LAYOUTS[layout]:
            raise ValueError(f"I2_S {layout} layout: k = {k} is not a multiple of {I2S_LAYOUTS[layout]}")
    else:
        raise ValueError(f"unknown I2_S layout {layout!r} (x86, neon, rows4)")


def i2s_unpack(codes: torch.Tensor, n: int, k: int, layout: str = "x86") -> torch.Tensor:
    """uint8 [n*k/4] I2_S code bytes -> ternary int8 [n, k]."""
    _check_layout(layout, n, k)
    if codes.numel() != n * k // 4:
        raise ValueError(f"I2_S tensor of {n} x {k}: n*k/4 = {n * k // 4} code bytes expected, got {codes.numel()}")
    shifts = torch.tensor([6, 4, 2, 0], dtype=torch.uint8, device=codes.device)
    if layout == "rows4":
        b = codes.reshape(n // 4, 1, k).to(torch.uint8)
        q = torch.bitwise_and(torch.bitwise_right_shift(b, shifts.reshape(1, 4, 1)), 3)  # [n/4, 4, k]
        return q.reshape(n, k).to(torch.int8) - 1
    blk = I2S_LAYOUTS[layout]
    b = codes.reshape(n, k // blk, 1, blk // 4).to(torch.uint8)
    q = torch.bitwise_and(torch.bitwise_right_shift(b, shifts.reshape(1, 1, 4, 1)), 3)  # [n, blocks, 4, blk/4]
    return (q.reshape(n, k).to(torch.int8) - 1)


def i2s_pack(w: torch.Tensor, layout: str = "x86") -> torch.Tensor:
    """ternary int8 [n, k] -> uint8 [n*k/4] I2_S code bytes."""
    n, k = w.shape
    _check_layout(layout, n, k)
    if w.dtype != torch.int8 or int(w.abs().max()) > 1:
        raise ValueError("ternary int8 weights expected")
    q = (w + 1).to(torch.uint8)
    if layout == "rows4":
        q = q.reshape(n // 4, 4, k)
        return ((q[:, 0] << 6) | (q[:, 1] << 4) | (q[:, 2] << 2) | q[:, 3]).reshape(-1)
    blk = I2S_LAYOUTS[layout]
    q = q.reshape(n, k // blk, 4, blk // 4)
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


def i2s_to_int2(parts: Sequence[Tuple[torch.Tensor, float, int]], k: int, layout: str = "x86"):
    """One to four I2_S tensors that share k -- (code bytes, scale, rows) each,
    e.g. q, k, v of a layer -- fused along N into the GPU layout: returns
    (packed int8 [N, k/4], weight_scale bf16 [4]) as BitLinearKernel holds them.
    The fp32 scales are rounded to bf16, the precision the GPU format stores."""
    if not 1 <= len(parts) <= 4:
        raise ValueError("1 to 4 tensors")
    ws = [i2s_unpack(c, n, k, layout) for c, _, n in parts]
    dev = ws[0].device
    scale = torch.zeros(4, dtype=torch.bfloat16, device=dev)
    scale[: len(parts)] = torch.tensor([s for _, s, _ in parts], dtype=torch.float32, device=dev).to(torch.bfloat16)
    return convert_weight_int8_to_int2(torch.cat(ws, dim=0), keep_device=True), scale


def int2_to_i2s(packed: torch.Tensor, weight_scale: torch.Tensor, rows: Sequence[int], layout: str = "x86"):
    """The inverse: a packed GPU tensor of N = sum(rows) rows -> one
    (code bytes, scale) pair per sub-tensor."""
    n, k4 = packed.shape
    if sum(rows) != n:
        raise ValueError("rows must add up to N")
    w = convert_weight_int2_to_int8(packed)
    out, lo = [], 0
    for i, r in enumerate(rows):
        out.append((i2s_pack(w[lo : lo + r].contiguous(), layout), float(weight_scale[i].float())))
        lo += r
    return out
