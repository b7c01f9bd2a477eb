"""Offline weight layout of the int8 x int2 path, written from the closed
form of what the reference packer produces (gpu/pack_weight.py:76-98).

For logical W[n, k] (ternary, stored as code w + 2):
    16-row block nb = n // 16, row r = n % 16
    32-wide k tile kb = k // 32, half h = (k % 32) // 16, element e = k % 16
    int32 word  = (nb * (K // 32) + kb) * 32 + (r // 8) * 16 + h * 8 + r % 8
    bit offset  = (e % 4) * 8 + (e // 4) * 2
i.e. byte (e % 4) of the little-endian word, bits 2 * (e // 4).  The flat byte
buffer is therefore ordered [nb][kb][r // 8][h][r % 8][e % 4], each byte
holding the four codes e // 4 = 0..3 from its low bits up, and is viewed as
int8 [N, K // 4].  Both directions are pure reshapes/permutes, so they run on
whatever device the tensor lives on.
"""
import torch


def _check_shape(N: int, K: int):
    if N % 16 or K % 32:
        raise ValueError(f"need N % 16 == 0 and K % 32 == 0, got {N}x{K}")


def convert_weight_int8_to_int2(weight: torch.Tensor, keep_device: bool = False) -> torch.Tensor:
    """Ternary int8 [N, K] -> packed int8 [N, K // 4]; same name and bytes as
    the reference's function (gpu/pack_weight.py:76), which also returns a
    CPU tensor whatever device the input is on.  keep_device=True leaves the
    result on the input's device."""
    w = torch.as_tensor(weight)
    N, K = w.shape
    _check_shape(N, K)
    if w.numel() and (int(w.min()) < -1 or int(w.max()) > 1):
        raise ValueError("weights must be ternary (-1, 0, +1)")
    q = (w.to(torch.int16) + 2).to(torch.uint8)
    # n -> (nb, r_hi, r_lo), k -> (kb, h, e_hi, e_lo)
    q = q.view(N // 16, 2, 8, K // 32, 2, 4, 4)
    q = q.permute(0, 3, 1, 4, 2, 6, 5)  # nb, kb, r_hi, h, r_lo, e_lo, e_hi
    byt = q[..., 0] | (q[..., 1] << 2) | (q[..., 2] << 4) | (q[..., 3] << 6)
    packed = byt.contiguous().view(torch.int8).reshape(N, K // 4)
    return packed if keep_device else packed.cpu()


def convert_weight_int2_to_int8(packed: torch.Tensor, N: int = None, K: int = None) -> torch.Tensor:
    """Inverse: packed int8 [N, K // 4] -> ternary int8 [N, K] (same device)."""
    p = torch.as_tensor(packed).contiguous()
    N = N or p.shape[0]
    K = K or p.shape[1] * 4
    _check_shape(N, K)
    b = p.view(torch.uint8).reshape(N // 16, K // 32, 2, 2, 8, 4)  # nb, kb, r_hi, h, r_lo, e_lo
    codes = torch.stack([(b >> (2 * i)) & 3 for i in range(4)], dim=-1)  # ..., e_lo, e_hi
    codes = codes.permute(0, 2, 4, 1, 3, 6, 5)  # nb, r_hi, r_lo, kb, h, e_hi, e_lo
    return (codes.reshape(N, K).to(torch.int16) - 2).to(torch.int8)
