"""CPU oracle for the ternary BitLinear path (numpy).

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module; it is the checker used by tests/, by the smoke entry and by the
cpu_baseline leg of the bench.  Every function restates one piece of the
reference (paths relative to the reference tree) and says where its result
is pinned.

Pinning summary (what independently fixes each function):
  acc_int32            closed form: it IS the integer matmul the reference's
                       own known-answer test uses (gpu/test.py:50-53,61).
  decode_i2s_to_i8s    exhaustive over every 2-bit field position/value.
  pack_int2 / pack_int2_closed_form / unpack_int2
                       staged restatement vs independently derived closed
                       form vs golden bytes written by the reference packer
                       (tests/golden/pack_fixture.npz) vs the kernel
                       emulation below (pack -> emulate == matmul).
  ladder_kernel_emulate thread-by-thread restatement of the CUDA kernel's
                       address arithmetic; must equal acc_int32 + epilogue.
  epilogue_bf16        formula at bitnet_kernels.h:82; special case s=ws=1
                       gives bf16(acc) (gpu/test.py:55-61); bf16 rounding
                       pinned against torch's own float32->bfloat16 cast.
  quant_input          two explicit rounding modes.  Mode 1 is bit-pinned
                       against torch eager evaluating gpu/model.py:69-71 on
                       bf16 tensors.  Mode 0 is bit-pinned against the same
                       expression under torch.compile with Inductor's CPU
                       backend (committed vectors).  The reference runs it
                       under torch.compile on CUDA; that code generator is
                       not available here, so against the CUDA-compiled
                       reference itself mode 0 stays PARITY UNPINNED.
  quant_weight_int8    3-line formula, pinned against torch eager.
  i2s_* (CPU I2_S)     layout has three agreeing statements in the reference;
                       value pinned by the closed form sum((w+1)*y).
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# bf16 helpers (bf16 values are carried as uint16 bit patterns)
# --------------------------------------------------------------------------


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit pattern, round-to-nearest-even (what both
    ``(__nv_bfloat16)float`` at bitnet_kernels.h:82 and torch's cast do)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if np.any(nan):
        r = np.where(nan, np.uint16(0x7FC0), r)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bf16, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


# --------------------------------------------------------------------------
# P: offline weight layout  (gpu/pack_weight.py:5-98)
# --------------------------------------------------------------------------

TILE_N = 16  # wmma_n, pack_weight.py:18
TILE_K = 32  # wmma_k, pack_weight.py:19


def tile_source_coord(i: int, j: int):
    """Where slot (i, j) of the permuted 16x32 tile takes its value from
    (pack_weight.py:5-14)."""
    tid = 2 * i + j // 16
    row = (tid // 16) * 8 + tid % 8
    col = j % 16 + 16 * ((tid % 16) // 8)
    return row, col


def pack_int2(w: np.ndarray) -> np.ndarray:
    """Ternary int8 [N, K] -> packed int8 [N, K/4], staged exactly as the
    reference does it (pack_weight.py:76-98): bias by +2, permute every
    16x32 tile (:17-43), squeeze 4 codes per byte little-end first (:46-53),
    re-order the 16 fields of every int32 (:56-72), flat reshape."""
    w = np.asarray(w)
    n, k = w.shape
    assert n % TILE_N == 0 and k % TILE_K == 0, (n, k)
    q = (w.astype(np.int16) + 2).astype(np.uint8)
    # stage 1: permutation inside each tile
    src_r = np.empty((TILE_N, TILE_K), dtype=np.int64)
    src_c = np.empty((TILE_N, TILE_K), dtype=np.int64)
    for i in range(TILE_N):
        for j in range(TILE_K):
            src_r[i, j], src_c[i, j] = tile_source_coord(i, j)
    tiles = q.reshape(n // TILE_N, TILE_N, k // TILE_K, TILE_K).transpose(0, 2, 1, 3)
    perm = tiles[:, :, src_r, src_c]  # [N/16, K/32, 16, 32]
    # stage 2: 4 codes per byte, code c of a group at bits 2c
    g = perm.reshape(n // TILE_N, k // TILE_K, TILE_N, TILE_K // 4, 4).astype(np.uint32)
    byt = g[..., 0] | (g[..., 1] << 2) | (g[..., 2] << 4) | (g[..., 3] << 6)
    # stage 3: view 4 bytes as one little-endian int32 and move field `o`
    # (bits 2o) to bits (o%4)*8 + (o//4)*2
    words = (
        byt[..., 0::4] | (byt[..., 1::4] << 8) | (byt[..., 2::4] << 16) | (byt[..., 3::4] << 24)
    ).astype(np.uint32)
    out = np.zeros_like(words)
    for o in range(16):
        out |= ((words >> np.uint32(2 * o)) & np.uint32(3)) << np.uint32((o % 4) * 8 + (o // 4) * 2)
    return np.ascontiguousarray(out, dtype="<u4").reshape(-1).view(np.int8).reshape(n, k // 4)


def packed_word_index(n_idx, k_idx, K):
    """Closed form of the layout: for logical W[n, k] return (int32 word
    index in the flat buffer, bit offset of its 2-bit code).  Derived from
    pack_weight.py:5-72 and, independently, from the load addresses of the
    CUDA kernel (bitnet_kernels.h:59-67)."""
    n_idx = np.asarray(n_idx)
    k_idx = np.asarray(k_idx)
    nb, r = n_idx // 16, n_idx % 16
    kb, c = k_idx // 32, k_idx % 32
    h, e = c // 16, c % 16
    t = (r // 8) * 16 + h * 8 + (r % 8)
    word = (nb * (K // 32) + kb) * 32 + t
    bit = (e % 4) * 8 + (e // 4) * 2
    return word, bit


def pack_int2_closed_form(w: np.ndarray) -> np.ndarray:
    w = np.asarray(w)
    n, k = w.shape
    assert n % 16 == 0 and k % 32 == 0
    nn, kk = np.meshgrid(np.arange(n), np.arange(k), indexing="ij")
    word, bit = packed_word_index(nn, kk, k)
    flat = np.zeros(n * k // 16, dtype=np.uint32)
    code = (w.astype(np.int64) + 2).astype(np.uint32)
    np.bitwise_or.at(flat, word.ravel(), (code << bit.astype(np.uint32)).ravel())
    return flat.astype("<u4").view(np.int8).reshape(n, k // 4)


def unpack_int2(packed: np.ndarray, n: int, k: int) -> np.ndarray:
    """Inverse of pack_int2: packed int8 [N, K/4] -> ternary int8 [N, K]."""
    flat = np.ascontiguousarray(packed).view(np.uint8).reshape(-1).view("<u4")
    nn, kk = np.meshgrid(np.arange(n), np.arange(k), indexing="ij")
    word, bit = packed_word_index(nn, kk, k)
    code = (flat[word] >> bit.astype(np.uint32)) & 3
    return (code.astype(np.int16) - 2).astype(np.int8)


# --------------------------------------------------------------------------
# K2: 2-bit -> int8 decoder  (gpu/bitnet_kernels/bitnet_kernels.h:23-44)
# --------------------------------------------------------------------------


def decode_i2s_to_i8s(word: np.ndarray) -> np.ndarray:
    """uint32 word(s) -> [..., 16] int8.  For i in 0..3 the masked word
    ``(word >> 2i) & 0x03030303`` holds elements 4i..4i+3 one per byte; a
    per-byte saturating subtract of 2 maps codes 1,2,3 to -1,0,+1 (code 0,
    never produced by the packer, would give -2)."""
    word = np.asarray(word, dtype=np.uint32)
    out = np.empty(word.shape + (16,), dtype=np.int8)
    for i in range(4):
        m = (word >> np.uint32(2 * i)) & np.uint32(0x03030303)
        for b in range(4):
            out[..., 4 * i + b] = ((m >> np.uint32(8 * b)) & 0xFF).astype(np.int16) - 2
    return out


# --------------------------------------------------------------------------
# K1: shape table  (gpu/bitnet_kernels/bitnet_kernels.cu:4-33)
# --------------------------------------------------------------------------

_WS_NUM_TABLE = {
    (3840, 2560): 3,
    (2560, 2560): 1,
    (13824, 2560): 2,
    (2560, 6912): 1,
    (4800, 3200): 6,
    (3200, 3200): 1,
    (20480, 3200): 2,
    (3200, 10240): 1,
    (5120, 27648): 1,
    (55296, 5120): 1,
}


def ws_num_for_shape(n: int, k: int) -> int:
    """Number of weight-scale slots the reference kernel is instantiated
    with for (N, K); shapes it has no instance for get 1 here."""
    return _WS_NUM_TABLE.get((n, k), 1)


def reference_supports(m: int, n: int, k: int) -> bool:
    return m == 1 and (n, k) in _WS_NUM_TABLE


# --------------------------------------------------------------------------
# K3: accumulators and epilogue  (gpu/bitnet_kernels/bitnet_kernels.h:46-83)
# --------------------------------------------------------------------------


def acc_int32(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    """acc[m, n] = sum_k a[m, k] * w[n, k] with a int8 [M, K], w ternary
    int8 [N, K].  Computed in int64 and checked to fit int32."""
    if a.shape[0] * w.shape[0] * w.shape[1] <= (1 << 24):
        acc = a.astype(np.int64) @ w.astype(np.int64).T
    else:
        # float64 BLAS: every product and partial sum is an integer below 2**53, hence exact
        acc = np.rint(a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64)
    assert np.all(np.abs(acc) < 2**31)
    return acc.astype(np.int32)


def ws_slot(n_total: int, ws_num: int) -> np.ndarray:
    """Scale slot of every output row: out_idx / (N / ws_num)
    (bitnet_kernels.h:80).  Equal-size slots, whatever the true segment
    boundaries of a fused tensor are."""
    return np.arange(n_total) // (n_total // ws_num)


def epilogue_bf16(acc: np.ndarray, s_bits: np.ndarray, ws_bits: np.ndarray, slot: np.ndarray) -> np.ndarray:
    """out = bf16( float(acc) / float(s[m]) * float(ws[slot[n]]) )
    (bitnet_kernels.h:82): one IEEE fp32 divide, one fp32 multiply, one RNE
    cast.  acc int32 [M, N]; s_bits bf16 [M]; ws_bits bf16 [>=max slot+1].
    Returns bf16 bit patterns [M, N]."""
    s = bf16_bits_to_f32(np.asarray(s_bits).reshape(-1))[:, None]
    ws = bf16_bits_to_f32(np.asarray(ws_bits).reshape(-1))[slot][None, :]
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        t = acc.astype(np.float32) / s
        t = (t * ws).astype(np.float32)
    return f32_to_bf16_bits(t)


def bitlinear_int8xint2(a, w, s_bits, ws_bits, ws_num=None):
    """Whole K3 for M >= 1 rows, each with its own s[m] (the reference
    only reads s[0]; M > 1 is its formula applied per row)."""
    n, k = w.shape
    if ws_num is None:
        ws_num = ws_num_for_shape(n, k)
    acc = acc_int32(a, w)
    return acc, epilogue_bf16(acc, s_bits, ws_bits, ws_slot(n, ws_num))


def bitlinear_int8xint2_seg(a, w, s_bits, ws_bits, seg_ends):
    """Variant with true segment boundaries: row n uses ws[j] for the first
    j with n < seg_ends[j] (the layout convert_checkpoint.py:42-77 writes:
    q/k/v or w1/w3 scales in consecutive slots)."""
    n = w.shape[0]
    slot = np.searchsorted(np.asarray(seg_ends), np.arange(n), side="right")
    acc = acc_int32(a, w)
    return acc, epilogue_bf16(acc, s_bits, ws_bits, slot)


def ladder_kernel_emulate(a: np.ndarray, packed: np.ndarray, n: int, k: int) -> np.ndarray:
    """Thread-for-thread emulation of ladder_int8xint2_kernel<1,N,K,...,8,16>
    reading the packed buffer with the kernel's own address arithmetic
    (bitnet_kernels.h:58-78).  Returns the int32 value each block/threadIdx.y
    holds after the 8-lane reduction, i.e. acc[n].  a: int8 [K]."""
    assert n % 16 == 0 and k % 128 == 0
    buf = np.ascontiguousarray(packed).view(np.uint8).reshape(-1)
    a = np.asarray(a, dtype=np.int8).reshape(-1)
    bx = np.arange(n // 16)[:, None, None]  # blockIdx.x
    ty = np.arange(16)[None, :, None]  # threadIdx.y
    tx = np.arange(8)[None, None, :]  # threadIdx.x
    acc = np.zeros((n // 16, 16, 8), dtype=np.int64)
    for k0 in range(k // 128):
        # A_local[j] = A[k0*128 + threadIdx.x*16 + j]            (:59)
        a_loc = a[k0 * 128 + tx[..., None] * 16 + np.arange(16)]  # [1,1,8,16]
        byte_off = (
            bx * 16 * k // 4
            + k0 * 8 * 16 * 16 // 4
            + (tx >> 1) * 32 * 16 // 4
            + (ty >> 3) * (32 * 16 // 2) // 4
            + (tx & 1) * (32 * 16 // 4) // 4
            + (ty & 7) * (32 // 2) // 4
        )
        word = (
            buf[byte_off].astype(np.uint32)
            | (buf[byte_off + 1].astype(np.uint32) << 8)
            | (buf[byte_off + 2].astype(np.uint32) << 16)
            | (buf[byte_off + 3].astype(np.uint32) << 24)
        )
        dec = decode_i2s_to_i8s(word)  # [nb,16,8,16]
        acc += np.sum(dec.astype(np.int64) * a_loc.astype(np.int64), axis=-1)
    return acc.sum(axis=-1).reshape(n).astype(np.int32)


# --------------------------------------------------------------------------
# Q: per-token absmax activation quantizer  (gpu/model.py:68-71)
# --------------------------------------------------------------------------

QUANT_COMPILED = 0  # what torch.compile makes of the expression (fp32 intermediates, bf16 scale)
QUANT_EAGER_BF16 = 1  # torch eager on bf16 tensors: every op rounded to bf16


def quant_input(x_bits: np.ndarray, mode: int = QUANT_COMPILED):
    """x: bf16 bit patterns [M, K].  Returns (q int8 [M, K], s bf16 bits [M]).
    Source expression (gpu/model.py:69-71):
        s = 127 / x.abs().max(-1, keepdim=True).values.clamp_(min=1e-5)
        q = (x * s).round().clamp(-128, 127).to(int8)
    torch evaluates ``127 / t`` as ``t.reciprocal() * 127`` (Tensor.__rtruediv__),
    so both modes take a reciprocal and then multiply.
    mode 0: r = fl32(1 / max(amax, 1e-5f)); s = bf16(fl32(r * 127));
            q = rint(x * f32(s)) -- the product of two bf16 values is exact
            in fp32, so only s is ever rounded to bf16.  This is bit for bit
            what Inductor's CPU backend generates for the expression
            (tests/golden/quant_compiled_fixture.npz).
    mode 1: amax, r, s and the product are each rounded to bf16, as torch
            eager does on bf16 tensors."""
    x = bf16_bits_to_f32(x_bits)
    amax = np.max(np.abs(x), axis=-1, keepdims=True).astype(np.float32)
    one = np.float32(1.0)
    if mode == QUANT_COMPILED:
        amax = np.maximum(amax, np.float32(1e-5))
        r = (one / amax).astype(np.float32)
        sb = bf16_round((r * np.float32(127.0)).astype(np.float32))
        p = (x * sb).astype(np.float32)
    elif mode == QUANT_EAGER_BF16:
        amax = np.maximum(amax, bf16_round(np.float32(1e-5)))
        r = bf16_round((one / amax).astype(np.float32))
        sb = bf16_round((r * np.float32(127.0)).astype(np.float32))
        p = bf16_round((x * sb).astype(np.float32))
    else:
        raise ValueError(mode)
    q = np.clip(np.rint(p), -128, 127).astype(np.int8)
    return q, f32_to_bf16_bits(sb).reshape(-1)


def fake_quant_input(x_bits: np.ndarray, mode: int = QUANT_COMPILED) -> np.ndarray:
    """F: BitLinear.quant_input of the fp path (gpu/model.py:78-81):
    round(x*s).clamp(-128,127)/s as float32; mode 1 rounds the quotient to
    bf16 as eager does, mode 0 leaves it in fp32."""
    q, s_bits = quant_input(x_bits, mode)
    s = bf16_bits_to_f32(s_bits)[:, None]
    # round() keeps the sign of a negative value that rounds to zero
    qf = np.where((q == 0) & (bf16_bits_to_f32(x_bits) < 0), np.float32(-0.0), q.astype(np.float32))
    d = (qf / s).astype(np.float32)
    return bf16_round(d) if mode == QUANT_EAGER_BF16 else d


# --------------------------------------------------------------------------
# Operations around a BitLinear in the decoder  (gpu/model.py:159-166, 195, 237-243)
# --------------------------------------------------------------------------


def rmsnorm_bf16(h_bits: np.ndarray, g_bits: np.ndarray, eps: float) -> np.ndarray:
    """y = bf16(h * rsqrt(mean(h^2) + eps) * g), rows of bf16 bit patterns.
    The reference calls xformers' RMSNorm, which is not in its tree; the
    rounding points are therefore a definition of this build: sum of squares
    in float64 rounded to fp32 and divided by K in fp32, rsqrt as 1/sqrt in fp32, two fp32 multiplies,
    one rounding to bf16.  Pinned against torch's fp32 RMSNorm within 1 bf16
    ulp (it cannot be pinned tighter against a library that is absent)."""
    h = bf16_bits_to_f32(h_bits)
    g = bf16_bits_to_f32(g_bits)
    k = h.shape[-1]
    mean = (np.sum(h.astype(np.float64) ** 2, axis=-1, keepdims=True).astype(np.float32) / np.float32(k)).astype(np.float32)
    rstd = (np.float32(1.0) / np.sqrt((mean + np.float32(eps)).astype(np.float32))).astype(np.float32)
    return f32_to_bf16_bits(((h * rstd).astype(np.float32) * g).astype(np.float32))


def squared_relu_glu_bf16(x13_bits: np.ndarray) -> np.ndarray:
    """[M, 2K] = (x1 | x3) -> h = bf16(bf16(relu(x1)^2) * x3): the reference's
    ``squared_relu(x1) * x3`` (gpu/model.py:164-166, 195) with a bf16 rounding
    after the square and after the product, as torch eager gives."""
    k = x13_bits.shape[-1] // 2
    x1 = bf16_bits_to_f32(x13_bits[..., :k])
    x3 = bf16_bits_to_f32(x13_bits[..., k:])
    r = np.maximum(x1, np.float32(0.0))
    sq = bf16_round((r * r).astype(np.float32))
    return f32_to_bf16_bits((sq * x3).astype(np.float32))


def residual_add_bf16(res_bits: np.ndarray, o_bits: np.ndarray) -> np.ndarray:
    """bf16(res + o) as ``h = x + attention(...)`` does on bf16 tensors."""
    return f32_to_bf16_bits((bf16_bits_to_f32(res_bits) + bf16_bits_to_f32(o_bits)).astype(np.float32))


def norm_bitlinear(x_bits, g_bits, eps, w, ws_bits, glu=False, residual_bits=None, mode=QUANT_COMPILED, ws_num=None,
                   seg_ends=None):
    """[gate ->] RMSNorm -> quantizer -> product -> epilogue [-> residual add];
    with seg_ends the weight scales follow the true segments
    (bitlinear_int8xint2_seg) instead of the equal slots."""
    h = squared_relu_glu_bf16(x_bits) if glu else x_bits
    y = rmsnorm_bf16(h, g_bits, eps)
    q, s_bits = quant_input(y, mode)
    if seg_ends is not None:
        _, out = bitlinear_int8xint2_seg(q, w, s_bits, ws_bits, seg_ends)
    else:
        _, out = bitlinear_int8xint2(q, w, s_bits, ws_bits, ws_num)
    return residual_add_bf16(residual_bits, out) if residual_bits is not None else out


# --------------------------------------------------------------------------
# W: absmean ternarisation  (gpu/convert_checkpoint.py:23-27, 42-77)
# --------------------------------------------------------------------------


def quant_weight_int8(w: np.ndarray):
    """float32 [N, K] -> (ternary int8 [N, K], scale bf16 bits [1]).
    s = 1/mean|w|.clamp(1e-5); w_t = round(w*s).clamp(-1,1); scale = bf16(1/s).
    The mean is taken in float64 and rounded to fp32 (torch reduces fp32
    tensors with wider partial sums; tests allow the last ulp of s to differ
    only where it cannot change any w_t)."""
    w = np.asarray(w, dtype=np.float32)
    mean = np.float32(np.mean(np.abs(w), dtype=np.float64))
    s = np.float32(1.0) / np.maximum(mean, np.float32(1e-5))
    wt = np.clip(np.rint((w * s).astype(np.float32)), -1, 1).astype(np.int8)
    scale = f32_to_bf16_bits(np.array([np.float32(1.0) / s], dtype=np.float32))
    return wt, scale


def fused_weight_and_scales(parts):
    """Fused tensors (wqkv, w13): ternarise every part on its own, stack the
    parts along N and put their scales in consecutive slots of a 4-slot bf16
    vector padded with zeros (convert_checkpoint.py:42-77)."""
    wts, scales = [], []
    for p in parts:
        wt, sc = quant_weight_int8(p)
        wts.append(wt)
        scales.append(sc)
    ws = np.zeros(4, dtype=np.uint16)
    ws[: len(scales)] = np.concatenate(scales)
    return np.concatenate(wts, axis=0), ws


# --------------------------------------------------------------------------
# C: CPU I2_S layout and dot  (src/ggml-bitnet-mad.cpp:51-92, 198-296)
# --------------------------------------------------------------------------

I2S_BLOCK = 128  # QK_I2_S on x86, ggml-bitnet-mad.cpp:12


def i2s_pack_x86(w: np.ndarray) -> np.ndarray:
    """Ternary int8 [N, K] -> uint8 [N, K/4] in the x86 I2_S layout
    (ggml-bitnet-mad.cpp:78-88): codes q = w+1 in {0,1,2}; inside every
    128-element block, byte p (0..31) holds elements p, 32+p, 64+p, 96+p at
    bit shifts 6, 4, 2, 0."""
    w = np.asarray(w)
    n, k = w.shape
    assert k % I2S_BLOCK == 0
    q = (w.astype(np.int16) + 1).astype(np.uint8).reshape(n, k // I2S_BLOCK, 4, 32)
    byt = (q[:, :, 0] << 6) | (q[:, :, 1] << 4) | (q[:, :, 2] << 2) | q[:, :, 3]
    return byt.reshape(n, k // 4).astype(np.uint8)


def i2s_unpack_x86(packed: np.ndarray, n: int, k: int) -> np.ndarray:
    b = np.asarray(packed, dtype=np.uint8).reshape(n, k // I2S_BLOCK, 32)
    q = np.stack([(b >> 6) & 3, (b >> 4) & 3, (b >> 2) & 3, b & 3], axis=2)
    return (q.reshape(n, k).astype(np.int16) - 1).astype(np.int8)


def i2s_pack_loops(w: np.ndarray, layout: str) -> np.ndarray:
    """The three I2_S byte layouts of quantize_i2_s, restated as its own loops
    (small cases only): "x86" = blocks of 128 elements of the flat stream, element
    j of a block -> byte 32 * block + j % 32 at shift 6 - 2 * (j / 32)
    (ggml-bitnet-mad.cpp:80-88); "neon" = blocks of 64, byte 16 * block + j % 16
    at shift 6 - 2 * (j / 16) (:177-186); "rows4" = the x86 build without
    activation-parallel kernels: byte (r / 4) * K + c holds rows 4g..4g+3 of
    column c at shifts 6, 4, 2, 0 (:121-141).  Returns uint8 [N * K / 4]."""
    w = np.asarray(w)
    n, k = w.shape
    q = (w.astype(np.int16) + 1).astype(np.uint8).reshape(-1)
    out = np.zeros(n * k // 4, dtype=np.uint8)
    if layout in ("x86", "neon"):
        blk, grp = (128, 32) if layout == "x86" else (64, 16)
        assert (n * k) % blk == 0
        for i in range(n * k // blk):
            for j in range(blk):
                out[i * grp + j % grp] |= q[i * blk + j] << (6 - 2 * (j // grp))
        return out
    assert layout == "rows4" and n % 4 == 0
    for rg in range(n // 4):
        for c in range(k):
            for r in range(4):
                out[rg * k + c] |= q[(rg * 4 + r) * k + c] << (6 - 2 * r)
    return out


def i2s_vec_dot(packed: np.ndarray, y: np.ndarray, n: int, k: int) -> np.ndarray:
    """What ggml_vec_dot_i2_i8_s returns per weight row (as float in the
    reference, ggml-bitnet-mad.cpp:292-293): sum_k q[k]*y[k] with the
    unsigned codes q = w+1; the caller owes the -sum(y) correction."""
    q = i2s_unpack_x86(packed, n, k).astype(np.int64) + 1
    return (y.astype(np.int64) @ q.T).astype(np.int32)
