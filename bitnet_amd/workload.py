"""Seeded synthetic inputs at the BitNet-b1.58-2B BitLinear shapes
(model dims from gpu/model.py:41-48 of the reference).

Everything is generated with numpy's Philox counter generator so that the
same (shape, seed) gives the same bytes on every machine.
"""
from dataclasses import dataclass

import numpy as np

# (name, K, N, row counts of the sub-tensors that share the fused weight)
SHAPES_2B = (
    ("wqkv", 2560, 3840, (2560, 640, 640)),
    ("wo", 2560, 2560, (2560,)),
    ("w13", 2560, 13824, (6912, 6912)),
    ("w2", 6912, 2560, (2560,)),
)
N_LAYERS_2B = 30

SEED_W = 0x0B170000
SEED_SCALE = 0x0005CA1E
SEED_ACT = 0x0AC70000
SEED_OUTLIER = 0x000711E5


def packed_bytes(K: int, N: int) -> int:
    return K * N // 4


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(seed))


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def ternary_weight(K: int, N: int, shape_id: int, layer: int = 0) -> np.ndarray:
    """int8 [N, K], iid with P(-1) = P(+1) = 0.3, P(0) = 0.4."""
    u = _rng(SEED_W + shape_id + 16 * layer).random((N, K), dtype=np.float32)
    return (u >= np.float32(0.7)).astype(np.int8) - (u < np.float32(0.3)).astype(np.int8)


def weight_scales(K: int, N: int, shape_id: int, parts) -> np.ndarray:
    """bf16 bit patterns [4]: slot j = mean |src| over the rows of sub-tensor
    j of a seeded N(0, 0.02^2) source matrix, zeros in the unused slots."""
    src = _rng(SEED_SCALE + shape_id).standard_normal((N, K), dtype=np.float32) * np.float32(0.02)
    ws = np.zeros(4, dtype=np.float32)
    r0 = 0
    for j, rows in enumerate(parts):
        ws[j] = np.float32(np.mean(np.abs(src[r0 : r0 + rows]), dtype=np.float64))
        r0 += rows
    out = f32_to_bf16_bits(ws)
    out[len(parts) :] = 0
    return out


def activations_bf16(M: int, K: int, shape_id: int, outliers: bool = False) -> np.ndarray:
    """bf16 bit patterns [M, K] of N(0, 1) draws; every row has its own seed.
    outliers=True multiplies a Bernoulli(0.01) subset by 20 before the cast."""
    rows = []
    for m in range(M):
        x = _rng(SEED_ACT + 1000 * shape_id + M + (m << 20)).standard_normal(K, dtype=np.float32)
        if outliers:
            mask = _rng(SEED_OUTLIER + 1000 * shape_id + M + (m << 20)).random(K, dtype=np.float32) < 0.01
            x = np.where(mask, x * np.float32(20.0), x).astype(np.float32)
        rows.append(x)
    return f32_to_bf16_bits(np.stack(rows))


@dataclass
class LayerShape:
    name: str
    shape_id: int
    K: int
    N: int
    parts: tuple

    @property
    def weight_bytes(self) -> int:
        return packed_bytes(self.K, self.N)


def shapes_2b():
    return [LayerShape(n, i, k, nn, p) for i, (n, k, nn, p) in enumerate(SHAPES_2B)]
