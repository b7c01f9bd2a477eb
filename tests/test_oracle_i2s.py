"""Pins the C restatement of the reference's CPU I2_S kernels: layout against
the numpy statement of the three agreeing layout descriptions, values against
the closed form sum((w + 1) * y) and the integer matmul."""
import numpy as np
import pytest

from oracle import bitlinear_oracle as o
from oracle import i2s_cpu


@pytest.fixture(scope="module", autouse=True)
def _built():
    i2s_cpu.build()
    assert i2s_cpu.load().i2s_has_avx2() == 1


def _case(n, k, m, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(-1, 2, size=(n, k), dtype=np.int8), rng.integers(-128, 128, size=(m, k), dtype=np.int8)


def test_layout_matches_numpy_statement_and_hand_example():
    w, _ = _case(8, 256, 1, 0)
    p = i2s_cpu.pack(w)
    assert np.array_equal(p, o.i2s_pack_x86(w))
    assert np.array_equal(o.i2s_unpack_x86(p, 8, 256), w)
    # element e of a block sits in byte e % 32 at bit 6 - 2 * (e // 32)
    one = np.zeros((1, 128), dtype=np.int8)  # all codes 1 -> every byte 0b01010101
    assert np.all(i2s_cpu.pack(one) == 0x55)
    one[0, 37] = 1  # code 2 at byte 5, bits 5:4
    b = i2s_cpu.pack(one)[0]
    assert b[5] == (0x55 & ~(3 << 4)) | (2 << 4) and np.all(np.delete(b, 5) == 0x55)


def test_quantize_classifies_by_sign_and_returns_max():
    src = np.array([[0.5, -0.25, 0.0, 1e-7, -3.0] + [0.0] * 123], dtype=np.float32)
    p, scale = i2s_cpu.quantize(src)
    assert scale == 3.0
    assert list(o.i2s_unpack_x86(p, 1, 128)[0, :5]) == [1, -1, 0, 0, -1]


@pytest.mark.parametrize("n,k", [(4, 128), (16, 2560), (8, 6912), (4, 128 * 33), (12, 128 * 64)])
def test_dot_kernels_return_sum_of_codes_times_y(n, k):
    w, y = _case(n, k, 1, n + k)
    p = i2s_cpu.pack(w)
    want = (w.astype(np.int64) + 1) @ y[0].astype(np.int64)
    for which in ("i2s_vec_dot", "i2s_vec_dot_1x1"):
        got = i2s_cpu.vec_dot(p, y, which)
        assert np.array_equal(got.astype(np.int64), want), which
    assert np.array_equal(want, o.i2s_vec_dot(p, y, n, k)[0])


@pytest.mark.parametrize("m", [1, 2, 4, 5, 8, 16])
def test_gemm_and_bitlinear_equal_integer_matmul(m):
    n, k = 260, 2560
    w, y = _case(n, k, m, 100 + m)
    p = i2s_cpu.pack(w)
    g = i2s_cpu.gemm(p, y)
    assert np.array_equal(g.astype(np.int64), y.astype(np.int64) @ (w.astype(np.int64) + 1).T)
    for threads in (1, 3, 8):
        acc = i2s_cpu.bitlinear_acc(p, y, threads)
        assert np.array_equal(acc, o.acc_int32(y, w)), threads


def test_same_accumulators_as_the_gpu_layout_path():
    """The two packings of the same ternary matrix describe the same product."""
    n, k = 32, 256
    w, y = _case(n, k, 1, 5)
    acc_cpu = i2s_cpu.bitlinear_acc(i2s_cpu.pack(w), y)
    assert np.array_equal(acc_cpu[0], o.ladder_kernel_emulate(y[0], o.pack_int2(w), n, k))
