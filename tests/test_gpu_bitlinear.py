"""GPU parity tests: every call goes through the C ABI of libbitlinear_hip.so
(via the ctypes host mirror) and is compared with the CPU oracle.

Bars: int32 accumulators bit-exact; bf16 outputs bit-exact against the
oracle's IEEE fp32 divide + multiply + RNE cast (the north star allows
1 bf16 ulp / rel 1e-3; the tests assert the tighter bound and would report
the ulp distance if it ever failed); quantizer outputs bit-exact.
"""
import numpy as np
import pytest
import torch

from bitnet_amd import _lib, bitlinear, pack_weight, workload
from oracle import bitlinear_oracle as o
from tests.gpu_util import bf16_ulp_distance, dev_bf16, dev_i8, host_bits

pytestmark = pytest.mark.gpu

SHAPES_2B = [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912)]  # (N, K)
SHAPES_3B = [(3200, 3200), (4800, 3200), (3200, 10240), (20480, 3200)]


@pytest.fixture(scope="module", autouse=True)
def _need_gpu_and_lib():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    _lib.load_library()  # raises if the HIP library is missing: no fallback
    yield
    _lib.load_library().bitlinear_set_tuning(0, 0, 0, 0)


def _rand_case(n, k, m, seed, full_range=True):
    rng = np.random.default_rng(seed)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    lo, hi = (-128, 128) if full_range else (-128, 127)  # gpu/test.py:48 draws from [-128, 127)
    a = rng.integers(lo, hi, size=(m, k), dtype=np.int8)
    return w, a


def _packed_dev(w):
    return pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w)).cuda()


def _assert_bits_equal(got_bits, want_bits, what):
    if not np.array_equal(got_bits, want_bits):
        d = bf16_ulp_distance(got_bits, want_bits)
        raise AssertionError(f"{what}: {int((d > 0).sum())} of {d.size} differ, max {int(d.max())} bf16 ulp")


@pytest.mark.parametrize("n,k", SHAPES_2B + SHAPES_3B + [(16, 64), (48, 192), (5120, 27648)])
def test_acc_bit_exact_m1(n, k):
    w, a = _rand_case(n, k, 1, seed=n * 7 + k)
    acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
    assert np.array_equal(acc.cpu().numpy(), o.acc_int32(a, w))


@pytest.mark.parametrize("n,k", SHAPES_2B + SHAPES_3B)
def test_reference_known_answer_unit_scales(n, k):
    """The reference's own check (gpu/test.py:42-61): s = ws = 1, output must
    equal the bf16 cast of the integer matmul exactly."""
    w, a = _rand_case(n, k, 1, seed=42 + n + k, full_range=False)
    s = torch.ones(1, dtype=torch.bfloat16, device="cuda")
    ws = torch.ones(6, dtype=torch.bfloat16, device="cuda")
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(a), _packed_dev(w), s, ws)
    want = torch.from_numpy(a.astype(np.int32) @ w.astype(np.int32).T).to(torch.bfloat16)
    assert out.shape == (1, n) and out.dtype == torch.bfloat16
    assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 15, 16, 17, 33])
@pytest.mark.parametrize("n,k", [(2560, 2560), (2560, 6912), (3840, 2560)])
def test_acc_bit_exact_small_m(n, k, m):
    w, a = _rand_case(n, k, m, seed=1000 + m)
    acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
    assert np.array_equal(acc.cpu().numpy(), o.acc_int32(a, w))


def test_acc_extreme_values():
    n, k = 64, 6912
    for wv, av in [(1, -128), (-1, -128), (1, 127), (0, -128)]:
        w = np.full((n, k), wv, dtype=np.int8)
        a = np.full((2, k), av, dtype=np.int8)
        acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
        assert np.array_equal(acc.cpu().numpy(), np.full((2, n), wv * av * k, dtype=np.int32))


def test_acc_single_nonzero_weight_picks_the_activation():
    n, k = 32, 256
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, size=(1, k), dtype=np.int8)
    for r, c, v in [(0, 0, 1), (5, 17, -1), (15, 31, 1), (16, 32, -1), (31, 255, 1), (9, 77, -1), (12, 200, 1)]:
        w = np.zeros((n, k), dtype=np.int8)
        w[r, c] = v
        acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w)).cpu().numpy()
        want = np.zeros((1, n), dtype=np.int32)
        want[0, r] = v * int(a[0, c])
        assert np.array_equal(acc, want), (r, c, v)


@pytest.mark.parametrize("shape_id", [0, 1, 2, 3])
@pytest.mark.parametrize("m", [1, 2, 4, 8, 16])
def test_scaled_output_at_2b_shapes(shape_id, m):
    """Configs 0-2: seeded N(0,1) activations, quantized per token, real
    weight scales in the slots this shape uses."""
    sh = workload.shapes_2b()[shape_id]
    w = workload.ternary_weight(sh.K, sh.N, shape_id)
    ws_bits = workload.weight_scales(sh.K, sh.N, shape_id, sh.parts)
    xb = workload.activations_bf16(m, sh.K, shape_id)
    q, s_bits = o.quant_input(xb, o.QUANT_COMPILED)
    acc, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(q), _packed_dev(w), dev_bf16(s_bits), dev_bf16(ws_bits))
    _assert_bits_equal(host_bits(out), want, f"{sh.name} M={m}")
    # and the whole BitLinearKernel.forward (quantizer + product) in one go
    mod = bitlinear.BitLinearKernel(sh.K, sh.N).cuda()
    mod.weight.data = _packed_dev(w)
    mod.weight_scale.data = dev_bf16(ws_bits)
    out2 = mod(dev_bf16(xb))
    _assert_bits_equal(host_bits(out2), want, f"{sh.name} forward M={m}")


@pytest.mark.parametrize("shape_id", [0, 1, 2, 3])
@pytest.mark.parametrize("m", [1, 2, 4, 8, 16])
def test_default_path_accumulators_bit_exact_at_2b_shapes(shape_id, m):
    """in_thread_C_local after the reduction (gpu/bitnet_kernels/bitnet_kernels.h:74-78),
    read from the kernels the library picks by itself: the accumulator export of
    the drop-in entry must run the kernel the drop-in entry runs, and the
    one-kernel forward (quantizer inside) exports its own.  Seeded workload data."""
    lib = _lib.load_library()
    sh = workload.shapes_2b()[shape_id]
    w = workload.ternary_weight(sh.K, sh.N, shape_id)
    ws_bits = workload.weight_scales(sh.K, sh.N, shape_id, sh.parts)
    xb = workload.activations_bf16(m, sh.K, shape_id)
    q, s_bits = o.quant_input(xb, o.QUANT_COMPILED)
    acc_want, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    pk, qd = _packed_dev(w), dev_i8(q)
    out = bitlinear.bitnet_int8xint2_linear(qd, pk, dev_bf16(s_bits), dev_bf16(ws_bits))
    k_dropin = bitlinear.last_kernel()
    acc = bitlinear.bitnet_int8xint2_acc(qd, pk)
    k_acc = bitlinear.last_kernel()
    assert k_acc == k_dropin, (k_acc, k_dropin)
    # what bench.py's product-only figures time: the LDS-staged kernel up to four tokens, the kernel
    # without staging beyond and on the shape with many row blocks
    assert k_dropin == ("bitlinear_fused_kernel<staged int8>" if (m <= 4 and sh.N // 16 < 432) else "gemv_i2_solo_kernel")
    assert np.array_equal(acc.cpu().numpy(), acc_want), k_acc
    _assert_bits_equal(host_bits(out), want, f"{sh.name} M={m} ({k_dropin})")
    # accumulators and output in ONE call of the export (s and ws given)
    import ctypes

    P = lambda t: ctypes.c_void_p(t.data_ptr())
    acc2 = torch.empty(m, sh.N, dtype=torch.int32, device="cuda")
    out2 = torch.empty(m, sh.N, dtype=torch.bfloat16, device="cuda")
    sd, wsd = dev_bf16(s_bits), dev_bf16(ws_bits)
    assert lib.bitlinear_int8xint2_acc_i32(P(qd), P(pk), P(acc2), P(out2), P(sd), P(wsd), m, sh.N, sh.K, None) == 0
    assert np.array_equal(acc2.cpu().numpy(), acc_want)
    _assert_bits_equal(host_bits(out2), want, "acc export with output")
    # the whole forward: quantizer + product in one kernel while the block is small
    out3, acc3 = bitlinear.bitlinear_forward_acc(dev_bf16(xb), pk, dev_bf16(ws_bits))
    k_fwd = bitlinear.last_kernel()
    if m == 1:
        assert k_fwd == "bitlinear_solo_kernel"  # what bench.py's headline times
    assert np.array_equal(acc3.cpu().numpy(), acc_want), k_fwd
    _assert_bits_equal(host_bits(out3), want, f"{sh.name} forward M={m} ({k_fwd})")


@pytest.mark.parametrize("rb,s_,upw", [(1, 8, 5), (2, 5, 8), (4, 4, 10), (2, 8, 5), (1, 16, 4), (3, 5, 8)])
@pytest.mark.parametrize("m", [1, 5, 16])
def test_fused_kernel_accumulators_for_every_launch_shape(rb, s_, upw, m):
    """The LDS-atomic reduction and the -2 * sum(q) correction of the fused kernel
    with one to four row blocks per workgroup, read as raw int32 (quantizer
    inside, and int8 rows staged)."""
    lib = _lib.load_library()
    n, k = 2560, 2560
    rng = np.random.default_rng(rb * 100 + s_ * 10 + m)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    xb = o.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0, 0, 0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, 0)
    acc_want, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    pk = _packed_dev(w)
    try:
        assert lib.bitlinear_set_tuning(3, rb, s_, upw) == 0
        out, acc = bitlinear.bitlinear_forward_acc(dev_bf16(xb), pk, dev_bf16(ws_bits))
        # (a thread of the one-kernel forward quantizes at most 8 vectors of 8 values: 16 tokens do not fit 512 threads)
        if m * k // 8 <= 8 * 64 * rb * s_:
            assert bitlinear.last_kernel() == "bitlinear_fused_kernel<quantizer>"
        assert lib.bitlinear_set_tuning(6, 1, 0, 0) == 0
        acc_staged = bitlinear.bitnet_int8xint2_acc(dev_i8(q), pk)
        assert bitlinear.last_kernel() == "bitlinear_fused_kernel<staged int8>"
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    assert np.array_equal(acc_staged.cpu().numpy(), acc_want)
    _assert_bits_equal(host_bits(out), want, "forward")


def test_qkv_scale_slots_follow_the_reference_rule_and_seg_variant():
    n, k = 3840, 2560
    w, a = _rand_case(n, k, 2, seed=77)
    s_bits = o.f32_to_bf16_bits(np.array([3.25, 17.5], dtype=np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.011, 0.023, 0.037, 0.0], dtype=np.float32))
    pk = _packed_dev(w)
    _, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)  # equal thirds
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(a), pk, dev_bf16(s_bits), dev_bf16(ws_bits))
    _assert_bits_equal(host_bits(out), want, "equal-slot rule")
    _, want_seg = o.bitlinear_int8xint2_seg(a, w, s_bits, ws_bits, [2560, 3200, 3840])
    out_seg = bitlinear.bitnet_int8xint2_linear_seg(dev_i8(a), pk, dev_bf16(s_bits), dev_bf16(ws_bits), [2560, 3200, 3840])
    _assert_bits_equal(host_bits(out_seg), want_seg, "segment rule")
    assert not np.array_equal(want, want_seg)


@pytest.mark.parametrize("m", [1, 2, 4, 5, 8, 16, 40, 130])
@pytest.mark.parametrize("n,k,ends", [
    (3840, 2560, (2560, 3200, 3840)),   # wqkv as convert_checkpoint.py:42-50 lays its scales out: six runs of 640 rows
    (13824, 2560, (6912, 13824)),       # w13: the segments coincide with the reference's equal halves
    (3840, 2560, (16, 3824, 3840)),     # boundaries whose common divisor leaves more than eight runs: the table kernels
    (2560, 6912, (640, 2560)),
    (1040, 3200, (1040,)),
])
def test_forward_entries_with_segment_scales(n, k, ends, m):
    """bitlinear_forward_bf16_seg and bitlinear_norm_forward_bf16_seg (with and without residual): row n takes the
    weight scale of the segment it lies in.  Bit for bit against the oracle's segmented product behind the oracle's
    quantizer / norm, at decode, batched-decode and prompt sizes; where the segments are the reference's equal slots
    the plain entry gives the same bits, elsewhere it must not."""
    import ctypes

    lib = _lib.load_library()
    rng = np.random.default_rng(n + 3 * k + m + len(ends))
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    xb = o.f32_to_bf16_bits((rng.standard_normal((m, k)) * 1.9).astype(np.float32))
    gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
    rb = o.f32_to_bf16_bits(rng.standard_normal((m, n)).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, o.QUANT_COMPILED)
    _, want = o.bitlinear_int8xint2_seg(q, w, s_bits, ws_bits, ends)
    pk, wsd = _packed_dev(w), dev_bf16(ws_bits)
    mod = bitlinear.BitLinearKernel(k, n, seg_ends=ends).cuda()
    mod.weight.data, mod.weight_scale.data = pk, wsd
    _assert_bits_equal(host_bits(mod(dev_bf16(xb))), want, f"forward, segments {ends}")
    plain = bitlinear.BitLinearKernel(k, n).cuda()
    plain.weight.data, plain.weight_scale.data = pk, wsd
    equal_rule = np.array_equal(np.searchsorted(np.asarray(ends), np.arange(n), side="right"),
                                o.ws_slot(n, o.ws_num_for_shape(n, k)))
    assert np.array_equal(host_bits(plain(dev_bf16(xb))), want) == equal_rule
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    ends_c = (ctypes.c_int * len(ends))(*ends)
    for res in (None, rb):
        want_n = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, residual_bits=res, seg_ends=ends)
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        q_ws = torch.empty(m, k, dtype=torch.int8, device="cuda")
        s_ws = torch.empty(m, dtype=torch.bfloat16, device="cuda")
        r = dev_bf16(res) if res is not None else None
        x, g = dev_bf16(xb), dev_bf16(gb)
        st = lib.bitlinear_norm_forward_bf16_seg(P(x), P(g), 1e-5, 0, P(pk), P(wsd), ends_c, len(ends), P(r), P(out), P(q_ws),
                                                 P(s_ws), m, n, k, 0, None)
        torch.cuda.synchronize()
        assert st == 0
        _assert_bits_equal(host_bits(out), want_n, f"norm forward, segments {ends}, residual {res is not None}")


def test_segment_entries_refuse_bad_segment_lists():
    import ctypes

    lib = _lib.load_library()
    n, k, m = 64, 128, 1
    x = torch.zeros(m, k, dtype=torch.bfloat16, device="cuda")
    pk = torch.zeros(n, k // 4, dtype=torch.int8, device="cuda")
    ws = torch.ones(4, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    for ends in [(32, 48), (48, 32, 64), (0, 64), tuple(range(8, 80, 8))]:
        ends_c = (ctypes.c_int * len(ends))(*ends)
        st = lib.bitlinear_forward_bf16_seg(P(x), P(pk), P(out), P(ws), ends_c, len(ends), None, None, m, n, k, 0, None)
        assert st == 4, ends
        st = lib.bitlinear_norm_forward_bf16_seg(P(x), P(x), 1e-5, 0, P(pk), P(ws), ends_c, len(ends), None, P(out), None,
                                                 None, m, n, k, 0, None)
        assert st == 4, ends
    assert lib.bitlinear_forward_bf16_seg(P(x), P(pk), P(out), P(ws), None, 1, None, None, m, n, k, 0, None) == 2
    with pytest.raises(ValueError):
        bitlinear.BitLinearKernel(k, n, seg_ends=(32, 48))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("m,k", [(1, 2560), (1, 6912), (16, 2560), (5, 27648), (3, 8), (2, 10240)])
def test_quantizer_bit_exact(mode, m, k):
    rng = np.random.default_rng(k + m + mode)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if m > 1:
        x[1] *= 1e-7  # below the clamp
    if m > 2:
        x[2, ::7] *= 20.0
    xb = o.f32_to_bf16_bits(x)
    q, s = bitlinear.quant_input(dev_bf16(xb), mode)
    wq, wsb = o.quant_input(xb, mode)
    assert q.shape == (m, k) and s.shape == (m, 1)
    assert np.array_equal(host_bits(s).reshape(-1), wsb)
    assert np.array_equal(q.cpu().numpy(), wq)


def test_quantizer_matches_committed_torch_vectors():
    import os

    fx = np.load(os.path.join(os.path.dirname(__file__), "golden", "quant_compiled_fixture.npz"))
    for K in (256, 2560):
        for mode, tag in ((0, "compiled"), (1, "eager")):
            q, s = bitlinear.quant_input(dev_bf16(fx[f"x_{K}"]), mode)
            assert np.array_equal(host_bits(s).reshape(-1), fx[f"s_{tag}_{K}"]), (K, tag)
            assert np.array_equal(q.cpu().numpy(), fx[f"q_{tag}_{K}"]), (K, tag)


def test_result_independent_of_kernel_and_launch_shape():
    lib = _lib.load_library()
    n, k = 2560, 6912
    try:
        for m in (1, 3, 4):
            w, a = _rand_case(n, k, m, seed=9 + m)
            pk, ad = _packed_dev(w), dev_i8(a)
            want = o.acc_int32(a, w)
            settings = [(2, wv, u) for wv, u in [(1, 1), (2, 8), (3, 4), (7, 8), (16, 2), (16, 8), (5, 1)]]
            settings += [(0, 0, 0)]
            for setting in settings:
                assert lib.bitlinear_set_tuning(*setting, 0) == 0
                acc = bitlinear.bitnet_int8xint2_acc(ad, pk)
                assert np.array_equal(acc.cpu().numpy(), want), (m, setting)
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)


@pytest.mark.parametrize("n,k", [(16, 64), (16, 128), (48, 192), (80, 320), (32, 3200), (1040, 256)])
@pytest.mark.parametrize("m", [1, 2, 4])
def test_default_kernels_on_ragged_shapes(n, k, m):
    """K not a multiple of 256 (partial last step) and row-block counts that
    do not fill the last workgroup, through whatever the library chooses."""
    w, a = _rand_case(n, k, m, seed=n + k + m)
    acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
    assert np.array_equal(acc.cpu().numpy(), o.acc_int32(a, w))


def _forward_raw(lib, xb, pk, ws_bits, m, n, k, mode, with_ws=True):
    import ctypes

    x = dev_bf16(xb)
    wsd = dev_bf16(ws_bits)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    q = torch.full((m, k), 99, dtype=torch.int8, device="cuda") if with_ws else None
    s = torch.zeros(m, dtype=torch.bfloat16, device="cuda") if with_ws else None
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    st = lib.bitlinear_forward_bf16(P(x), P(pk), P(out), P(wsd), P(q), P(s), m, n, k, mode, None)
    torch.cuda.synchronize()
    return st, out, q, s


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("m", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("n,k", [(2560, 2560), (2560, 6912), (3840, 2560), (48, 192), (1040, 3200)])
def test_fused_forward_equals_oracle_chain(n, k, m, mode):
    """One-kernel forward (or its two-kernel form when the activation block is
    too large) == oracle quantizer -> oracle product, bit for bit, including the
    q / s workspaces it fills."""
    lib = _lib.load_library()
    rng = np.random.default_rng(n + k + m)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if m > 1:
        x[1, ::5] *= 20.0
    xb = o.f32_to_bf16_bits(x)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, mode)
    _, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    st, out, qd, sd = _forward_raw(lib, xb, _packed_dev(w), ws_bits, m, n, k, mode)
    assert st == 0
    _assert_bits_equal(host_bits(out), want, "forward")
    assert np.array_equal(qd.cpu().numpy(), q)
    assert np.array_equal(host_bits(sd), s_bits)


@pytest.mark.parametrize("m", [1, 3, 4])
@pytest.mark.parametrize("n,k", [(20480, 3200), (16384, 2560), (16400, 6912), (55296, 5120)])
def test_many_row_blocks_launch_shape(n, k, m):
    """N >= 16384 with up to 4 tokens runs small workgroups that walk K in
    several rounds (one, two and three rounds, with and without idle k-steps
    in the last one, at these K): the drop-in product and the forward call,
    bit for bit against the oracle."""
    lib = _lib.load_library()
    rng = np.random.default_rng(7 * n + k + m)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    x = rng.standard_normal((m, k)).astype(np.float32)
    xb = o.f32_to_bf16_bits(x)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, 0)
    _, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    pk = _packed_dev(w)
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(q), pk, dev_bf16(s_bits), dev_bf16(ws_bits))
    _assert_bits_equal(host_bits(out), want, "drop-in product")
    st, out2, qd, sd = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
    assert st == 0
    _assert_bits_equal(host_bits(out2), want, "forward")
    assert np.array_equal(qd.cpu().numpy(), q)


@pytest.mark.parametrize("m", [1, 4])
@pytest.mark.parametrize("n,k", [(23088, 21504), (16384, 8192), (17600, 27648)])
def test_many_row_blocks_with_long_rows(n, k, m):
    """N >= 16384 together with K >= 8192: four row blocks per workgroup leave
    room for four waves per block only (a plan with five asked for 1280 threads
    and the launch failed).  Accumulators against the integer product computed
    on the device in fp64 (exact: |acc| < 2^53), drop-in product and forward
    against each other bit for bit."""
    g = torch.Generator(device="cuda").manual_seed(n + k + m)
    w = torch.randint(-1, 2, (n, k), generator=g, device="cuda", dtype=torch.int8)
    a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
    pk = pack_weight.convert_weight_int8_to_int2(w, keep_device=True)
    want = (a.double() @ w.double().t()).to(torch.int32)
    assert torch.equal(bitlinear.bitnet_int8xint2_acc(a, pk), want)
    x = torch.randn(m, k, generator=g, device="cuda").to(torch.bfloat16)
    ws = torch.tensor([0.0161, 0.0, 0.0, 0.0], device="cuda").to(torch.bfloat16)
    mod = bitlinear.BitLinearKernel(k, n).cuda()
    mod.weight.data, mod.weight_scale.data = pk, ws
    q, s = bitlinear.quant_input(x)
    y = bitlinear.bitnet_int8xint2_linear(q, pk, s.reshape(-1), ws)
    assert torch.equal(mod(x).view(torch.int16), y.view(torch.int16))
    acc = (q.double() @ w.double().t()).float()
    want_y = (acc / s.float() * ws[0].float()).to(torch.bfloat16)
    assert torch.equal(y.view(torch.int16), want_y.view(torch.int16))


def _random_shape_cases(count=36, seed=20240611):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        n = 16 * int(rng.integers(1, 260))
        if len(cases) % 6 == 5:
            n = 16 * int(rng.integers(1024, 1400))  # many row blocks: the small-workgroup launch shape
        k = 64 * int(rng.integers(1, 121))
        m = int(rng.integers(1, 17))
        if n * k > 9_000_000:
            continue
        cases.append((n, k, m))
    # the row-block counts at which the library changes kernels or launch shapes (432, 864, 1024, 2048 and
    # their neighbours), at token counts on both sides of its limits, short and decode-sized rows
    for blocks in (431, 432, 433, 863, 864, 865, 1023, 1024, 2047, 2048):
        for k, m in ((192, 1), (320, 5), (2560, 1), (2560, 4), (2560, 16)):
            if blocks * 16 * k <= 45_000_000 and (k < 2560 or blocks in (432, 865, 1023, 2048)):
                cases.append((blocks * 16, k, m))
    return cases


@pytest.mark.parametrize("n,k,m", _random_shape_cases())
def test_random_shapes_product_forward_and_norm_forward(n, k, m):
    """Seeded random (N, K, M) outside the model shapes: ragged row blocks, K that
    no wave count divides, every launch-shape rule; drop-in product, forward and
    norm forward (with residual) against the oracle, bit for bit."""
    import ctypes

    lib = _lib.load_library()
    rng = np.random.default_rng(n * 31 + k * 7 + m)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    x = rng.standard_normal((m, k)).astype(np.float32) * float(rng.choice([0.03, 1.0, 40.0]))
    xb = o.f32_to_bf16_bits(x)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, 0)
    _, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    pk = _packed_dev(w)
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(q), pk, dev_bf16(s_bits), dev_bf16(ws_bits))
    _assert_bits_equal(host_bits(out), want, "drop-in product")
    st, out2, qd, sd = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
    assert st == 0
    _assert_bits_equal(host_bits(out2), want, "forward")
    assert np.array_equal(qd.cpu().numpy(), q)
    assert np.array_equal(host_bits(sd), s_bits)
    # norm forward with a residual
    gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
    rb = o.f32_to_bf16_bits(rng.standard_normal((m, n)).astype(np.float32))
    want_n = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=False, residual_bits=rb)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    xd, g, r, wsd = dev_bf16(xb), dev_bf16(gb), dev_bf16(rb), dev_bf16(ws_bits)
    out3 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    q_ws = torch.empty(m, k, dtype=torch.int8, device="cuda")
    s_ws = torch.empty(m, dtype=torch.bfloat16, device="cuda")
    st = lib.bitlinear_norm_forward_bf16(P(xd), P(g), 1e-5, 0, P(pk), P(wsd), P(r), P(out3), P(q_ws), P(s_ws), m, n, k, 0, None)
    torch.cuda.synchronize()
    assert st == 0
    _assert_bits_equal(host_bits(out3), want_n, "norm forward")


def _random_prefill_cases(count=14, seed=977):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        n = 16 * int(rng.integers(1, 400))
        k = 64 * int(rng.integers(1, 60))
        m = int(rng.integers(17, 700))
        if n * k * m > 1_500_000_000:
            continue
        cases.append((n, k, m))
    return cases


@pytest.mark.parametrize("n,k,m", _random_prefill_cases())
def test_random_shapes_beyond_decode_sizes(n, k, m):
    """Seeded random (N, K, M) with M > 16: whichever of the split-K kernel and
    the MFMA GEMM the library picks, ragged row and column tiles, a ragged last
    k-chunk; int32 accumulators and scaled outputs bit for bit."""
    rng = np.random.default_rng(n + 3 * k + 5 * m)
    w, a = _rand_case(n, k, m, seed=n + k + m)
    s_bits = o.f32_to_bf16_bits((0.5 + 3.0 * rng.random(m)).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    acc_want, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    pk = _packed_dev(w)
    acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), pk)
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(a), pk, dev_bf16(s_bits), dev_bf16(ws_bits))
    _assert_bits_equal(host_bits(out), want, "scaled output")


def test_fused_forward_launch_shapes_and_null_workspaces():
    lib = _lib.load_library()
    n, k = 2560, 2560
    rng = np.random.default_rng(123)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    pk = _packed_dev(w)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0, 0, 0], dtype=np.float32))
    try:
        for m in (1, 3, 4):
            xb = o.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
            q, s_bits = o.quant_input(xb, 0)
            _, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
            for setting in [(3, 1, 10, 4), (3, 1, 5, 8), (3, 2, 5, 8), (3, 4, 4, 10), (3, 2, 8, 5), (3, 1, 16, 4),
                            (3, 4, 1, 16), (3, 1, 3, 4), (4, 0, 0, 0), (0, 0, 0, 0)]:
                assert lib.bitlinear_set_tuning(*setting) == 0
                st, out, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
                assert st == 0, setting
                _assert_bits_equal(host_bits(out), want, f"forward {setting} M={m}")
            lib.bitlinear_set_tuning(0, 0, 0, 0)
            st, out, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0, with_ws=False)
            assert st == 0
            _assert_bits_equal(host_bits(out), want, "forward without workspaces")
        # a block too large for the one-kernel path needs the workspaces
        m, kk = 16, 6912
        xb = o.f32_to_bf16_bits(rng.standard_normal((m, kk)).astype(np.float32))
        wbig = rng.integers(-1, 2, size=(64, kk), dtype=np.int8)
        st, _, _, _ = _forward_raw(lib, xb, _packed_dev(wbig), ws_bits, m, 64, kk, 0, with_ws=False)
        assert st == 2
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)


@pytest.mark.parametrize("m,n,k", [(17, 48, 128), (33, 16, 256), (64, 272, 384), (65, 1040, 640), (100, 2560, 768), (128, 2560, 2560),
                                   (129, 3840, 2560), (300, 1040, 3200), (512, 2560, 6912), (1000, 13824, 2560)])
def test_prefill_gemm_through_the_direct_to_lds_kernel(m, n, k):
    """gemm_i2_prefill_dma_kernel (activation chunks straight into LDS, one weight request per k-step for two
    interleaved column tiles, codes expanded to 64 * w): forced for every shape with K % 128 == 0 -- one to 54
    chunks of 128 or 256 k, chunk counts that leave 0, 1 and 2 chunks behind the loop's rounds of three, ragged
    M and N, a last workgroup whose waves lie partly or wholly beyond N -- accumulators equal to the oracle's,
    bf16 outputs (the reference's scale slots, and explicit segments cutting through a register quad's 8
    columns) equal bit for bit.  (The residual epilogue: test_norm_forward_with_residual_beyond_decode_sizes.)"""
    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=m + n + k)
    s_bits = o.f32_to_bf16_bits(np.linspace(3.0, 90.0, m).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    acc_want, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    ends = [n] if n < 64 else [20, n // 2 + 4, n]  # boundaries inside a register quad's 8 columns
    _, want_seg = o.bitlinear_int8xint2_seg(a, w, s_bits, ws_bits, ends)
    ad, pk, sd, wsd = dev_i8(a), _packed_dev(w), dev_bf16(s_bits), dev_bf16(ws_bits)
    try:
        assert lib.bitlinear_set_tuning(5, 5, 0, 0) == 0
        acc = bitlinear.bitnet_int8xint2_acc(ad, pk)
        name = bitlinear.last_kernel()
        out = bitlinear.bitnet_int8xint2_linear(ad, pk, sd, wsd)
        out_seg = bitlinear.bitnet_int8xint2_linear_seg(ad, pk, sd, wsd, ends)
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert name == "gemm_i2_prefill_dma_kernel"
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    _assert_bits_equal(host_bits(out), want, "direct-to-LDS GEMM")
    _assert_bits_equal(host_bits(out_seg), want_seg, f"direct-to-LDS GEMM, segments {ends}")


@pytest.mark.parametrize("m,n,k", [(512, 2560, 256), (1000, 4368, 384), (500, 8448, 1280), (2017, 2560, 512), (1024, 4112, 2560),
                                   (2100, 2560, 384), (40, 272, 128)])
def test_prefill_gemm_with_tiles_of_two_sizes_in_one_launch(m, n, k):
    """gemm_i2_prefill_mix_kernel: 64 x 256 tiles on the first columns and 32 x 128 tiles (two waves of a workgroup)
    behind them, one launch: all columns in big tiles; a ragged rest of 272 and of 16 columns; ragged M; row tile
    counts that the eight bands do not divide; fewer row tiles than bands; one to ten chunks of 128 or 256 k.
    Accumulators and outputs (equal slots, and segments cutting through a register quad) equal to the oracle's bit
    for bit; M = 2048 at N = 2560 is where the library takes it by itself."""
    assert _lib.plan_name(0, 2048, 2560, 2560).startswith("gemm_i2_prefill_mix_kernel<256> grid=(512,1,1)")
    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=m + n + k)
    s_bits = o.f32_to_bf16_bits(np.linspace(3.0, 90.0, m).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    acc_want, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    ends = [20, n // 2 + 4, n]
    _, want_seg = o.bitlinear_int8xint2_seg(a, w, s_bits, ws_bits, ends)
    ad, pk, sd, wsd = dev_i8(a), _packed_dev(w), dev_bf16(s_bits), dev_bf16(ws_bits)
    try:
        assert lib.bitlinear_set_tuning(5, 8, 0, 0) == 0
        acc = bitlinear.bitnet_int8xint2_acc(ad, pk)
        name = bitlinear.last_kernel()
        out = bitlinear.bitnet_int8xint2_linear(ad, pk, sd, wsd)
        out_seg = bitlinear.bitnet_int8xint2_linear_seg(ad, pk, sd, wsd, ends)
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert name == "gemm_i2_prefill_mix_kernel"
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    _assert_bits_equal(host_bits(out), want, "tiles of two sizes")
    _assert_bits_equal(host_bits(out_seg), want_seg, f"tiles of two sizes, segments {ends}")


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5])
@pytest.mark.parametrize("m,n,k", [(17, 48, 192), (64, 128, 64), (100, 272, 320), (128, 2560, 2560), (129, 3840, 2560),
                                   (300, 1040, 3200), (512, 2560, 6912)])
def test_prefill_gemm_acc_bit_exact(m, n, k, tile):
    """MFMA GEMM path (M > 16), both tile sizes, ragged M and N."""
    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=m + n + k)
    try:
        assert lib.bitlinear_set_tuning(5, tile, 0, 0) == 0
        acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc.cpu().numpy(), o.acc_int32(a, w))


@pytest.mark.parametrize("tile,ks", [(4, 2), (4, 4), (0, 2), (2, 2)])
@pytest.mark.parametrize("m,n,k", [(17, 48, 192), (64, 128, 64), (100, 272, 320), (128, 2560, 2560), (33, 3840, 2560),
                                   (300, 1040, 3200), (512, 2560, 6912), (70, 256, 768), (40, 512, 1024)])
def test_prefill_gemm_with_k_split_between_wave_groups(m, n, k, tile, ks):
    """The small GEMM tiles with 2 or 4 groups of waves splitting a tile's K
    (chunk counts that do and do not divide by the number of groups, a K of
    fewer chunks than groups): accumulators bit-exact, and the scaled bf16
    output equal to the oracle's."""
    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=m + n + k + ks)
    s_bits = o.f32_to_bf16_bits(np.linspace(3.0, 90.0, m).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    _, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    try:
        assert lib.bitlinear_set_tuning(5, tile, 0, ks) == 0
        acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
        out = bitlinear.bitnet_int8xint2_linear(dev_i8(a), _packed_dev(w), dev_bf16(s_bits), dev_bf16(ws_bits))
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc.cpu().numpy(), o.acc_int32(a, w))
    _assert_bits_equal(host_bits(out), want, f"k-split tile={tile} ks={ks}")


def test_prefill_extreme_values_and_split_k_agreement():
    lib = _lib.load_library()
    n, k, m = 256, 6912, 64
    for wv, av in [(1, -128), (-1, -128), (1, 127)]:
        w = np.full((n, k), wv, dtype=np.int8)
        a = np.full((m, k), av, dtype=np.int8)
        acc = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
        assert np.array_equal(acc.cpu().numpy(), np.full((m, n), wv * av * k, dtype=np.int32))
    w, a = _rand_case(512, 1280, 96, seed=4)
    pk, ad = _packed_dev(w), dev_i8(a)
    acc_gemm = bitlinear.bitnet_int8xint2_acc(ad, pk).cpu().numpy()
    try:
        lib.bitlinear_set_tuning(2, 10, 4, 0)  # the split-K kernel, 16 tokens per workgroup
        acc_splitk = bitlinear.bitnet_int8xint2_acc(ad, pk).cpu().numpy()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc_gemm, acc_splitk)


@pytest.mark.parametrize("shape_id", [0, 1, 2, 3])
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_prefill_scaled_output_with_outliers(shape_id, m):
    """Config 3, all twelve (shape, M) pairs: N(0,1) activations with 1% of
    entries x20, quantized per token, through BitLinearKernel.forward (quantizer
    kernel + int8 MFMA GEMM) and through the accumulator export of the drop-in
    entry: quantized rows, scales, int32 accumulators and bf16 outputs of every
    row against the oracle, bit for bit."""
    sh = workload.shapes_2b()[shape_id]
    w = workload.ternary_weight(sh.K, sh.N, shape_id)
    ws_bits = workload.weight_scales(sh.K, sh.N, shape_id, sh.parts)
    xb = workload.activations_bf16(m, sh.K, shape_id, outliers=True)
    q, s_bits = o.quant_input(xb, o.QUANT_COMPILED)
    acc_want, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    mod = bitlinear.BitLinearKernel(sh.K, sh.N).cuda()
    mod.weight.data = _packed_dev(w)
    mod.weight_scale.data = dev_bf16(ws_bits)
    out = mod(dev_bf16(xb))
    assert bitlinear.last_kernel() in ("gemm_i2_prefill_kernel", "gemm_i2_prefill_dma_kernel", "gemm_i2_prefill_mix_kernel")
    _assert_bits_equal(host_bits(out), want, f"{sh.name} prefill M={m}")
    qd, sd = mod.quant_input(dev_bf16(xb))
    assert np.array_equal(qd.cpu().numpy(), q) and np.array_equal(host_bits(sd).reshape(-1), s_bits)
    acc = bitlinear.bitnet_int8xint2_acc(qd, mod.weight.data)
    assert np.array_equal(acc.cpu().numpy(), acc_want)


@pytest.mark.parametrize("shape_id", [0, 1, 2, 3])
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_fp_path_agrees_with_the_int8_path(shape_id, m):
    """The reference runs every M > 1 through its fp module (gpu/model.py:77-85,
    chosen at gpu/generate.py:56-57): fake-quantized bf16 activations times
    dequantised bf16 weights (gpu/convert_checkpoint.py:29-32), a bf16 GEMM with
    fp32 accumulation.  The int8 path computes the same products exactly.  With
    a = q / s the fake-quantized activation and w * ws the dequantised weight,
    the fp result is  sum_k bf16(q_k / s) * bf16(w_k * ws)  and the int8 result
    bf16(acc / s * ws):
      * bf16(w * ws) = +-ws or 0 exactly (ws is a bf16 value), so the weight side adds no error;
      * bf16(q / s) carries a relative rounding error of at most 2^-9 per element
        (the reference rounds the fake-quantized activation to bf16), so the fp
        sum differs from acc / s * ws by at most 2^-9 * sum_k |q_k w_k| / s * ws,
        plus fp32 accumulation error (K * 2^-24 relative to the same sum, below
        2^-11 here) and the final bf16 roundings of both results (2^-9 each,
        relative to the result).
    Asserted per element:  |fp - int8| <= 2^-8 * (sum_k |q_k w_k|) / s * ws + 2^-7 * |int8|.
    The fp module quantizes in eager bf16 arithmetic, so the int8 side runs the
    quantizer mode that is bit-identical to that (mode 1) and both sides see the
    same integers q (asserted).  Config-3 data (1% outliers), every (shape, M) pair."""
    sh = workload.shapes_2b()[shape_id]
    w = workload.ternary_weight(sh.K, sh.N, shape_id)
    ws_bits = workload.weight_scales(sh.K, sh.N, shape_id, sh.parts)
    xb = workload.activations_bf16(m, sh.K, shape_id, outliers=True)
    x = dev_bf16(xb)
    wd = torch.from_numpy(w).cuda()
    ws = dev_bf16(ws_bits)
    # quantizer mode 1 = torch eager on bf16 tensors, which is how the fp module quantizes
    mod = bitlinear.BitLinearKernel(sh.K, sh.N, quant_mode=bitlinear.QUANT_EAGER_BF16).cuda()
    mod.weight.data = _packed_dev(w)
    mod.weight_scale.data = ws
    y_int8 = mod(x).float()
    # the fp module with the weights its converter writes: per sub-tensor (w * scale) in bf16
    # (equal slots here, as the int8 kernel indexes them: bitnet_kernels.h:80)
    ws_num = _lib.load_library().bitlinear_ws_num(sh.N, sh.K)
    slot = torch.arange(sh.N, device="cuda") // (sh.N // ws_num)
    w_fp = (wd.to(torch.bfloat16) * ws[slot][:, None]).to(torch.bfloat16)
    fp = bitlinear.BitLinear(sh.K, sh.N, bias=False, device="cuda", dtype=torch.bfloat16)
    fp.weight.data = w_fp
    with torch.no_grad():
        y_fp = fp(x).float()
    q, s = mod.quant_input(x)
    # both paths multiply the same integers: the fake-quantized activation is bf16(q / s)
    with torch.no_grad():
        assert torch.equal(fp.quant_input(x), q.to(torch.bfloat16) / s)
    mag = (q.double().abs() @ wd.double().abs().t()).float() / s.float() * ws[slot].float()[None, :]
    bound = mag * 2.0 ** -8 + y_int8.abs() * 2.0 ** -7
    excess = (y_fp - y_int8).abs() - bound
    assert float(excess.max()) <= 0.0, f"fp vs int8: worst excess {float(excess.max())} at {sh.name} M={m}"
    # and the bound is not vacuous: typical relative difference is far below one percent
    rel = float((y_fp - y_int8).norm() / y_int8.norm())
    assert rel < 4e-3, rel


@pytest.mark.parametrize("m", [17, 24, 48, 100, 130, 250])
@pytest.mark.parametrize("n,k", [(2560, 2560), (2560, 6912), (13824, 2560)])
def test_mid_size_token_counts_built_in_kernel_choice(n, k, m):
    """Between decode and prefill sizes the library picks the split-K kernel
    or the MFMA GEMM by an estimate of their times: same bits either way."""
    w, a = _rand_case(n, k, m, seed=n + k + m)
    got = bitlinear.bitnet_int8xint2_acc(dev_i8(a), _packed_dev(w))
    assert np.array_equal(got.cpu().numpy(), o.acc_int32(a, w))
    s_bits = o.f32_to_bf16_bits(np.linspace(2.0, 120.0, m).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    _, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    out = bitlinear.bitnet_int8xint2_linear(dev_i8(a), _packed_dev(w), dev_bf16(s_bits), dev_bf16(ws_bits))
    _assert_bits_equal(host_bits(out), want, f"M={m}")


def test_prefill_full_size_linearity_property():
    """M = 2048 at the widest shape, checked without a CPU product: the result
    for activations a + b equals the sum of the results for a and for b."""
    n, k, m = 13824, 2560, 2048
    rng = np.random.default_rng(8)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    a = rng.integers(-64, 64, size=(m, k), dtype=np.int8)
    b = rng.integers(-63, 64, size=(m, k), dtype=np.int8)
    pk = _packed_dev(w)
    ra = bitlinear.bitnet_int8xint2_acc(dev_i8(a), pk)
    rb = bitlinear.bitnet_int8xint2_acc(dev_i8(b), pk)
    rab = bitlinear.bitnet_int8xint2_acc(dev_i8((a + b).astype(np.int8)), pk)
    assert torch.equal(rab, ra + rb)
    # and a few rows against the oracle
    rows = [0, 1, 777, 2047]
    assert np.array_equal(ra[rows].cpu().numpy(), o.acc_int32(a[rows], w))


@pytest.mark.parametrize("glu,res", [(0, 0), (0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("m,path", [(1, 0), (2, 0), (4, 0), (8, 0), (8, 3), (16, 0), (3, 4), (16, 3)])
@pytest.mark.parametrize("n,k", [(2560, 2560), (3840, 2560), (2560, 6912), (48, 192), (1040, 3200)])
def test_fused_norm_gate_residual_forward(n, k, m, path, glu, res):
    """[gate ->] RMSNorm -> quantizer -> product -> epilogue [-> residual]
    against the oracle chain, bit for bit: as one kernel (small blocks, or
    path 3 = forced), and as norm/quantizer kernel + product kernel (large
    blocks, or path 4 = forced)."""
    import ctypes

    lib = _lib.load_library()
    if path == 3 and m * (k + 64) > 60 * 1024:
        pytest.skip("activation block beyond the one-kernel limit")
    if path == 3:
        assert lib.bitlinear_set_tuning(3, 1, 8, 16 if k > 4096 else 5) == 0
    elif path == 4:
        assert lib.bitlinear_set_tuning(4, 0, 0, 0) == 0
    rng = np.random.default_rng(n + k + m + 7 * glu + res)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    xin = rng.standard_normal((m, 2 * k if glu else k)).astype(np.float32) * 1.7
    xb = o.f32_to_bf16_bits(xin)
    gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
    rb = o.f32_to_bf16_bits(rng.standard_normal((m, n)).astype(np.float32)) if res else None
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    want = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=bool(glu), residual_bits=rb)
    x, g, pk, wsd = dev_bf16(xb), dev_bf16(gb), _packed_dev(w), dev_bf16(ws_bits)
    r = dev_bf16(rb) if res else None
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    q_ws = torch.empty(m, k, dtype=torch.int8, device="cuda")
    s_ws = torch.empty(m, dtype=torch.bfloat16, device="cuda")
    try:
        st = lib.bitlinear_norm_forward_bf16(P(x), P(g), 1e-5, glu, P(pk), P(wsd), P(r), P(out), P(q_ws), P(s_ws), m, n, k, 0, None)
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert st == 0
    _assert_bits_equal(host_bits(out), want, f"norm forward glu={glu} res={res}")


@pytest.mark.parametrize("glu,res", [(0, 0), (0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,k,s_,upw", [(2560, 2560, 8, 5), (13824, 2560, 5, 8), (2560, 6912, 16, 7), (48, 192, 1, 4),
                                        (1040, 3200, 10, 5), (1040, 3200, 8, 7), (64, 8192, 16, 8)])
def test_solo_norm_gate_residual_forward(n, k, s_, upw, m, glu, res):
    """The kernel whose waves prepare their own slices, with the RMSNorm / gate
    prologues and the residual epilogue, forced for one to four tokens (the
    library takes it by itself at one token): bit for bit against the oracle
    chain, and the kernel that ran is the one meant."""
    import ctypes

    lib = _lib.load_library()
    rng = np.random.default_rng(3 * n + k + m + 7 * glu + res)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    xin = rng.standard_normal((m, 2 * k if glu else k)).astype(np.float32) * 2.3
    xin[0, 5] = -41.0  # the row maximum sits in one wave's slice
    xb = o.f32_to_bf16_bits(xin)
    gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
    rb = o.f32_to_bf16_bits(rng.standard_normal((m, n)).astype(np.float32)) if res else None
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    want = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=bool(glu), residual_bits=rb)
    x, g, pk, wsd = dev_bf16(xb), dev_bf16(gb), _packed_dev(w), dev_bf16(ws_bits)
    r = dev_bf16(rb) if res else None
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    assert lib.bitlinear_set_tuning(8, 1, s_, upw) == 0
    try:
        st = lib.bitlinear_norm_forward_bf16(P(x), P(g), 1e-5, glu, P(pk), P(wsd), P(r), P(out), None, None, m, n, k, 0, None)
        name = bitlinear.last_kernel()
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert st == 0
    assert name == ("bitlinear_solo_kernel<gate+norm>" if glu else "bitlinear_solo_kernel<norm>")
    _assert_bits_equal(host_bits(out), want, f"solo norm forward glu={glu} res={res}")


def test_norm_forward_without_workspaces_and_beyond_decode_sizes():
    import ctypes

    lib = _lib.load_library()
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    n, k = 2560, 2560
    rng = np.random.default_rng(99)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    gb = o.f32_to_bf16_bits(np.ones(k, dtype=np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.02, 0, 0, 0], dtype=np.float32))
    pk, g, wsd = _packed_dev(w), dev_bf16(gb), dev_bf16(ws_bits)
    # M = 8 without workspaces: still one kernel, same bits
    xb = o.f32_to_bf16_bits(rng.standard_normal((8, k)).astype(np.float32))
    want = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=False, residual_bits=None)
    out = torch.full((8, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    xd8 = dev_bf16(xb)
    st = lib.bitlinear_norm_forward_bf16(P(xd8), P(g), 1e-5, 0, P(pk), P(wsd), None, P(out), None, None, 8, n, k, 0, None)
    torch.cuda.synchronize()
    assert st == 0
    _assert_bits_equal(host_bits(out), want, "norm forward, no workspaces")
    # M = 40: norm/quantizer kernel + MFMA GEMM
    m = 40
    xb = o.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    want = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=False, residual_bits=None)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    q_ws = torch.empty(m, k, dtype=torch.int8, device="cuda")
    s_ws = torch.empty(m, dtype=torch.bfloat16, device="cuda")
    xd = dev_bf16(xb)
    st = lib.bitlinear_norm_forward_bf16(P(xd), P(g), 1e-5, 0, P(pk), P(wsd), None, P(out), P(q_ws), P(s_ws), m, n, k, 0, None)
    torch.cuda.synchronize()
    assert st == 0
    _assert_bits_equal(host_bits(out), want, "norm forward, M=40")
    st = lib.bitlinear_norm_forward_bf16(P(xd), P(g), 1e-5, 0, P(pk), P(wsd), None, P(out), None, None, m, n, k, 0, None)
    assert st != 0


@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("m,n,k,glu", [(40, 2560, 2560, 0), (130, 3840, 2560, 0), (300, 2560, 6912, 1), (77, 48, 192, 1),
                                       (513, 1040, 640, 0), (1030, 64, 2560, 0), (1025, 272, 640, 0), (1024, 48, 4096, 0),
                                       (1026, 32, 6912, 1)])  # from 1024 rows on without the gate: a wave per row
def test_norm_forward_with_residual_beyond_decode_sizes(m, n, k, glu, tile):
    """Prompt-sized blocks: gate / norm / quantizer kernel, then the product with
    the residual added in its epilogue -- through the library's own choice of
    product kernel (tile -1: split-K or GEMM), through every GEMM tile and through the launch with tiles of two
    sizes (8) -- against the oracle chain, bit for bit."""
    import ctypes

    lib = _lib.load_library()
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    rng = np.random.default_rng(m + n + k + glu)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    xb = o.f32_to_bf16_bits(rng.standard_normal((m, 2 * k if glu else k)).astype(np.float32) * 1.3)
    gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
    rb = o.f32_to_bf16_bits(rng.standard_normal((m, n)).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    want = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=bool(glu), residual_bits=rb)
    x, g, pk, wsd, r = dev_bf16(xb), dev_bf16(gb), _packed_dev(w), dev_bf16(ws_bits), dev_bf16(rb)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    q_ws = torch.empty(m, k, dtype=torch.int8, device="cuda")
    s_ws = torch.empty(m, dtype=torch.bfloat16, device="cuda")
    try:
        if tile >= 0:
            assert lib.bitlinear_set_tuning(5, tile, 0, 0) == 0
        st = lib.bitlinear_norm_forward_bf16(P(x), P(g), 1e-5, glu, P(pk), P(wsd), P(r), P(out), P(q_ws), P(s_ws), m, n, k, 0, None)
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert st == 0
    _assert_bits_equal(host_bits(out), want, f"norm forward with residual M={m} tile={tile}")


@pytest.mark.parametrize("m", [1, 3, 5, 8, 13, 16])
@pytest.mark.parametrize("n,k", [(2560, 2560), (13824, 2560), (2560, 6912), (48, 192), (1040, 3200)])
@pytest.mark.parametrize("staged", [1, 2])
def test_product_through_the_lds_staged_kernel(n, k, m, staged):
    """The drop-in entry with the int8 rows staged in LDS (tuning 6 = 1) and
    without (= 2): same bits as the oracle either way."""
    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=n + k + m)
    s_bits = o.f32_to_bf16_bits(np.linspace(3.0, 90.0, m).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    _, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    try:
        assert lib.bitlinear_set_tuning(6, staged, 0, 0) == 0
        out = bitlinear.bitnet_int8xint2_linear(dev_i8(a), _packed_dev(w), dev_bf16(s_bits), dev_bf16(ws_bits))
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    _assert_bits_equal(host_bits(out), want, f"staged={staged} M={m}")


@pytest.mark.parametrize("depth,waves", [(0, 0), (4, 3), (7, 16), (10, 1)])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,k", [(16, 64), (48, 192), (32, 3200), (1040, 256), (3840, 2560), (2560, 6912), (20480, 3200)])
def test_streaming_kernel_bit_exact(n, k, m, depth, waves):
    """The streaming kernel (one wave per 16-row block, activations in LDS, a
    ring of weight loads that runs across row blocks) forced for shapes it would
    not be chosen for: a single row block, a K of one partial step, 12.5 steps,
    runs of one to several row blocks per wave, every ring depth; three scale
    slots at 3840 x 2560.  Accumulators and scaled outputs bit for bit."""
    if (n, k) in ((3840, 2560), (2560, 6912), (20480, 3200)) and (depth, waves) not in ((0, 0), (7, 16)):
        pytest.skip("large shapes: two launch shapes are enough")
    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=n + 3 * k + m)
    s_bits = o.f32_to_bf16_bits(np.linspace(3.0, 90.0, m).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    acc_want, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    pk, ad = _packed_dev(w), dev_i8(a)
    try:
        assert lib.bitlinear_set_tuning(7, 1, depth, waves) == 0
        out = bitlinear.bitnet_int8xint2_linear(ad, pk, dev_bf16(s_bits), dev_bf16(ws_bits))
        assert bitlinear.last_kernel() == "gemv_i2_stream_kernel"
        acc = bitlinear.bitnet_int8xint2_acc(ad, pk)
        assert bitlinear.last_kernel() == "gemv_i2_stream_kernel"
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    _assert_bits_equal(host_bits(out), want, f"stream N={n} K={k} M={m}")


def test_streaming_kernel_is_the_choice_for_the_largest_shape_and_respects_segments():
    """55296 x 5120 (bitnet_kernels.cu:32) at up to four tokens goes through the
    streaming kernel by itself; five tokens do not.  Checked against the integer
    product computed on the device in fp64 (exact).  Scale segments that are not
    multiples of 16 rows keep the call away from it (it takes one slot per row block)."""
    lib = _lib.load_library()
    n, k = 55296, 5120
    g = torch.Generator(device="cuda").manual_seed(55296)
    w = torch.randint(-1, 2, (n, k), generator=g, device="cuda", dtype=torch.int8)
    pk = pack_weight.convert_weight_int8_to_int2(w, keep_device=True)
    ws = torch.tensor([0.0161, 0.0, 0.0, 0.0], device="cuda").to(torch.bfloat16)
    for m, want_kernel in ((1, "gemv_i2_stream_kernel"), (4, "gemv_i2_stream_kernel"), (5, None)):
        a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
        s = (torch.rand(m, generator=g, device="cuda") * 50 + 2).to(torch.bfloat16)
        acc_want = (a.double() @ w.double().t())
        y = bitlinear.bitnet_int8xint2_linear(a, pk, s, ws)
        if want_kernel:
            assert bitlinear.last_kernel() == want_kernel
        else:
            assert bitlinear.last_kernel() != "gemv_i2_stream_kernel"
        assert torch.equal(bitlinear.bitnet_int8xint2_acc(a, pk), acc_want.to(torch.int32))
        want_y = (acc_want.float() / s.float()[:, None] * ws[0].float()).to(torch.bfloat16)
        assert torch.equal(y.view(torch.int16), want_y.view(torch.int16))
    # segments
    n2, k2 = 3840, 2560
    w2, a2 = _rand_case(n2, k2, 2, seed=11)
    s_bits = o.f32_to_bf16_bits(np.array([3.25, 17.5], dtype=np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.011, 0.023, 0.037, 0.0], dtype=np.float32))
    pk2 = _packed_dev(w2)
    try:
        assert lib.bitlinear_set_tuning(7, 1, 0, 0) == 0
        for ends, streams in (([2560, 3200, 3840], True), ([1000, 3001, 3840], False)):
            _, want_seg = o.bitlinear_int8xint2_seg(a2, w2, s_bits, ws_bits, ends)
            out_seg = bitlinear.bitnet_int8xint2_linear_seg(dev_i8(a2), pk2, dev_bf16(s_bits), dev_bf16(ws_bits), ends)
            assert (bitlinear.last_kernel() == "gemv_i2_stream_kernel") == streams
            _assert_bits_equal(host_bits(out_seg), want_seg, f"segments {ends}")
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)


def _grouped_call(lib, problems):
    """problems: list of (a, packed, out, s, ws, M, N, K) device tensors / ints."""
    import ctypes

    arr = (_lib.Problem * max(1, len(problems)))()
    for i, (a, pk, out, s, ws, m, n, k) in enumerate(problems):
        arr[i] = _lib.Problem(a.data_ptr(), pk.data_ptr(), out.data_ptr(), s.data_ptr(), ws.data_ptr(), m, n, k)
    return lib.bitlinear_int8xint2_grouped(arr, len(problems), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))


@pytest.mark.parametrize("shape_id", [0, 1, 2, 3])
@pytest.mark.parametrize("m", [1, 4])
def test_grouped_launch_at_2b_shapes(shape_id, m):
    """bitlinear_int8xint2_grouped over the weights of five layers of one 2B shape
    (distinct weights, activations and scales per problem): one launch of the
    streaming kernel, every problem's output equal to the oracle's bit for bit."""
    lib = _lib.load_library()
    sh = workload.shapes_2b()[shape_id]
    ws_bits = workload.weight_scales(sh.K, sh.N, shape_id, sh.parts)
    problems, wants = [], []
    for layer in range(5):
        w = workload.ternary_weight(sh.K, sh.N, shape_id, layer)
        rng = np.random.default_rng(1000 * shape_id + 10 * layer + m)
        xb = o.f32_to_bf16_bits(rng.standard_normal((m, sh.K)).astype(np.float32) * (1.0 + layer))
        q, s_bits = o.quant_input(xb, o.QUANT_COMPILED)
        _, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
        wants.append(want)
        out = torch.full((m, sh.N), float("nan"), dtype=torch.bfloat16, device="cuda")
        problems.append((dev_i8(q), _packed_dev(w), out, dev_bf16(s_bits), dev_bf16(ws_bits), m, sh.N, sh.K))
    assert _grouped_call(lib, problems) == 0
    assert bitlinear.last_kernel() == "gemv_i2_stream_kernel"
    torch.cuda.synchronize()
    for i, (p, want) in enumerate(zip(problems, wants)):
        _assert_bits_equal(host_bits(p[2]), want, f"{sh.name} problem {i}")


def test_grouped_launch_mixed_shapes_long_runs_and_errors():
    """Runs of equal shape become one launch each, more than 48 equal problems
    several, M > 4 and lone problems go through the ordinary choice of kernel;
    an empty list is fine; a bad element is refused before anything is launched."""
    lib = _lib.load_library()
    rng = np.random.default_rng(77)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    wsd = dev_bf16(ws_bits)
    spec = [(3840, 2560, 1), (3840, 2560, 1), (2560, 2560, 2), (2560, 6912, 8), (2560, 6912, 8), (2560, 2560, 2), (48, 192, 3)]
    spec += [(64, 256, 1)] * 53
    problems, wants = [], []
    for (n, k, m) in spec:
        w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
        a = rng.integers(-128, 128, size=(m, k), dtype=np.int8)
        s_bits = o.f32_to_bf16_bits((2.0 + 50.0 * rng.random(m)).astype(np.float32))
        _, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
        wants.append(want)
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        problems.append((dev_i8(a), _packed_dev(w), out, dev_bf16(s_bits), wsd, m, n, k))
    assert _grouped_call(lib, problems) == 0
    torch.cuda.synchronize()
    for i, (p, want) in enumerate(zip(problems, wants)):
        _assert_bits_equal(host_bits(p[2]), want, f"problem {i} {spec[i]}")
    assert _grouped_call(lib, []) == 0
    # a bad shape in the middle: status 1, and the outputs in front of it stay untouched
    for p in problems[:3]:
        p[2].fill_(float("nan"))
    bad = list(problems[:3])
    bad[2] = bad[2][:5] + (2, 100, 2560)
    assert _grouped_call(lib, bad) == 1
    torch.cuda.synchronize()
    assert torch.isnan(problems[0][2].float()).all()
    # in a captured graph, replayed
    good = problems[:2]
    for p in good:
        p[2].zero_()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        assert _grouped_call(lib, good) == 0
    for _ in range(3):
        for p in good:
            p[2].zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for p, want in zip(good, wants[:2]):
            _assert_bits_equal(host_bits(p[2]), want, "grouped graph replay")


@pytest.mark.parametrize("coop", [0, 1, 2])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,k,shape", [(2560, 2560, (1, 8, 5)), (2560, 2560, (2, 5, 8)), (3840, 2560, (1, 10, 4)),
                                       (13824, 2560, (3, 5, 8)), (13824, 2560, (0, 0, 0)), (2560, 6912, (1, 16, 7)),
                                       (48, 192, (1, 1, 4)), (48, 192, (3, 3, 4)), (1040, 3200, (1, 7, 8)),
                                       (64, 8192, (1, 16, 8)), (3200, 3200, (0, 0, 0)), (32, 64, (0, 0, 0))])
def test_forward_kernel_whose_waves_quantize_their_own_slices(n, k, m, shape, coop):
    """bitlinear_solo_kernel: forced launch shapes (row blocks per workgroup, waves
    per row block, k-steps per wave; (0, 0, 0) = the library's own plan at one
    token), K that no wave count divides, a row of a single partial k-step, three
    scale slots; int32 accumulators, bf16 outputs and the q / s workspaces bit for
    bit against the oracle chain, with and without workspaces; both ways of taking
    the row maximum (rows too long for a wave to scan fall back to the exchange)."""
    lib = _lib.load_library()
    if shape == (0, 0, 0):
        shape = (1, 16, 8) if k > 4096 else ((1, 10, 5) if k > 2560 else (1, 8, 5))  # what the library's plan may not take
    rng = np.random.default_rng(n + 5 * k + m)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    x = rng.standard_normal((m, k)).astype(np.float32) * float(rng.choice([0.05, 1.0, 30.0]))
    if m > 1:
        x[1, ::5] *= 20.0
    xb = o.f32_to_bf16_bits(x)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, 0)
    acc_want, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    pk = _packed_dev(w)
    try:
        assert lib.bitlinear_set_tuning(8, *shape) == 0
        assert lib.bitlinear_set_tuning(9, coop, 0, 0) == 0  # row maximum: built-in choice / exchanged between waves / every wave scans
        out, acc = bitlinear.bitlinear_forward_acc(dev_bf16(xb), pk, dev_bf16(ws_bits))
        assert bitlinear.last_kernel() == "bitlinear_solo_kernel"
        st, out2, qd, sd = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
        assert st == 0 and bitlinear.last_kernel() == "bitlinear_solo_kernel"
        st, out3, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0, with_ws=False)
        assert st == 0
        # quantizer mode 1 is not this kernel's: the built-in kernels take over
        st, out4, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 1)
        assert st == 0 and bitlinear.last_kernel() != "bitlinear_solo_kernel"
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    for t, what in ((out, "forward + acc"), (out2, "forward"), (out3, "forward without workspaces")):
        _assert_bits_equal(host_bits(t), want, what)
    assert np.array_equal(qd.cpu().numpy(), q)
    assert np.array_equal(host_bits(sd), s_bits)
    q1, s1 = o.quant_input(xb, 1)
    _, want1 = o.bitlinear_int8xint2(q1, w, s1, ws_bits)
    _assert_bits_equal(host_bits(out4), want1, "mode 1")


TOK_SHAPES = [(2560, 2560), (3840, 2560), (13824, 2560), (13840, 2560), (7008, 2560), (1040, 3200), (48, 192), (176, 4480),
              (64, 5120), (2560, 6912)]


@pytest.mark.parametrize("m", [1, 2, 5, 7, 8, 9])
@pytest.mark.parametrize("n,k", TOK_SHAPES)
def test_forward_kernel_whose_lanes_quantize_for_their_own_token(n, k, m):
    """bitlinear_solo_tok_kernel (one launch for up to eight tokens; the library's choice from five tokens on for
    rows of up to 3200 values): int32 accumulators, bf16 outputs and the q / s workspaces bit for bit against the
    oracle chain, with and without workspaces, over 1 and 4 row blocks per wave (13840 rows: a last workgroup with
    one row block of its four), one to sixteen waves, K that the waves do not divide, three scale slots; where the kernel has no launch shape (nine tokens, K = 6912, 7008
    rows) the other kernels give the same."""
    lib = _lib.load_library()
    rng = np.random.default_rng(n + 3 * k + m)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    x = rng.standard_normal((m, k)).astype(np.float32) * rng.choice([0.05, 1.0, 30.0], size=(m, 1)).astype(np.float32)
    x[m // 2, ::5] *= 20.0
    x[m - 1, k - 1] = 97.0  # the last token's maximum sits in the last wave's slice
    xb = o.f32_to_bf16_bits(x)
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    q, s_bits = o.quant_input(xb, 0)
    acc_want, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
    pk = _packed_dev(w)
    # the launch plan's row blocks per wave: two from 432 row blocks on (four from 864 on with more than four
    # tokens), and for two there is no instance
    rpw = 1 if n // 16 < 432 else (4 if n // 16 >= 864 and m > 4 else 2)
    applies = m <= 8 and k != 6912 and rpw != 2
    try:
        if 5 <= m <= 8 and k <= 3200 and applies:  # the library's own choice
            st, out0, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
            assert st == 0 and bitlinear.last_kernel() == "bitlinear_solo_tok_kernel"
            _assert_bits_equal(host_bits(out0), want, "built-in choice")
        assert lib.bitlinear_set_tuning(8, 5, 0, 0) == 0  # not the one-to-four-token kernel
        assert lib.bitlinear_set_tuning(11, 1, 0, 0) == 0
        out, acc = bitlinear.bitlinear_forward_acc(dev_bf16(xb), pk, dev_bf16(ws_bits))
        assert (bitlinear.last_kernel() == "bitlinear_solo_tok_kernel") == applies
        st, out2, qd, sd = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
        assert st == 0 and (bitlinear.last_kernel() == "bitlinear_solo_tok_kernel") == applies
        st, out3, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0, with_ws=False)
        if not applies and st == 2:  # a block that only the two-kernel path takes needs the workspaces
            out3 = out2
        assert st == 0 or not applies
        st, out4, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 1)  # quantizer mode 1: the other kernels
        assert st == 0 and bitlinear.last_kernel() != "bitlinear_solo_tok_kernel"
        assert lib.bitlinear_set_tuning(11, 2, 0, 0) == 0
        st, out5, _, _ = _forward_raw(lib, xb, pk, ws_bits, m, n, k, 0)
        assert st == 0 and bitlinear.last_kernel() != "bitlinear_solo_tok_kernel"
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    for t, what in ((out, "forward + acc"), (out2, "forward"), (out3, "forward without workspaces"), (out5, "switched off")):
        _assert_bits_equal(host_bits(t), want, what)
    assert np.array_equal(qd.cpu().numpy(), q)
    assert np.array_equal(host_bits(sd), s_bits)
    q1, s1 = o.quant_input(xb, 1)
    _, want1 = o.bitlinear_int8xint2(q1, w, s1, ws_bits)
    _assert_bits_equal(host_bits(out4), want1, "mode 1")


@pytest.mark.parametrize("norm", [0, 1])
@pytest.mark.parametrize("coop", [1, 2])
@pytest.mark.parametrize("rpw", [0, 2, 3, 4])
@pytest.mark.parametrize("n,k,s_,upw", [(13824, 2560, 8, 5), (13824, 2560, 5, 8), (7008, 2560, 8, 5), (80, 320, 1, 5),
                                        (1040, 3200, 10, 5), (20480, 3200, 10, 5), (176, 2048, 4, 8)])
def test_solo_kernel_with_several_row_blocks_per_wave(n, k, s_, upw, rpw, coop, norm):
    """One token, waves that multiply their slice with two to four consecutive row
    blocks (rpw = 0: the library's own plan, which takes them for many row blocks):
    row-block counts that the group does not divide, three scale slots, a group
    larger than the waves per row block (falls back to one); accumulators and
    outputs bit for bit against the oracle chain, plain and behind the RMSNorm."""
    import ctypes

    lib = _lib.load_library()
    if norm and coop == 2:
        pytest.skip("the norm prologue always exchanges")
    rng = np.random.default_rng(n + 3 * k + rpw)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    xb = o.f32_to_bf16_bits(rng.standard_normal((1, k)).astype(np.float32) * 3.0)
    gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    pk, wsd = _packed_dev(w), dev_bf16(ws_bits)
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    try:
        if rpw:
            assert lib.bitlinear_set_tuning(8, 1, s_, upw) == 0
            assert lib.bitlinear_set_tuning(9, coop, rpw, 0) == 0
        if norm:
            want = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=False, residual_bits=None)
            out = torch.full((1, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            xd, gd = dev_bf16(xb), dev_bf16(gb)  # named: the device buffers must outlive the call
            st = lib.bitlinear_norm_forward_bf16(P(xd), P(gd), 1e-5, 0, P(pk), P(wsd), None, P(out), None, None, 1, n, k, 0, None)
            assert st == 0 and bitlinear.last_kernel() == "bitlinear_solo_kernel<norm>"
        else:
            q, s_bits = o.quant_input(xb, 0)
            acc_want, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
            out, acc = bitlinear.bitlinear_forward_acc(dev_bf16(xb), pk, wsd)
            assert bitlinear.last_kernel() == "bitlinear_solo_kernel"
            assert np.array_equal(acc.cpu().numpy(), acc_want)
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    _assert_bits_equal(host_bits(out), want, f"rpw={rpw}")


@pytest.mark.parametrize("res", [0, 1])
@pytest.mark.parametrize("m", [1, 3, 4, 8, 13, 16])
@pytest.mark.parametrize("n,k,s_,upw,rpw", [(2560, 2560, 8, 5, 1), (3840, 2560, 5, 8, 1), (13824, 2560, 8, 5, 2),
                                            (13824, 2560, 8, 5, 4), (13824, 2560, 0, 0, 0), (2560, 6912, 16, 7, 1),
                                            (2560, 6912, 0, 0, 0), (7008, 2560, 10, 4, 4), (48, 192, 1, 4, 1),
                                            (1040, 3200, 10, 5, 2), (80, 8192, 16, 8, 1)])
def test_product_kernel_without_staging(n, k, s_, upw, rpw, m, res):
    """gemv_i2_solo_kernel (int8 rows in, activation operands straight from the
    caller's rows, the code offset removed with a product against ones): forced
    launch shapes and the library's own choice ((0, 0, 0): many row blocks, or
    more than four tokens), one to four row blocks per wave with counts the group
    does not divide, three scale slots, every token count up to 16, with and
    without the residual epilogue (the two-kernel path of the norm-fused call);
    int32 accumulators and bf16 outputs bit for bit against the oracle."""
    import ctypes

    lib = _lib.load_library()
    w, a = _rand_case(n, k, m, seed=n + k + 7 * m)
    rng = np.random.default_rng(m + n)
    s_bits = o.f32_to_bf16_bits((0.5 + 30 * rng.random(m)).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    acc_want, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    pk, ad, sd, wsd = _packed_dev(w), dev_i8(a), dev_bf16(s_bits), dev_bf16(ws_bits)
    try:
        if s_:
            assert lib.bitlinear_set_tuning(10, 1, s_, upw) == 0
            assert lib.bitlinear_set_tuning(9, 0, rpw, 0) == 0
        out = bitlinear.bitnet_int8xint2_linear(ad, pk, sd, wsd)
        name = bitlinear.last_kernel()
        acc = bitlinear.bitnet_int8xint2_acc(ad, pk)
        assert bitlinear.last_kernel() == name
        if res:
            # the residual epilogue: RMSNorm + quantizer kernel, then this product (path 4 = never one kernel)
            assert lib.bitlinear_set_tuning(4, 0, 0, 0) == 0
            if s_:
                assert lib.bitlinear_set_tuning(10, 1, s_, upw) == 0
            xin = rng.standard_normal((m, k)).astype(np.float32) * 1.3
            xb = o.f32_to_bf16_bits(xin)
            gb = o.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32))
            rb_ = o.f32_to_bf16_bits(rng.standard_normal((m, n)).astype(np.float32))
            want_n = o.norm_bitlinear(xb, gb, 1e-5, w, ws_bits, glu=False, residual_bits=rb_)
            xd, gd, rd = dev_bf16(xb), dev_bf16(gb), dev_bf16(rb_)
            out_n = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            q_ws = torch.empty(m, k, dtype=torch.int8, device="cuda")
            s_ws = torch.empty(m, dtype=torch.bfloat16, device="cuda")
            P = lambda t: ctypes.c_void_p(t.data_ptr())
            st = lib.bitlinear_norm_forward_bf16(P(xd), P(gd), 1e-5, 0, P(pk), P(wsd), P(rd), P(out_n), P(q_ws), P(s_ws), m, n, k, 0, None)
            name_n = bitlinear.last_kernel()
            assert st == 0
        torch.cuda.synchronize()
    finally:
        lib.bitlinear_set_tuning(0, 0, 0, 0)
    if s_ or n // 16 >= 432 or m > 4:
        assert name == "gemv_i2_solo_kernel"
    assert np.array_equal(acc.cpu().numpy(), acc_want)
    _assert_bits_equal(host_bits(out), want, f"product {name}")
    if res:
        if s_:
            assert name_n == "gemv_i2_solo_kernel"
        _assert_bits_equal(host_bits(out_n), want_n, f"norm + product with residual {name_n}")


def test_matrix_pipe_probe_runs_and_reports_its_operations():
    """bitlinear_probe_mfma_i8 (the bench's ceiling leg): both operand modes
    launch, report 32 MFMAs of 32 x 32 x 32 per iteration for three waves on
    every SIMD, and refuse bad arguments."""
    import ctypes

    lib = _lib.load_library()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for mode in (0, 1):
        ops = ctypes.c_longlong(0)
        assert lib.bitlinear_probe_mfma_i8(mode, 10, None, ctypes.byref(ops), None) == 0
        torch.cuda.synchronize()
        assert ops.value == 2 * 32 ** 3 * 32 * 10 * 4 * 3 * cus
    assert lib.bitlinear_probe_mfma_i8(2, 10, None, None, None) == 4
    assert lib.bitlinear_probe_mfma_i8(0, 0, None, None, None) == 4


def test_quantizer_row_sums_and_the_identity_repack():
    """bitlinear_quant_absmax_rowsum: q and s as the plain quantizer, rowsum[m] =
    sum_k q[m, k]; bitlinear_repack: the converted weight is byte-identical to
    what the reference packer wrote, and the product on it equals the product on
    the original."""
    import ctypes

    lib = _lib.load_library()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    for m, k, mode in ((1, 2560, 0), (5, 6912, 0), (3, 27648, 1), (16, 64, 0), (2, 8, 1)):
        rng = np.random.default_rng(m * 7 + k)
        xb = o.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32) * 3.0)
        x = dev_bf16(xb)
        q = torch.empty(m, k, dtype=torch.int8, device="cuda")
        s = torch.empty(m, dtype=torch.bfloat16, device="cuda")
        rs = torch.full((m,), 12345, dtype=torch.int32, device="cuda")
        assert lib.bitlinear_quant_absmax_rowsum(P(x), P(q), P(s), P(rs), m, k, mode, None) == 0
        torch.cuda.synchronize()
        wq, wsb = o.quant_input(xb, mode)
        assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(host_bits(s), wsb)
        assert np.array_equal(rs.cpu().numpy(), wq.astype(np.int64).sum(axis=1).astype(np.int32))
    n, k = 3840, 2560
    w, a = _rand_case(n, k, 2, seed=4)
    pk = _packed_dev(w)
    assert lib.bitlinear_repacked_size(n, k) == pk.numel()
    conv = torch.zeros_like(pk)
    assert lib.bitlinear_repack(P(pk), P(conv), n, k, None) == 0
    assert lib.bitlinear_repack(P(pk), P(pk), n, k, None) == 0  # in place
    torch.cuda.synchronize()
    assert torch.equal(conv, pk)
    assert torch.equal(bitlinear.bitnet_int8xint2_acc(dev_i8(a), conv), bitlinear.bitnet_int8xint2_acc(dev_i8(a), pk))


def test_3d_input_and_out_argument():
    n, k = 2560, 2560
    w, a = _rand_case(n, k, 6, seed=3)
    a3 = a.reshape(2, 3, k)
    s_bits = o.f32_to_bf16_bits(np.linspace(1.0, 40.0, 6).astype(np.float32))
    ws_bits = o.f32_to_bf16_bits(np.array([0.016, 0, 0, 0], dtype=np.float32))
    out = torch.full((2, 3, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    ret = bitlinear.bitnet_int8xint2_linear(dev_i8(a3), _packed_dev(w), dev_bf16(s_bits).reshape(2, 3, 1), dev_bf16(ws_bits), out=out)
    assert ret is out and out.shape == (2, 3, n)
    _, want = o.bitlinear_int8xint2(a, w, s_bits, ws_bits)
    _assert_bits_equal(host_bits(out).reshape(6, n), want, "3d")


def test_empty_batch_returns_empty_outputs():
    """No token rows (a [0, K] activation): outputs of the right shape, no launch, no error."""
    n, k = 2560, 2560
    pk = _packed_dev(np.zeros((n, k), dtype=np.int8))
    ws = torch.ones(4, dtype=torch.bfloat16, device="cuda")
    a = torch.empty(0, k, dtype=torch.int8, device="cuda")
    s = torch.empty(0, 1, dtype=torch.bfloat16, device="cuda")
    assert bitlinear.bitnet_int8xint2_linear(a, pk, s, ws).shape == (0, n)
    assert bitlinear.bitnet_int8xint2_acc(a, pk).shape == (0, n)
    x = torch.empty(2, 0, k, dtype=torch.bfloat16, device="cuda")
    q, sc = bitlinear.quant_input(x)
    assert q.shape == (2, 0, k) and sc.shape == (2, 0, 1)
    mod = bitlinear.BitLinearKernel(k, n).cuda()
    assert mod(x).shape == (2, 0, n)


def test_unsupported_shape_reports_status_and_launches_nothing():
    lib = _lib.load_library()
    a = torch.zeros(1, 2560, dtype=torch.int8, device="cuda")
    wbad = torch.zeros(100, 640, dtype=torch.int8, device="cuda")  # N = 100
    s = torch.ones(1, dtype=torch.bfloat16, device="cuda")
    ws = torch.ones(4, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.BitLinearLibraryError):
        bitlinear.bitnet_int8xint2_linear(a, wbad, s, ws)
    assert lib.bitlinear_last_status() == 1
    with pytest.raises(ValueError):
        bitlinear.bitnet_int8xint2_linear(a.cpu(), wbad, s, ws)


def test_runs_on_a_side_stream_and_in_a_graph():
    """The reference call sits inside a captured graph (gpu/generate.py:181-203):
    no allocation, no sync, launches on the given stream only."""
    n, k = 2560, 2560
    w, a = _rand_case(n, k, 1, seed=21)
    pk, ad = _packed_dev(w), dev_i8(a)
    s = dev_bf16(o.f32_to_bf16_bits(np.array([7.0], dtype=np.float32)))
    ws_bits = o.f32_to_bf16_bits(np.array([0.02, 0, 0, 0], dtype=np.float32))
    wsd = dev_bf16(ws_bits)
    _, want = o.bitlinear_int8xint2(a, w, o.f32_to_bf16_bits(np.array([7.0], dtype=np.float32)), ws_bits)
    out = torch.zeros(1, n, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        bitlinear.bitnet_int8xint2_linear(ad, pk, s, wsd, out=out)
    side.synchronize()
    _assert_bits_equal(host_bits(out), want, "side stream")
    out.zero_()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        bitlinear.bitnet_int8xint2_linear(ad, pk, s, wsd, out=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        _assert_bits_equal(host_bits(out), want, "graph replay")


def test_kernel_test_harness_reports_the_reference_lines():
    """bitnet_amd.kernel_test mirrors gpu/test.py:31-86: per shape a known-answer line and a timing line."""
    from bitnet_amd import kernel_test

    lines = []
    res = kernel_test.check_and_time(shapes=kernel_test.REFERENCE_SHAPES[:2] + ((4800, 3200),), iters=5, out=lines.append)
    assert [r["equal"] for r in res] == [True, True, True]
    assert lines[0] == "custom == np True" and lines[1].startswith("Shape(2560, 2560), W2A8: ")
    assert "torch BF16: " in lines[1] and len(lines) == 6
    assert all(r["w2a8_graph_us"] > 0 and r["bf16_graph_us"] > 0 for r in res)
    assert len(kernel_test.REFERENCE_SHAPES) == 8


def test_flag_round_trip_probe_completes_and_checks_its_arguments():
    """bitlinear_probe_flag_roundtrip (the bench's hand-over leg): both workgroups see every round, on the same
    XCD and across XCDs; bad arguments are refused before any launch."""
    import ctypes

    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    lib = _lib.load_library()
    dev = torch.device("cuda")
    flags = torch.zeros(128, dtype=torch.int32, device=dev)
    gave_up = torch.zeros(1, dtype=torch.int32, device=dev)
    for wa, wb in ((0, 8), (0, 1), (5, 2)):
        flags.zero_()
        assert lib.bitlinear_probe_flag_roundtrip(P(flags), wa, wb, 300, P(gave_up), None) == 0
        torch.cuda.synchronize()
        assert int(gave_up[0]) == 0
        assert int(flags[0]) == 300 and int(flags[64]) == 300  # both sides reached the last round
    assert lib.bitlinear_probe_flag_roundtrip(P(flags), 3, 3, 10, P(gave_up), None) == 4
    assert lib.bitlinear_probe_flag_roundtrip(P(flags), 0, 1, 0, P(gave_up), None) == 4
    assert lib.bitlinear_probe_flag_roundtrip(None, 0, 1, 10, P(gave_up), None) == 2
