"""Pins the oracle's floating-point pieces (bf16 rounding, epilogue,
activation quantizer, weight ternarisation) against torch's own CPU
routines evaluating the reference's expressions."""
import numpy as np
import torch

from oracle import bitlinear_oracle as o


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def test_bf16_rounding_matches_torch_cast():
    rng = np.random.default_rng(0)
    x = np.concatenate(
        [
            rng.standard_normal(20000).astype(np.float32) * np.float32(1000.0),
            rng.standard_normal(20000).astype(np.float32) * np.float32(1e-3),
            np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40, -1e-40, 65280.0], dtype=np.float32),
            # exact ties between two bf16 neighbours
            (np.arange(1, 300, dtype=np.uint32) << 16 | 0x8000).view(np.float32),
        ]
    )
    assert np.array_equal(o.f32_to_bf16_bits(x), _bits(torch.from_numpy(x).to(torch.bfloat16)))
    b = o.f32_to_bf16_bits(x)
    assert np.array_equal(o.bf16_bits_to_f32(b), _bf16(b).float().numpy())


def test_epilogue_unit_scales_is_bf16_of_acc():
    # the reference's own known-answer case: s = 1, ws = 1  (gpu/test.py:55-61)
    rng = np.random.default_rng(1)
    acc = rng.integers(-300000, 300000, size=(2, 64)).astype(np.int32)
    one = o.f32_to_bf16_bits(np.ones(2, dtype=np.float32))
    got = o.epilogue_bf16(acc, one, one, o.ws_slot(64, 1))
    assert np.array_equal(got, _bits(torch.from_numpy(acc).to(torch.bfloat16)))


def test_epilogue_matches_torch_fp32_ops():
    rng = np.random.default_rng(2)
    acc = rng.integers(-200000, 200000, size=(3, 48)).astype(np.int32)
    s = o.f32_to_bf16_bits((rng.random(3) * 50 + 1).astype(np.float32))
    ws = o.f32_to_bf16_bits((rng.random(3) * 0.05 + 0.001).astype(np.float32))
    slot = o.ws_slot(48, 3)
    got = o.epilogue_bf16(acc, s, ws, slot)
    t = torch.from_numpy(acc).float() / _bf16(s).float()[:, None] * _bf16(ws).float()[torch.from_numpy(slot)][None, :]
    assert np.array_equal(got, _bits(t.to(torch.bfloat16)))


def _torch_quant_eager(x: torch.Tensor):
    # gpu/model.py:69-71 evaluated by torch eager
    s = 127 / x.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    return (x * s).round().clamp(-128, 127).to(torch.int8), s


def test_quant_mode1_is_torch_eager_on_bf16():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 2560)).astype(np.float32)
    x[1] *= 1e-7  # exercises the 1e-5 clamp
    x[2] *= 300.0
    x[3, ::7] *= 20.0
    x[4] = 0.0
    xb = o.f32_to_bf16_bits(x)
    q, s = o.quant_input(xb, o.QUANT_EAGER_BF16)
    tq, ts = _torch_quant_eager(_bf16(xb))
    assert ts.dtype == torch.bfloat16
    assert np.array_equal(s, _bits(ts).reshape(-1))
    assert np.array_equal(q, tq.numpy())


def test_quant_modes_match_committed_torch_vectors():
    """mode 0 == torch.compile (Inductor CPU), mode 1 == torch eager, on the
    vectors tests/golden/make_quant_fixture.py wrote."""
    import os

    fx = np.load(os.path.join(os.path.dirname(__file__), "golden", "quant_compiled_fixture.npz"))
    for K in (256, 2560):
        xb = fx[f"x_{K}"]
        for mode, tag in ((o.QUANT_COMPILED, "compiled"), (o.QUANT_EAGER_BF16, "eager")):
            q, s = o.quant_input(xb, mode)
            assert np.array_equal(s, fx[f"s_{tag}_{K}"]), (K, tag)
            assert np.array_equal(q, fx[f"q_{tag}_{K}"]), (K, tag)
        # the two modes really differ on these vectors, so the check above can tell them apart
        assert not np.array_equal(fx[f"q_compiled_{K}"], fx[f"q_eager_{K}"])


def test_quant_saturation_and_half_even():
    # absmax element maps to +-127; ties round to even
    x = np.zeros((1, 8), dtype=np.float32)
    x[0] = [127.0, -127.0, 0.5, 1.5, 2.5, -0.5, -1.5, 126.5]
    for mode in (0, 1):
        q, s = o.quant_input(o.f32_to_bf16_bits(x), mode)
        assert o.bf16_bits_to_f32(s)[0] == 1.0
        # 126.5 is not a bf16 value (it becomes 126.5 -> 126.5 needs 9 bits): use what bf16 keeps
        xs = o.bf16_bits_to_f32(o.f32_to_bf16_bits(x))[0]
        assert list(q[0]) == [int(v) for v in np.clip(np.rint(xs), -128, 127)]
        assert list(q[0][:7]) == [127, -127, 0, 2, 2, 0, -2]


def test_fake_quant_matches_torch_eager():
    rng = np.random.default_rng(5)
    xb = o.f32_to_bf16_bits(rng.standard_normal((3, 256)).astype(np.float32))
    x = _bf16(xb)
    s = 127 / x.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    ref = (x * s).round().clamp(-128, 127) / s  # gpu/model.py:79-81, eager
    got = o.fake_quant_input(xb, o.QUANT_EAGER_BF16)
    assert np.array_equal(o.f32_to_bf16_bits(got), _bits(ref))


def test_quant_weight_int8_matches_torch_eager():
    rng = np.random.default_rng(6)
    w = (rng.standard_normal((64, 256)) * 0.02).astype(np.float32)
    wt, sc = o.quant_weight_int8(w)
    t = torch.from_numpy(w)
    s = 1.0 / t.abs().mean().clamp_(min=1e-5)  # gpu/convert_checkpoint.py:24-26, eager
    tw = (t * s).round().clamp(-1, 1).to(torch.int8)
    assert np.array_equal(wt, tw.numpy())
    assert np.array_equal(sc, _bits((1.0 / s).to(torch.bfloat16).reshape(1)))
    assert set(np.unique(wt)) <= {-1, 0, 1}


def test_fused_scales_layout():
    rng = np.random.default_rng(7)
    parts = [(rng.standard_normal((r, 64)) * sd).astype(np.float32) for r, sd in [(32, 0.02), (16, 0.05), (16, 0.01)]]
    w, ws = o.fused_weight_and_scales(parts)
    assert w.shape == (64, 64) and ws.shape == (4,) and ws[3] == 0
    for j, p in enumerate(parts):
        assert ws[j] == o.quant_weight_int8(p)[1][0]


def test_glu_matches_torch_eager_and_norm_is_within_one_ulp_of_torch_fp32():
    rng = np.random.default_rng(8)
    x13 = o.f32_to_bf16_bits(rng.standard_normal((4, 512)).astype(np.float32))
    t = _bf16(x13)
    x1, x3 = t.chunk(2, -1)
    ref = torch.relu(x1) ** 2 * x3  # gpu/model.py:164-166, 195 evaluated by torch eager on bf16
    assert np.array_equal(o.squared_relu_glu_bf16(x13), _bits(ref))

    h = o.f32_to_bf16_bits((rng.standard_normal((5, 2560)) * np.array([[1], [30], [0.01], [1], [1]])).astype(np.float32))
    g = o.f32_to_bf16_bits((1.0 + 0.1 * rng.standard_normal(2560)).astype(np.float32))
    got = o.rmsnorm_bf16(h, g, 1e-5)
    hf = _bf16(h).float()
    want = (hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + 1e-5) * _bf16(g).float()).to(torch.bfloat16)
    a, b = got.astype(np.int32), _bits(want).astype(np.int32)
    assert np.max(np.abs(a - b)) <= 1 and np.mean(a != b) < 0.01
    # closed form: a constant row normalises to +-g (eps negligible)
    c = o.f32_to_bf16_bits(np.full((1, 256), -3.0, dtype=np.float32))
    g1 = o.f32_to_bf16_bits(np.linspace(0.5, 2.0, 256).astype(np.float32))
    assert np.array_equal(o.rmsnorm_bf16(c, g1, 0.0)[0], o.f32_to_bf16_bits(-o.bf16_bits_to_f32(g1)))

    r = o.f32_to_bf16_bits(rng.standard_normal(64).astype(np.float32))
    v = o.f32_to_bf16_bits(rng.standard_normal(64).astype(np.float32))
    assert np.array_equal(o.residual_add_bf16(r, v), _bits(_bf16(r) + _bf16(v)))
