"""The allocation-free forward entry (bitlinear_forward_bf16_static): called
through the C ABI, compared bit for bit with bitlinear_forward_bf16 (whose
workspaces the caller allocates), on calls in a row that share the library's
static scratch, each second call with a smaller input than the first."""
import ctypes

import numpy as np
import pytest
import torch

from bitnet_amd import _lib, pack_weight
from oracle import bitlinear_oracle as o
from tests.gpu_util import dev_bf16, host_bits

pytestmark = pytest.mark.gpu


def _P(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, x, pk, ws, m, n, k, mode=0):
    out_s = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    st = lib.bitlinear_forward_bf16_static(_P(x), _P(pk), _P(out_s), _P(ws), m, n, k, mode, None)
    assert st == 0, lib.bitlinear_status_string(st)
    torch.cuda.synchronize()
    out_w = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    q = torch.empty(m, k, dtype=torch.int8, device="cuda")
    s = torch.empty(m, dtype=torch.bfloat16, device="cuda")
    st = lib.bitlinear_forward_bf16(_P(x), _P(pk), _P(out_w), _P(ws), _P(q), _P(s), m, n, k, mode, None)
    assert st == 0, lib.bitlinear_status_string(st)
    torch.cuda.synchronize()
    return out_s, out_w


@pytest.mark.parametrize("n,k,m_first,m_second", [(3840, 2560, 512, 24), (2560, 6912, 2048, 7), (2560, 2560, 16, 1),
                                                  (13824, 2560, 130, 129), (1040, 3200, 40, 3)])
def test_static_scratch_forward_equals_workspace_forward(n, k, m_first, m_second):
    assert torch.cuda.is_available()
    lib = _lib.load_library()
    rng = np.random.default_rng(n + k + m_first)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    pk = pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w)).cuda()
    ws_bits = o.f32_to_bf16_bits(np.array([0.0161, 0.0247, 0.0093, 0.0], dtype=np.float32))
    ws = dev_bf16(ws_bits)
    for i, m in enumerate((m_first, m_second)):  # the second call finds the first call's rows in the scratch
        x_np = rng.standard_normal((m, k)).astype(np.float32)
        x_np[m // 2, ::9] *= 20.0
        xb = o.f32_to_bf16_bits(x_np)
        x = dev_bf16(xb)
        out_s, out_w = _both(lib, x, pk, ws, m, n, k)
        assert np.array_equal(host_bits(out_s), host_bits(out_w)), f"call {i} (M = {m})"
        if m <= 130:  # and against the oracle, where the CPU product is quick
            q, s_bits = o.quant_input(xb, 0)
            _, want = o.bitlinear_int8xint2(q, w, s_bits, ws_bits)
            assert np.array_equal(host_bits(out_s), want), f"call {i} (M = {m}) against the oracle"


def test_static_scratch_forward_in_a_graph_and_size_limit():
    lib = _lib.load_library()
    n, k, m = 2560, 2560, 64
    rng = np.random.default_rng(5)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    pk = pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w)).cuda()
    ws = dev_bf16(o.f32_to_bf16_bits(np.array([0.02, 0, 0, 0], dtype=np.float32)))
    x = dev_bf16(o.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32)))
    out_s, out_w = _both(lib, x, pk, ws, m, n, k)  # first call on the device: outside any capture
    assert torch.equal(out_s.view(torch.int16), out_w.view(torch.int16))
    out_g = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.bitlinear_forward_bf16_static(_P(x), _P(pk), _P(out_g), _P(ws), m, n, k, 0, sp) == 0
    for _ in range(3):
        out_g.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g.view(torch.int16), out_w.view(torch.int16))
    # beyond the scratch: refused before anything is launched
    assert lib.bitlinear_forward_bf16_static(_P(x), _P(pk), _P(out_g), _P(ws), 16385, n, 64, 0, None) == 5
    assert lib.bitlinear_forward_bf16_static(_P(x), _P(pk), _P(out_g), _P(ws), 4096, n, 4160, 0, None) == 5
    assert b"static scratch" in lib.bitlinear_status_string(5)
