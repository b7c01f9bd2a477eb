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
    assert b"capture" in lib.bitlinear_status_string(6)


def test_static_scratch_forward_at_the_exact_limit():
    """M * K = 16 MiB - 32 KiB = 16744448 elements (511 rows of 32768) is the largest block the scratch holds: it
    runs, bit-equal to the workspace entry; one row more is refused before anything is launched."""
    lib = _lib.load_library()
    m, n, k = 511, 16, 32768
    assert m * k == (16 << 20) - 2 * 16384
    rng = np.random.default_rng(9)
    w = rng.integers(-1, 2, size=(n, k), dtype=np.int8)
    pk = pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w)).cuda()
    ws = dev_bf16(o.f32_to_bf16_bits(np.array([0.02, 0, 0, 0], dtype=np.float32)))
    x = dev_bf16(o.f32_to_bf16_bits(rng.standard_normal((m + 1, k)).astype(np.float32)))
    out_s, out_w = _both(lib, x, pk, ws, m, n, k)
    assert torch.equal(out_s.view(torch.int16), out_w.view(torch.int16))
    assert not torch.isnan(out_s.float()).any()
    out = torch.zeros(m + 1, n, dtype=torch.bfloat16, device="cuda")
    assert lib.bitlinear_forward_bf16_static(_P(x), _P(pk), _P(out), _P(ws), m + 1, n, k, 0, None) == 5


def test_first_static_call_on_a_device_under_capture_says_so():
    """In a fresh process whose first call of the entry sits inside a stream capture, the call launches nothing and
    returns the status of its own (6); after one call outside a capture, the captured call works."""
    import subprocess
    import sys
    code = r"""
import ctypes, torch
from bitnet_amd import _lib
lib = _lib.load_library()
P = lambda t: ctypes.c_void_p(t.data_ptr())
m, n, k = 4, 16, 256
x = torch.randn(m, k, device="cuda").bfloat16()
pk = torch.zeros(n // 4, k, dtype=torch.int8, device="cuda")
ws = torch.ones(4, device="cuda").bfloat16()
out = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
torch.cuda.synchronize()
g = torch.cuda.CUDAGraph()
with torch.cuda.graph(g):
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    first = lib.bitlinear_forward_bf16_static(P(x), P(pk), P(out), P(ws), m, n, k, 0, sp)
    torch.zeros(1, device="cuda")
torch.cuda.synchronize()
eager = lib.bitlinear_forward_bf16_static(P(x), P(pk), P(out), P(ws), m, n, k, 0, None)
torch.cuda.synchronize()
g2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g2):
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    later = lib.bitlinear_forward_bf16_static(P(x), P(pk), P(out), P(ws), m, n, k, 0, sp)
g2.replay()
torch.cuda.synchronize()
print("STATUS", first, eager, later)
"""
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "STATUS 6 0 0" in r.stdout, r.stdout + r.stderr[-2000:]
