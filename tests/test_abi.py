"""The C-ABI library loads without a GPU and exports every function the
header declares; host-only entry points behave as documented."""
import ctypes
import os
import re

import pytest

from bitnet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    names = []
    for header in ("bitlinear_hip.h", "bitnet_decoder_ops.h", "bitlinear_probes.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(bit(?:linear|net)_[a-z0-9_]+)\s*\(", text)
    return names


def test_header_declares_the_drop_in_symbol():
    names = _declared_functions()
    assert "bitlinear_int8xint2" in names
    assert len(names) == len(set(names)) >= 9


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built (run python -m bitnet_amd.build)")
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(raw, name), name
    # and the binding table covers exactly the header
    assert set(_lib.SIGNATURES) == set(_declared_functions())


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(_lib.BitLinearLibraryError):
        _lib.load_library(str(tmp_path / "nope.so"))


def test_host_only_entry_points():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built")
    lib = _lib.load_library()
    # shape table of the reference dispatcher (gpu/bitnet_kernels/bitnet_kernels.cu:4-33)
    table = {(3840, 2560): 3, (2560, 2560): 1, (13824, 2560): 2, (2560, 6912): 1, (4800, 3200): 6,
             (3200, 3200): 1, (20480, 3200): 2, (3200, 10240): 1, (5120, 27648): 1, (55296, 5120): 1}
    for (n, k), v in table.items():
        assert lib.bitlinear_ws_num(n, k) == v
    assert lib.bitlinear_ws_num(1024, 4096) == 1
    # the load-time converter is the identity: the converted weight has the reference's size
    assert lib.bitlinear_repacked_size(2560, 6912) == 2560 * 6912 // 4
    assert lib.bitlinear_repacked_size(100, 2560) == 0 and lib.bitlinear_repacked_size(2560, 100) == 0
    assert lib.bitlinear_repack(None, None, 100, 2560, None) == 1 and lib.bitlinear_repack(None, None, 2560, 2560, None) == 2
    assert lib.bitlinear_quant_absmax_rowsum(None, None, None, None, 1, 2560, 0, None) == 2
    assert lib.bitlinear_status_string(0) == b"ok"
    assert b"shape" in lib.bitlinear_status_string(1)
    assert lib.bitlinear_set_tuning(2, 8, 4, 0) == 0
    assert lib.bitlinear_set_tuning(2, 17, 4, 0) != 0
    assert lib.bitlinear_set_tuning(2, 8, 3, 0) != 0
    assert lib.bitlinear_set_tuning(1, 4, 0, 0) != 0  # no kernel 1
    assert lib.bitlinear_set_tuning(3, 1, 1, 0) != 0
    assert lib.bitlinear_set_tuning(3, 2, 8, 5) == 0
    assert lib.bitlinear_set_tuning(3, 4, 5, 4) != 0
    assert lib.bitlinear_set_tuning(5, 1, 0, 0) == 0
    assert lib.bitlinear_set_tuning(6, 1, 0, 0) == 0
    assert lib.bitlinear_set_tuning(6, 3, 0, 0) != 0
    assert lib.bitlinear_set_tuning(7, 1, 0, 0) == 0
    assert lib.bitlinear_set_tuning(7, 3, 0, 0) != 0
    assert lib.bitlinear_set_tuning(8, 1, 8, 5) == 0 and lib.bitlinear_set_tuning(8, 5, 0, 0) == 0
    assert lib.bitlinear_set_tuning(8, 2, 9, 5) != 0 and lib.bitlinear_set_tuning(8, 1, 8, 6) != 0
    assert lib.bitlinear_set_tuning(9, 2, 0, 0) == 0 and lib.bitlinear_set_tuning(9, 3, 0, 0) != 0
    assert lib.bitlinear_set_tuning(9, 1, 4, 0) == 0 and lib.bitlinear_set_tuning(9, 1, 5, 0) != 0
    assert lib.bitlinear_set_tuning(10, 1, 8, 5) == 0 and lib.bitlinear_set_tuning(10, 2, 0, 0) == 0
    assert lib.bitlinear_set_tuning(10, 1, 8, 6) != 0 and lib.bitlinear_set_tuning(10, 3, 0, 0) != 0
    assert lib.bitlinear_set_tuning(11, 1, 0, 0) == 0 and lib.bitlinear_set_tuning(11, 2, 0, 0) == 0
    assert lib.bitlinear_set_tuning(11, 3, 0, 0) != 0 and lib.bitlinear_set_tuning(12, 0, 0, 0) != 0
    assert lib.bitlinear_set_tuning(0, 0, 0, 0) == 0


def test_argument_checks_need_no_gpu(capfd):
    """Shape and NULL checks run before any HIP call."""
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built")
    lib = _lib.load_library()
    # N not a multiple of 16: the reference's message, nothing launched
    lib.bitlinear_int8xint2(None, None, None, None, None, 1, 100, 2560, None)
    assert lib.bitlinear_last_status() == 1
    assert "required ladder gemm kernel: M 1, N 100, K 2560" in capfd.readouterr().out
    lib.bitlinear_int8xint2(None, None, None, None, None, 1, 2560, 2560, None)
    assert lib.bitlinear_last_status() == 2
    assert lib.bitlinear_quant_absmax(None, None, None, 1, 2560, 0, None) == 2
    assert lib.bitlinear_quant_absmax(None, None, None, 1, 2563, 0, None) == 1
    assert lib.bitlinear_int8xint2_acc_i32(None, None, None, None, None, None, 1, 2560, 100, None) == 1
    # the allocation-free forward: sizes beyond its static scratch, then nulls, before any HIP call
    assert lib.bitlinear_forward_bf16_static(None, None, None, None, 16385, 2560, 64, 0, None) == 5
    assert lib.bitlinear_forward_bf16_static(None, None, None, None, 4096, 2560, 4160, 0, None) == 5
    assert lib.bitlinear_forward_bf16_static(None, None, None, None, 2048, 2560, 6912, 0, None) == 2


def test_decoder_entry_argument_checks_need_no_gpu():
    """The decoder-side entry points refuse bad shapes (1) and null pointers (2)
    before any HIP call."""
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built")
    lib = _lib.load_library()
    # bitnet_attn_decode: head_dim, group size, split count, nulls
    assert lib.bitnet_attn_decode(None, None, None, None, None, None, None, None, None, 1, 1, 64, 4, 2, 64, None) == 1
    assert lib.bitnet_attn_decode(None, None, None, None, None, None, None, None, None, 1, 1, 64, 6, 2, 128, None) == 1
    assert lib.bitnet_attn_decode(None, None, None, None, None, None, None, None, None, 17, 1, 64, 4, 2, 128, None) == 1
    assert lib.bitnet_attn_decode(None, None, None, None, None, None, None, None, None, 1, 1, 64, 4, 2, 128, None) == 2
    assert lib.bitnet_attn_decode_rows(None, None, None, None, None, None, None, None, None, None, 1, 1, 64, 4, 2, 128, None) == 2
    assert lib.bitnet_attn_decode_workspace_floats(1, 20, 5, 8) == 1 * 5 * 8 * 4 * 130 * 2 + 5 + 2
    assert lib.bitnet_attn_decode_error_index(1, 20, 5, 8) == 1 * 5 * 8 * 4 * 130 * 2 + 5
    assert lib.bitnet_attn_decode_error_index(1, 20, 6, 8) == -1
    assert lib.bitnet_attn_decode_set_spin_limit(5) == 0 and lib.bitnet_attn_decode_set_spin_limit(-1) == 0
    assert len(lib.bitlinear_last_kernel()) > 0  # "none", or whatever an earlier test of this process launched
    assert lib.bitnet_attn_decode_workspace_floats(1, 20, 6, 8) == -1
    # prompt side: start + T beyond the cache, head_dim, nulls
    assert lib.bitnet_attn_prefill(None, None, None, None, 1, 40, 64, 30, 4, 2, 128, None) == 1
    assert lib.bitnet_attn_prefill(None, None, None, None, 1, 40, 64, 0, 4, 2, 64, None) == 1
    assert lib.bitnet_attn_prefill(None, None, None, None, 1, 40, 64, 0, 4, 2, 128, None) == 2
    assert lib.bitnet_rope_cache_tokens(None, None, None, None, None, None, None, 1, 0, 64, 4, 2, 128, None) == 1
    assert lib.bitnet_rope_cache_tokens(None, None, None, None, None, None, None, 1, 8, 64, 4, 2, 128, None) == 2
    assert lib.bitnet_decode_step_begin(None, None, None, None, None, None, None, 1, 100, 250, 64, 128, None) == 1  # dim % 8
    assert lib.bitnet_decode_step_begin(None, None, None, None, None, None, None, 1, 100, 256, 64, 128, None) == 2
